// HBM-bound kernels of the llama path for gfx950: RMSNorm, RoPE, SwiGLU,
// residual add, embedding gather / scatter-add; forward and adjoint.
//
// All of them stream 16-byte vectors per lane, keep a row in registers where a
// reduction is needed, reduce across the 64-lane wavefront with DPP shuffles
// and compute in fp32 whatever the storage type is.
#include <mutex>

#include "emi_device.h"

namespace emi {

// ---------------------------------------------------------------------------
// RMSNorm (test/llama.py:6-10): y = gamma * x * rsqrt(mean(x^2) + eps)
// TPR threads cooperate on one row (64 = one wavefront per row, four rows per
// 256-thread block; 256 = one block per row); each thread keeps up to NCH
// chunks of 8 elements in registers so x is read from HBM exactly once.
// ---------------------------------------------------------------------------

template <int TPR> __device__ __forceinline__ void row_reduce2(float& a, float& b, float (*red)[4][2], int it) {
  a = wave_sum(a);
  b = wave_sum(b);
  if constexpr (TPR == 256) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float(*buf)[2] = red[it & 1];
    if (lane == 0) {
      buf[wave][0] = a;
      buf[wave][1] = b;
    }
    __syncthreads();
    a = buf[0][0] + buf[1][0] + buf[2][0] + buf[3][0];
    b = buf[0][1] + buf[1][1] + buf[2][1] + buf[3][1];
  }
}

template <typename T, int TPR, int NCH>
__global__ __launch_bounds__(256) void rmsnorm_fwd_kernel(const T* __restrict__ x, const T* __restrict__ gamma,
                                                          T* __restrict__ y, int64_t rows, int dim, float eps) {
  // NCH groups of 8 elements per thread, held as 16-byte pieces (8 bf16 or 4 floats): consecutive lanes cover
  // consecutive 16 bytes, the access shape the streaming loads and stores want.
  constexpr int RPB = 256 / TPR, N = Chunk<T>::N, NC = NCH * 8 / N;
  __shared__ float red[2][4][2];
  const int tir = threadIdx.x % TPR;
  const int rib = threadIdx.x / TPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + rib;
  const bool active = row < rows;
  const int nchunk = dim / N;
  const T* xr = x + row * dim;
  float v[NC][N];
  float ss = 0.f, dummy = 0.f;
#pragma unroll
  for (int j = 0; j < NC; j++) {
    const int c = tir + j * TPR;
    if (active && c < nchunk) {
      Chunk<T>::load(xr + c * N, v[j]);
#pragma unroll
      for (int e = 0; e < N; e++) ss += v[j][e] * v[j][e];
    }
  }
  row_reduce2<TPR>(ss, dummy, red, 0);
  const float r = 1.0f / sqrtf(ss / (float)dim + eps);
  T* yr = y + row * dim;
#pragma unroll
  for (int j = 0; j < NC; j++) {
    const int c = tir + j * TPR;
    if (active && c < nchunk) {
      float g[N], o[N];
      ChunkCached<T>::load(gamma + c * N, g);
#pragma unroll
      for (int e = 0; e < N; e++) o[e] = g[e] * v[j][e] * r;
      Chunk<T>::store(yr + c * N, o);
    }
  }
}

// Sums of NV values over the TPR threads of a row with one barrier.
template <int TPR, int NV> __device__ __forceinline__ void row_reduce_n(float (&v)[NV], float (*red)[4][NV], int it) {
#pragma unroll
  for (int i = 0; i < NV; i++) v[i] = wave_sum(v[i]);
  if constexpr (TPR == 256) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float(*buf)[NV] = red[it & 1];
    if (lane == 0) {
#pragma unroll
      for (int i = 0; i < NV; i++) buf[wave][i] = v[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NV; i++) v[i] = buf[0][i] + buf[1][i] + buf[2][i] + buf[3][i];
  }
}

// Adjoint.  Blocks walk rows with a grid stride, NR rows per step, and keep this
// thread's share of dgamma in registers; partial[blockIdx*RPB + rib][dim] is reduced
// by colsum_kernel.  dx = [dx_add +] r*g - x * r^3 * mean(g*x), g = dy*gamma.
template <typename T, int TPR, int NCH, int NR>
__global__ __launch_bounds__(256) void rmsnorm_bwd_kernel(const T* __restrict__ x, const T* __restrict__ gamma,
                                                          const T* __restrict__ dy, const T* dx_add, T* dx,
                                                          float* __restrict__ partial, int64_t rows, int dim,
                                                          float eps) {
  // NCH groups of 8 elements per thread, held as 16-byte pieces (8 bf16 or 4 floats) so that consecutive lanes cover
  // consecutive 16 bytes (the access shape of the streaming loads and stores)
  constexpr int RPB = 256 / TPR, N = Chunk<T>::N, NC = NCH * 8 / N;
  __shared__ float red[2][4][2 * NR];
  const int tir = threadIdx.x % TPR;
  const int rib = threadIdx.x / TPR;
  const int nchunk = dim / N;
  float gm[NC][N], acc[NC][N];
#pragma unroll
  for (int j = 0; j < NC; j++) {
    const int c = tir + j * TPR;
#pragma unroll
    for (int e = 0; e < N; e++) acc[j][e] = 0.f, gm[j][e] = 0.f;
    if (c < nchunk) ChunkCached<T>::load(gamma + c * N, gm[j]);
  }
  const int64_t nstep = (rows + RPB * NR - 1) / (RPB * NR);   // steps of RPB*NR rows
  // Steps are software pipelined: the loads of the next step are issued before the
  // reduction (shuffles, LDS, barrier) of the current one, which keeps twice the
  // bytes in flight per block.
  typename Chunk<T>::Raw xn[NR][NC], gn[NR][NC];      // kept in storage format to save registers
  auto load_step = [&](int64_t sg) {
#pragma unroll
    for (int u = 0; u < NR; u++) {
      const int64_t row = (sg * NR + u) * RPB + rib;
#pragma unroll
      for (int j = 0; j < NC; j++) {
        const int c = tir + j * TPR;
        if (sg < nstep && row < rows && c < nchunk) {
          xn[u][j] = Chunk<T>::load_raw(x + row * dim + c * N);
          gn[u][j] = Chunk<T>::load_raw(dy + row * dim + c * N);
        } else {
          xn[u][j] = typename Chunk<T>::Raw{};
          gn[u][j] = typename Chunk<T>::Raw{};
        }
      }
    }
  };
  load_step(blockIdx.x);
  int it = 0;
  for (int64_t sg = blockIdx.x; sg < nstep; sg += gridDim.x, ++it) {
    typename Chunk<T>::Raw xc[NR][NC], gc[NR][NC];
    float red_v[2 * NR];
#pragma unroll
    for (int u = 0; u < NR; u++) {
      float ss = 0.f, gx = 0.f;
#pragma unroll
      for (int j = 0; j < NC; j++) {
        xc[u][j] = xn[u][j];
        gc[u][j] = gn[u][j];
        float xv[N], gv[N];
        Chunk<T>::unpack(xc[u][j], xv);
        Chunk<T>::unpack(gc[u][j], gv);
#pragma unroll
        for (int e = 0; e < N; e++) {
          ss += xv[e] * xv[e];
          gx += gv[e] * gm[j][e] * xv[e];
        }
      }
      red_v[2 * u] = ss;
      red_v[2 * u + 1] = gx;
    }
    load_step(sg + gridDim.x);
    row_reduce_n<TPR, 2 * NR>(red_v, red, it);
#pragma unroll
    for (int u = 0; u < NR; u++) {
      const int64_t row = (sg * NR + u) * RPB + rib;
      const bool active = row < rows;
      const float r = 1.0f / sqrtf(red_v[2 * u] / (float)dim + eps);
      const float coef = r * r * r * (red_v[2 * u + 1] / (float)dim);
#pragma unroll
      for (int j = 0; j < NC; j++) {
        const int c = tir + j * TPR;
        if (active && c < nchunk) {
          float xv[N], gv[N], o[N];
          Chunk<T>::unpack(xc[u][j], xv);
          Chunk<T>::unpack(gc[u][j], gv);
#pragma unroll
          for (int e = 0; e < N; e++) {
            acc[j][e] += gv[e] * xv[e] * r;
            o[e] = r * gv[e] * gm[j][e] - xv[e] * coef;
          }
          if (dx_add != nullptr) {
            float a[N];
            Chunk<T>::load(dx_add + row * dim + c * N, a);
#pragma unroll
            for (int e = 0; e < N; e++) o[e] += a[e];
          }
          Chunk<T>::store(dx + row * dim + c * N, o);
        }
      }
    }
  }
  if constexpr (RPB > 1) {
    // the rows-in-block of a narrow-row block add their partial sums in index order: one partial row per block
    __shared__ float comb[(RPB - 1) * TPR * NC * N];
    if (rib > 0) {
#pragma unroll
      for (int j = 0; j < NC; j++)
#pragma unroll
        for (int e = 0; e < N; e++) comb[(((rib - 1) * NC + j) * N + e) * TPR + tir] = acc[j][e];
    }
    __syncthreads();
    if (rib > 0) return;
#pragma unroll
    for (int r = 0; r < RPB - 1; r++)
#pragma unroll
      for (int j = 0; j < NC; j++)
#pragma unroll
        for (int e = 0; e < N; e++) acc[j][e] += comb[((r * NC + j) * N + e) * TPR + tir];
  }
  float* prow = partial + (int64_t)blockIdx.x * dim;
#pragma unroll
  for (int j = 0; j < NC; j++) {
    const int c = tir + j * TPR;
    if (c < nchunk) {
#pragma unroll
      for (int q = 0; q < N / 4; q++)
        *reinterpret_cast<float4*>(prow + c * N + 4 * q) = make_float4(acc[j][4 * q], acc[j][4 * q + 1], acc[j][4 * q + 2], acc[j][4 * q + 3]);
    }
  }
}

// Any dim (not a multiple of 8, or beyond the register budget): one block per
// row group, scalar accesses, x re-read from cache.
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_fwd_generic_kernel(const T* __restrict__ x, const T* __restrict__ gamma,
                                                                  T* __restrict__ y, int64_t rows, int64_t dim,
                                                                  float eps) {
  __shared__ float red[2][4][2];
  const int64_t row = blockIdx.x;
  const T* xr = x + row * dim;
  float ss = 0.f, dummy = 0.f;
  for (int64_t c = threadIdx.x; c < dim; c += 256) {
    const float v = to_f32(xr[c]);
    ss += v * v;
  }
  row_reduce2<256>(ss, dummy, red, 0);
  const float r = 1.0f / sqrtf(ss / (float)dim + eps);
  for (int64_t c = threadIdx.x; c < dim; c += 256) y[row * dim + c] = from_f32<T>(to_f32(gamma[c]) * to_f32(xr[c]) * r);
}

template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_bwd_generic_kernel(const T* __restrict__ x, const T* __restrict__ gamma,
                                                                  const T* __restrict__ dy, const T* dx_add, T* dx,
                                                                  float* __restrict__ partial, int64_t rows,
                                                                  int64_t dim, float eps) {
  __shared__ float red[2][4][2];
  float* prow = partial + (int64_t)blockIdx.x * dim;
  for (int64_t c = threadIdx.x; c < dim; c += 256) prow[c] = 0.f;
  int it = 0;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x, ++it) {
    float ss = 0.f, gx = 0.f;
    for (int64_t c = threadIdx.x; c < dim; c += 256) {
      const float xv = to_f32(x[row * dim + c]);
      ss += xv * xv;
      gx += to_f32(dy[row * dim + c]) * to_f32(gamma[c]) * xv;
    }
    row_reduce2<256>(ss, gx, red, it);
    const float r = 1.0f / sqrtf(ss / (float)dim + eps);
    const float coef = r * r * r * (gx / (float)dim);
    for (int64_t c = threadIdx.x; c < dim; c += 256) {
      const float xv = to_f32(x[row * dim + c]);
      const float gv = to_f32(dy[row * dim + c]);
      prow[c] += gv * xv * r;   // this thread owns column c of this block's partial row
      float o = r * gv * to_f32(gamma[c]) - xv * coef;
      if (dx_add != nullptr) o += to_f32(dx_add[row * dim + c]);
      dx[row * dim + c] = from_f32<T>(o);
    }
  }
}

// Column sums of partial[nparts][dim]: block (cb, rc) adds rows [CS_ROWS*rc, CS_ROWS*rc +
// CS_ROWS) of 64 columns into row rc of `out`.  1024 threads = 16 float4 columns x 64 row
// lanes (a wavefront reads 256 contiguous bytes of four rows), eight loads in flight per
// lane, so the 512 partial rows of the adjoint's grid are one round of loads.  The
// launcher applies it until one row is left (one pass for the grids the adjoint uses);
// the last pass writes type T.
constexpr int CS_ROWS = 512;
template <typename TO>
__global__ __launch_bounds__(1024) void colsum_kernel(const float* __restrict__ partial, int nparts, int64_t dim,
                                                      TO* __restrict__ out) {
  __shared__ float red[64][64 + 4];
  const int cq = threadIdx.x & 15, rl = threadIdx.x >> 4;
  const int64_t col = (int64_t)blockIdx.x * 64 + cq * 4;
  const int r0 = blockIdx.y * CS_ROWS;
  const int r1 = r0 + CS_ROWS < nparts ? r0 + CS_ROWS : nparts;
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  if ((dim & 3) == 0 && col + 4 <= dim) {
    float4 v[8];
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const int p = r0 + rl + 64 * u;
      v[u] = p < r1 ? *reinterpret_cast<const float4*>(partial + (int64_t)p * dim + col) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int u = 0; u < 8; u++) { s[0] += v[u].x; s[1] += v[u].y; s[2] += v[u].z; s[3] += v[u].w; }
  } else {
    for (int p = r0 + rl; p < r1; p += 64)
#pragma unroll
      for (int e = 0; e < 4; e++)
        if (col + e < dim) s[e] += partial[(int64_t)p * dim + col + e];
  }
#pragma unroll
  for (int e = 0; e < 4; e++) red[rl][cq * 4 + e] = s[e];
  __syncthreads();
  // 64 columns x 16 row groups of four, then the 16 partial sums of a column
  {
    const int c = threadIdx.x & 63, g = threadIdx.x >> 6;
    const float t = red[4 * g][c] + red[4 * g + 1][c] + red[4 * g + 2][c] + red[4 * g + 3][c];
    __syncthreads();
    red[g][c] = t;
  }
  __syncthreads();
  if (threadIdx.x < 64) {
    const int64_t c = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (c < dim) {
      float t = 0.f;
#pragma unroll
      for (int i = 0; i < 16; i++) t += red[i][threadIdx.x];
      out[(int64_t)blockIdx.y * dim + c] = from_f32<TO>(t);
    }
  }
}

// ---------------------------------------------------------------------------
// RoPE (test/llama.py:127-140,161-168): adjacent pairs, angle table in fp32.
// ---------------------------------------------------------------------------

__global__ void rope_table_kernel(float2* __restrict__ table, int64_t seq, int half, int head_dim, double theta,
                                  int64_t pos0) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= seq * half) return;
  const int64_t s = i / half;
  const int j = (int)(i % half);
  const double freq = 1.0 / pow(theta, (double)(2 * j) / (double)head_dim);
  const double ang = (double)(pos0 + s) * freq;
  table[i] = make_float2((float)cos(ang), (float)sin(ang));
}

// One block row of the grid per row of x (a sequence position of one sequence), a thread per 16-byte chunk (8 bf16 /
// 4 fp32 elements): the indices are 32-bit and the position is the block's.  (Two or more rows per thread, with
// their loads in flight together, measured slower: 75 -> 73 -> 64 % of peak for 2, 4, 8 rows in bf16.)
template <typename T>
__global__ __launch_bounds__(256) void rope_kernel(const T* x, const float2* __restrict__ table, T* y, int seq,
                                                   int row_elems, int head_dim, int inverse) {
  constexpr int V = ChunkCached<T>::N, NP = V / 2;
  const int col = (blockIdx.y * blockDim.x + threadIdx.x) * V;
  if (col >= row_elems) return;
  const int row = blockIdx.x, s = row % seq;
  const float4* tp = reinterpret_cast<const float4*>(table + (int64_t)s * (head_dim >> 1) + ((col % head_dim) >> 1));
  float4 t[NP / 2];                                          // two (cos, sin) entries each
#pragma unroll
  for (int q = 0; q < NP / 2; q++) t[q] = tp[q];
  float v[V], o[V];
  ChunkCached<T>::load(x + (int64_t)row * row_elems + col, v);              // (streaming accesses measured slower here)
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const float cs = (p & 1) ? t[p >> 1].z : t[p >> 1].x;
    const float sn = (p & 1) ? t[p >> 1].w : t[p >> 1].y;
    const float sp = inverse ? -sn : sn;
    o[2 * p] = cs * v[2 * p] - sp * v[2 * p + 1];
    o[2 * p + 1] = sp * v[2 * p] + cs * v[2 * p + 1];
  }
  ChunkCached<T>::store(y + (int64_t)row * row_elems + col, o);
}

template <typename T>
__global__ __launch_bounds__(256) void rope_pair_kernel(const T* x, const float2* __restrict__ table, T* y,
                                                        int64_t npairs, int seq, int row_elems, int head_dim,
                                                        int inverse) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= npairs) return;
  const int64_t e = i * 2;
  const int in_head = (int)(e % head_dim);
  const int s = (int)((e / row_elems) % seq);
  const float2 t = table[(int64_t)s * (head_dim >> 1) + (in_head >> 1)];
  const float sp = inverse ? -t.y : t.y;
  const float v0 = to_f32(x[e]), v1 = to_f32(x[e + 1]);
  y[e] = from_f32<T>(t.x * v0 - sp * v1);
  y[e + 1] = from_f32<T>(sp * v0 + t.x * v1);
}

// ---------------------------------------------------------------------------
// SwiGLU (test/llama.py:21-28,229-231) and elementwise add
// ---------------------------------------------------------------------------

__device__ __forceinline__ float sigmoidf(float a) { return emi_sigmoid(a); }

template <typename T>
__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                         T* __restrict__ g, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t nchunks = n >> 3;
  if (i < nchunks) {
    float av[8], bv[8], o[8];
    Vec8<T>::load(a + i * 8, av);
    Vec8<T>::load(b + i * 8, bv);
#pragma unroll
    for (int e = 0; e < 8; e++) o[e] = av[e] * sigmoidf(av[e]) * bv[e];
    Vec8<T>::store(g + i * 8, o);
  } else if (i - nchunks < (n & 7)) {
    const int64_t e = (nchunks << 3) + (i - nchunks);
    const float av = to_f32(a[e]);
    g[e] = from_f32<T>(av * sigmoidf(av) * to_f32(b[e]));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                         const T* __restrict__ dg, T* __restrict__ da,
                                                         T* __restrict__ db, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t nchunks = n >> 3;
  if (i < nchunks) {
    float av[8], bv[8], gv[8], oa[8], ob[8];
    Vec8<T>::load(a + i * 8, av);
    Vec8<T>::load(b + i * 8, bv);
    Vec8<T>::load(dg + i * 8, gv);
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float s = sigmoidf(av[e]);
      oa[e] = gv[e] * bv[e] * s * (1.0f + av[e] * (1.0f - s));
      ob[e] = gv[e] * av[e] * s;
    }
    Vec8<T>::store(da + i * 8, oa);
    Vec8<T>::store(db + i * 8, ob);
  } else if (i - nchunks < (n & 7)) {
    const int64_t e = (nchunks << 3) + (i - nchunks);
    const float av = to_f32(a[e]), bv = to_f32(b[e]), gv = to_f32(dg[e]);
    const float s = sigmoidf(av);
    da[e] = from_f32<T>(gv * bv * s * (1.0f + av * (1.0f - s)));
    db[e] = from_f32<T>(gv * av * s);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void add_kernel(const T* a, const T* b, T* y, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t nchunks = n >> 3;
  if (i < nchunks) {
    float av[8], bv[8];
    Vec8<T>::load(a + i * 8, av);
    Vec8<T>::load(b + i * 8, bv);
#pragma unroll
    for (int e = 0; e < 8; e++) av[e] += bv[e];
    Vec8<T>::store(y + i * 8, av);
  } else if (i - nchunks < (n & 7)) {
    const int64_t e = (nchunks << 3) + (i - nchunks);
    y[e] = from_f32<T>(to_f32(a[e]) + to_f32(b[e]));
  }
}

// ---------------------------------------------------------------------------
// Embedding gather and scatter-add
// ---------------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(256) void embedding_fwd_kernel(const int32_t* __restrict__ tokens,
                                                            const T* __restrict__ table, T* __restrict__ x,
                                                            int64_t n_tokens, int64_t vocab, int64_t dim) {
  const int64_t t = blockIdx.x;
  int64_t tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);   // clamp like XLA's gather
  for (int64_t c = threadIdx.x; c < dim; c += 256) x[t * dim + c] = table[tok * dim + c];
}

template <typename T>
__global__ __launch_bounds__(256) void embedding_bwd_kernel(const int32_t* __restrict__ tokens,
                                                            const T* __restrict__ dx, float* __restrict__ acc,
                                                            int64_t n_tokens, int64_t vocab, int64_t dim) {
  const int64_t t = blockIdx.x;
  int64_t tok = tokens[t];
  // Out-of-range updates are dropped while the forward clamps: this pair is what the reference's program does
  // (gather clamps its start indices, the scatter-add its adjoint rule emits drops updates that fall outside).
  if (tok < 0 || tok >= vocab) return;
  for (int64_t c = threadIdx.x; c < dim; c += 256) atomicAdd(acc + tok * dim + c, to_f32(dx[t * dim + c]));
}

__global__ __launch_bounds__(256) void fill_zero_kernel(float* p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) p[i] = 0.f;
}

__global__ __launch_bounds__(256) void f32_to_bf16_kernel(const float* __restrict__ in, bf16* __restrict__ out,
                                                          int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
    out[i] = from_f32<bf16>(in[i]);
}

// ---------------------------------------------------------------------------
// 2-D transpose out[c][r] = in[r][c] through a padded 64x64 LDS tile.  Used to put
// the contraction index of the adjoint GEMMs innermost (W -> W^T for dX = dY.W,
// dY -> dY^T and X -> X^T for dW = dY^T.X) so that they run on the k-contiguous
// MFMA path.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t rows,
                                                        int64_t cols, int vec_ok) {
  constexpr int TS = 64, PADW = TS + (sizeof(T) == 2 ? 2 : 1);
  __shared__ T tile[TS][PADW];
  const int64_t r0 = (int64_t)blockIdx.y * TS, c0 = (int64_t)blockIdx.x * TS;
  const int t = threadIdx.x;
  if (vec_ok && r0 + TS <= rows && c0 + TS <= cols) {
    constexpr int V = 16 / sizeof(T);            // elements per 16-byte access
    constexpr int CPR = TS / V;                  // chunks per tile row
#pragma unroll
    for (int i = 0; i < TS * CPR / 256; i++) {
      const int idx = t + i * 256, r = idx / CPR, c = (idx % CPR) * V;
      const uint4 v = *reinterpret_cast<const uint4*>(in + (r0 + r) * cols + c0 + c);
      const T* e = reinterpret_cast<const T*>(&v);
#pragma unroll
      for (int j = 0; j < V; j++) tile[r][c + j] = e[j];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TS * CPR / 256; i++) {
      const int idx = t + i * 256, c = idx / CPR, r = (idx % CPR) * V;
      uint4 v;
      T* e = reinterpret_cast<T*>(&v);
#pragma unroll
      for (int j = 0; j < V; j++) e[j] = tile[r + j][c];
      *reinterpret_cast<uint4*>(out + (c0 + c) * rows + r0 + r) = v;
    }
  } else {
    for (int idx = t; idx < TS * TS; idx += 256) {
      const int r = idx / TS, c = idx % TS;
      if (r0 + r < rows && c0 + c < cols) tile[r][c] = in[(r0 + r) * cols + c0 + c];
    }
    __syncthreads();
    for (int idx = t; idx < TS * TS; idx += 256) {
      const int c = idx / TS, r = idx % TS;
      if (r0 + r < rows && c0 + c < cols) out[(c0 + c) * rows + r0 + r] = tile[r][c];
    }
  }
}

// The same for whole 16-byte pieces (rows and cols multiples of V = 16 / sizeof(T), aligned buffers) without LDS:
// a thread owns a V x V block, reads its V rows as one 16-byte piece each, transposes the block in registers and
// writes V pieces.  The lanes of a wavefront form an 8 x 8 grid of such blocks, so that every read and every write
// instruction covers whole 128-byte lines (8 lanes x 16 bytes per row).
template <typename T, bool STREAM>
__global__ __launch_bounds__(256) void transpose_blocks_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t rows,
                                                               int64_t cols) {
  constexpr int V = 16 / sizeof(T);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // Blocks that run at the same time differ in both block coordinates (block row (y + x) mod rows of blocks): with
  // power-of-two row lengths, blocks of one block row write pieces that lie a multiple of 64 KiB apart, and those
  // of one block column read such pieces: either way a few memory channels would take all the traffic.
  const unsigned by = (blockIdx.y + blockIdx.x) % gridDim.y;
  const int64_t r = ((int64_t)by * 2 + (wave >> 1)) * 8 * V + (lane >> 3) * V;
  const int64_t c = ((int64_t)blockIdx.x * 2 + (wave & 1)) * 8 * V + (lane & 7) * V;
  if (r >= rows || c >= cols) return;
  uint32_t x[V][4], y[V][4];
#pragma unroll
  for (int i = 0; i < V; i++) {
    // weight-sized operands are read again soon (cached loads); activation-sized ones stream through
    const uint4 v = STREAM ? stream_load(reinterpret_cast<const uint4*>(in + (r + i) * cols + c))
                           : *reinterpret_cast<const uint4*>(in + (r + i) * cols + c);
    x[i][0] = v.x; x[i][1] = v.y; x[i][2] = v.z; x[i][3] = v.w;
  }
  if constexpr (V == 4) {
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int i = 0; i < 4; i++) y[j][i] = x[i][j];
  } else {
    // 16-bit elements: dword k of output row j holds input rows 2k and 2k + 1 at column j
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
      for (int k = 0; k < 4; k++) {
        const uint32_t a = x[2 * k][j >> 1], b = x[2 * k + 1][j >> 1];
        y[j][k] = (j & 1) ? ((a >> 16) | (b & 0xffff0000u)) : ((a & 0xffffu) | (b << 16));
      }
  }
#pragma unroll
  for (int j = 0; j < V; j++) {
    if (STREAM) stream_store(reinterpret_cast<uint4*>(out + (c + j) * rows + r), make_uint4(y[j][0], y[j][1], y[j][2], y[j][3]));
    else *reinterpret_cast<uint4*>(out + (c + j) * rows + r) = make_uint4(y[j][0], y[j][1], y[j][2], y[j][3]);
  }
}

// ---------------------------------------------------------------------------
// launch helpers
// ---------------------------------------------------------------------------

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
static inline unsigned blocks_for(int64_t n, int per) { return (unsigned)((n + per - 1) / per); }

// grid used by the RMSNorm adjoint; the workspace holds one fp32 partial row
// of dgamma per block.
static inline void rms_bwd_shape(int64_t rows, int64_t dim, int* tpr, int* nch, int64_t* grid, int64_t* nparts) {
  if ((dim & 7) == 0 && dim <= 8192) {
    const int64_t chunks = dim >> 3;
    *tpr = chunks <= 128 ? 64 : 256;
    const int64_t per = (chunks + *tpr - 1) / *tpr;
    *nch = per <= 1 ? 1 : (per <= 2 ? 2 : 4);
    const int rpb = 256 / *tpr;
    const int64_t groups = (rows + rpb - 1) / rpb;
    // Two resident blocks per CU: more blocks add partial rows (written here, read
    // again by the column sum) without adding bandwidth.  (Narrow rows, four per block: the same 512 blocks;
    // 128 left half of the CUs idle on the 768-wide model.)
    const int64_t cap = 512;
    *grid = groups < cap ? (groups > 0 ? groups : 1) : cap;
    *nparts = *grid;
  } else {
    *tpr = 0;
    *nch = 0;
    *grid = rows < 1024 ? (rows > 0 ? rows : 1) : 1024;
    *nparts = *grid;
  }
}

template <typename T>
static int rmsnorm_fwd_launch(hipStream_t st, const void* x, const void* gamma, void* y, int64_t rows, int64_t dim,
                              float eps) {
  const T* xp = static_cast<const T*>(x);
  const T* gp = static_cast<const T*>(gamma);
  T* yp = static_cast<T*>(y);
  int tpr, nch;
  int64_t grid, nparts;
  rms_bwd_shape(rows, dim, &tpr, &nch, &grid, &nparts);
  if (tpr == 0) {
    hipLaunchKernelGGL(rmsnorm_fwd_generic_kernel<T>, dim3((unsigned)rows), dim3(256), 0, st, xp, gp, yp, rows, dim, eps);
  } else {
    const unsigned g = blocks_for(rows, 256 / tpr);
#define EMI_RMS_FWD(TPR, NCH) \
  hipLaunchKernelGGL((rmsnorm_fwd_kernel<T, TPR, NCH>), dim3(g), dim3(256), 0, st, xp, gp, yp, rows, (int)dim, eps)
    if (tpr == 64 && nch == 1) EMI_RMS_FWD(64, 1);
    else if (tpr == 64) EMI_RMS_FWD(64, 2);
    else if (nch == 1) EMI_RMS_FWD(256, 1);
    else if (nch == 2) EMI_RMS_FWD(256, 2);
    else EMI_RMS_FWD(256, 4);
#undef EMI_RMS_FWD
  }
  EMI_CHECK_LAUNCH("emi_rmsnorm_fwd");
  return EMI_OK;
}

template <typename T>
static int rmsnorm_bwd_launch(hipStream_t st, const void* x, const void* gamma, const void* dy, const void* dx_add,
                              void* dx, void* dgamma, void* ws, int64_t rows, int64_t dim, float eps) {
  const T* xp = static_cast<const T*>(x);
  const T* gp = static_cast<const T*>(gamma);
  const T* dyp = static_cast<const T*>(dy);
  const T* ap = static_cast<const T*>(dx_add);
  T* dxp = static_cast<T*>(dx);
  float* part = static_cast<float*>(ws);
  int tpr, nch;
  int64_t grid, nparts;
  rms_bwd_shape(rows, dim, &tpr, &nch, &grid, &nparts);
  if (tpr == 0) {
    hipLaunchKernelGGL(rmsnorm_bwd_generic_kernel<T>, dim3((unsigned)grid), dim3(256), 0, st, xp, gp, dyp, ap, dxp, part,
                       rows, dim, eps);
  } else {
#define EMI_RMS_BWD(TPR, NCH)                                                                                   \
  hipLaunchKernelGGL((rmsnorm_bwd_kernel<T, TPR, NCH, (sizeof(T) == 2 ? 2 : 1)>), dim3((unsigned)grid), dim3(256), 0, st, xp, gp, dyp, ap, dxp, \
                     part, rows, (int)dim, eps)
    if (tpr == 64 && nch == 1) EMI_RMS_BWD(64, 1);
    else if (tpr == 64) EMI_RMS_BWD(64, 2);
    else if (nch == 1) EMI_RMS_BWD(256, 1);
    else if (nch == 2) EMI_RMS_BWD(256, 2);
    else EMI_RMS_BWD(256, 4);
#undef EMI_RMS_BWD
  }
  EMI_CHECK_LAUNCH("emi_rmsnorm_bwd");
  // [nparts, dim] -> [ceil(nparts/CS_ROWS), dim] -> ... -> dgamma
  float* cur = part;
  float* nxt = part + nparts * dim;
  int64_t n = nparts;
  while (n > CS_ROWS) {
    const int64_t m = (n + CS_ROWS - 1) / CS_ROWS;
    hipLaunchKernelGGL(colsum_kernel<float>, dim3(blocks_for(dim, 64), (unsigned)m), dim3(1024), 0, st, cur, (int)n, dim, nxt);
    EMI_CHECK_LAUNCH("emi_rmsnorm_bwd(colsum)");
    float* t = cur;
    cur = nxt;
    nxt = t;
    n = m;
  }
  hipLaunchKernelGGL(colsum_kernel<T>, dim3(blocks_for(dim, 64), 1), dim3(1024), 0, st, cur, (int)n, dim,
                     static_cast<T*>(dgamma));
  EMI_CHECK_LAUNCH("emi_rmsnorm_bwd(colsum)");
  return EMI_OK;
}

}  // namespace emi

using namespace emi;

#define EMI_DISPATCH_DTYPE(name, dtype, call_f32, call_bf16)                           \
  switch (dtype) {                                                                     \
    case EMI_F32: return call_f32;                                                     \
    case EMI_BF16: return call_bf16;                                                   \
    default: return emi_fail(EMI_INVALID_ARGUMENT, "%s: unsupported dtype code %d (want 11=f32 or 16=bf16)", name, dtype); \
  }

extern "C" int emi_rmsnorm_fwd(emi_stream_t stream, const void* x, const void* gamma, void* y, int64_t rows,
                               int64_t dim, float eps, int dtype) {
  EMI_REQUIRE(rows >= 0 && dim > 0, "emi_rmsnorm_fwd: bad shape rows=%lld dim=%lld", (long long)rows, (long long)dim);
  EMI_REQUIRE(rows <= 0x7fffffffLL * 4, "emi_rmsnorm_fwd: rows=%lld too large", (long long)rows);
  if (rows == 0) return EMI_OK;
  EMI_REQUIRE(x && gamma && y, "emi_rmsnorm_fwd: null buffer");
  EMI_REQUIRE(aligned16(x) && aligned16(gamma) && aligned16(y), "emi_rmsnorm_fwd: buffers must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  EMI_DISPATCH_DTYPE("emi_rmsnorm_fwd", dtype, rmsnorm_fwd_launch<float>(st, x, gamma, y, rows, dim, eps),
                     rmsnorm_fwd_launch<bf16>(st, x, gamma, y, rows, dim, eps));
}

extern "C" size_t emi_rmsnorm_bwd_workspace_bytes(int64_t rows, int64_t dim) {
  if (rows <= 0 || dim <= 0) return 0;
  int tpr, nch;
  int64_t grid, nparts;
  rms_bwd_shape(rows, dim, &tpr, &nch, &grid, &nparts);
  // first-level partial rows + one ping-pong area for the second level of the column sum
  return ((size_t)nparts + (size_t)((nparts + CS_ROWS - 1) / CS_ROWS)) * (size_t)dim * sizeof(float);
}

extern "C" int emi_rmsnorm_bwd(emi_stream_t stream, const void* x, const void* gamma, const void* dy,
                               const void* dx_add, void* dx, void* dgamma, void* workspace, size_t workspace_bytes,
                               int64_t rows, int64_t dim, float eps, int dtype) {
  EMI_REQUIRE(rows > 0 && dim > 0, "emi_rmsnorm_bwd: bad shape rows=%lld dim=%lld", (long long)rows, (long long)dim);
  EMI_REQUIRE(x && gamma && dy && dx && dgamma, "emi_rmsnorm_bwd: null buffer");
  EMI_REQUIRE(aligned16(x) && aligned16(gamma) && aligned16(dy) && aligned16(dx) && aligned16(dx_add) &&
                  aligned16(workspace),
              "emi_rmsnorm_bwd: buffers must be 16-byte aligned");
  const size_t need = emi_rmsnorm_bwd_workspace_bytes(rows, dim);
  EMI_REQUIRE(workspace != nullptr && workspace_bytes >= need, "emi_rmsnorm_bwd: workspace of %zu bytes needed, got %zu",
              need, workspace_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  EMI_DISPATCH_DTYPE("emi_rmsnorm_bwd", dtype,
                     rmsnorm_bwd_launch<float>(st, x, gamma, dy, dx_add, dx, dgamma, workspace, rows, dim, eps),
                     rmsnorm_bwd_launch<bf16>(st, x, gamma, dy, dx_add, dx, dgamma, workspace, rows, dim, eps));
}

// ---------------------------------------------------------------------------
// Allocation-free variant of emi_rmsnorm_bwd for callers that cannot allocate (HIP graph capture, serving loops):
// the fp32 partial rows of dgamma live in a file-scope device array instead of a caller workspace.  The array's
// name is a host-side stand-in, not a device address; its address on each device is looked up once, with that
// device current, and only that pointer is ever handed to a kernel.  Every call on a device shares the device's
// array (overlapping calls on one device race); the kernels write every partial row they later read, so nothing
// needs clearing between calls.
// ---------------------------------------------------------------------------
constexpr size_t kRmsScratchBytes = EMI_RMSNORM_BWD_NOALLOC_MAX_BYTES;      // (512 + 1) partial rows of 8192 floats
static __device__ __align__(256) unsigned char emi_rms_scratch[kRmsScratchBytes];
constexpr int kMaxDevices = 64;
static void* g_rms_scratch_ptr[kMaxDevices];
static std::mutex g_rms_scratch_mu;

static int rms_scratch_for_current_device(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return emi_fail(EMI_INTERNAL, "emi_rmsnorm_bwd_noalloc: cannot identify the current device");
  std::lock_guard<std::mutex> lock(g_rms_scratch_mu);
  if (g_rms_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(emi_rms_scratch));
    if (e != hipSuccess || p == nullptr)
      return emi_fail(EMI_INTERNAL, "emi_rmsnorm_bwd_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
    g_rms_scratch_ptr[dev] = p;
  }
  *out = g_rms_scratch_ptr[dev];
  return EMI_OK;
}

extern "C" int emi_rmsnorm_bwd_noalloc(emi_stream_t stream, const void* x, const void* gamma, const void* dy,
                                       const void* dx_add, void* dx, void* dgamma, int64_t rows, int64_t dim, float eps,
                                       int dtype) {
  EMI_REQUIRE(rows > 0 && dim > 0, "emi_rmsnorm_bwd_noalloc: bad shape rows=%lld dim=%lld", (long long)rows, (long long)dim);
  const size_t need = emi_rmsnorm_bwd_workspace_bytes(rows, dim);
  EMI_REQUIRE(need <= kRmsScratchBytes,
              "emi_rmsnorm_bwd_noalloc: rows=%lld dim=%lld needs %zu bytes of scratch, the built-in array holds %zu "
              "(dim <= 8192 and a multiple of 8 always fits); use emi_rmsnorm_bwd with a workspace",
              (long long)rows, (long long)dim, need, kRmsScratchBytes);
  void* scratch = nullptr;
  if (int rc = rms_scratch_for_current_device(&scratch)) return rc;
  return emi_rmsnorm_bwd(stream, x, gamma, dy, dx_add, dx, dgamma, scratch, kRmsScratchBytes, rows, dim, eps, dtype);
}

extern "C" int emi_rope_table(emi_stream_t stream, float* table, int64_t seq, int64_t head_dim, double theta,
                              int64_t pos0) {
  EMI_REQUIRE(seq > 0 && head_dim > 0 && (head_dim & 1) == 0, "emi_rope_table: bad shape seq=%lld head_dim=%lld",
              (long long)seq, (long long)head_dim);
  EMI_REQUIRE(table != nullptr && aligned16(table), "emi_rope_table: table must be a 16-byte aligned device buffer");
  EMI_REQUIRE(theta > 0.0, "emi_rope_table: theta must be positive");
  const int half = (int)(head_dim / 2);
  hipLaunchKernelGGL(rope_table_kernel, dim3(blocks_for(seq * half, 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<float2*>(table), seq, half, (int)head_dim, theta, pos0);
  EMI_CHECK_LAUNCH("emi_rope_table");
  return EMI_OK;
}

template <typename T>
static int rope_launch(hipStream_t st, const void* x, const float* table, void* y, int64_t batch, int64_t seq,
                       int64_t heads, int64_t head_dim, int inverse) {
  const int64_t n = batch * seq * heads * head_dim;
  const float2* tp = reinterpret_cast<const float2*>(table);
  const int64_t rows = batch * seq, row_elems = heads * head_dim;
  constexpr int V = ChunkCached<T>::N;
  if (head_dim % V == 0 && rows <= 0x7fffffff && (row_elems / V + 255) / 256 <= 65535) {
    const int chunks = (int)(row_elems / V);
    const int bs = chunks >= 256 ? 256 : (chunks + 63) / 64 * 64;            // short rows: no idle wavefronts
    const dim3 grid((unsigned)rows, (unsigned)((chunks + bs - 1) / bs));
    hipLaunchKernelGGL(rope_kernel<T>, grid, dim3(bs), 0, st, static_cast<const T*>(x), tp, static_cast<T*>(y), (int)seq,
                       (int)row_elems, (int)head_dim, inverse);
  } else {
    hipLaunchKernelGGL(rope_pair_kernel<T>, dim3(blocks_for(n / 2, 256)), dim3(256), 0, st, static_cast<const T*>(x), tp,
                       static_cast<T*>(y), n / 2, (int)seq, (int)(heads * head_dim), (int)head_dim, inverse);
  }
  EMI_CHECK_LAUNCH("emi_rope");
  return EMI_OK;
}

extern "C" int emi_rope(emi_stream_t stream, const void* x, const float* table, void* y, int64_t batch, int64_t seq,
                        int64_t heads, int64_t head_dim, int inverse, int dtype) {
  EMI_REQUIRE(batch >= 0 && seq > 0 && heads > 0 && head_dim > 0 && (head_dim & 1) == 0,
              "emi_rope: bad shape [%lld,%lld,%lld,%lld] (head_dim must be even)", (long long)batch, (long long)seq,
              (long long)heads, (long long)head_dim);
  EMI_REQUIRE(heads * head_dim <= 0x7fffffff && seq <= 0x7fffffff, "emi_rope: row too large");
  if (batch == 0) return EMI_OK;
  EMI_REQUIRE(x && y && table, "emi_rope: null buffer");
  EMI_REQUIRE(aligned16(x) && aligned16(y) && aligned16(table), "emi_rope: buffers must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  EMI_DISPATCH_DTYPE("emi_rope", dtype, rope_launch<float>(st, x, table, y, batch, seq, heads, head_dim, inverse),
                     rope_launch<bf16>(st, x, table, y, batch, seq, heads, head_dim, inverse));
}

template <typename T>
static int swiglu_fwd_launch(hipStream_t st, const void* a, const void* b, void* g, int64_t n) {
  hipLaunchKernelGGL(swiglu_fwd_kernel<T>, dim3(blocks_for((n >> 3) + (n & 7), 256)), dim3(256), 0, st,
                     static_cast<const T*>(a), static_cast<const T*>(b), static_cast<T*>(g), n);
  EMI_CHECK_LAUNCH("emi_swiglu_fwd");
  return EMI_OK;
}
template <typename T>
static int swiglu_bwd_launch(hipStream_t st, const void* a, const void* b, const void* dg, void* da, void* db,
                             int64_t n) {
  hipLaunchKernelGGL(swiglu_bwd_kernel<T>, dim3(blocks_for((n >> 3) + (n & 7), 256)), dim3(256), 0, st,
                     static_cast<const T*>(a), static_cast<const T*>(b), static_cast<const T*>(dg), static_cast<T*>(da),
                     static_cast<T*>(db), n);
  EMI_CHECK_LAUNCH("emi_swiglu_bwd");
  return EMI_OK;
}
template <typename T> static int add_launch(hipStream_t st, const void* a, const void* b, void* y, int64_t n) {
  hipLaunchKernelGGL(add_kernel<T>, dim3(blocks_for((n >> 3) + (n & 7), 256)), dim3(256), 0, st, static_cast<const T*>(a),
                     static_cast<const T*>(b), static_cast<T*>(y), n);
  EMI_CHECK_LAUNCH("emi_add");
  return EMI_OK;
}

extern "C" int emi_swiglu_fwd(emi_stream_t stream, const void* a, const void* b, void* g, int64_t n, int dtype) {
  EMI_REQUIRE(n >= 0, "emi_swiglu_fwd: negative size");
  if (n == 0) return EMI_OK;
  EMI_REQUIRE(a && b && g, "emi_swiglu_fwd: null buffer");
  EMI_REQUIRE(aligned16(a) && aligned16(b) && aligned16(g), "emi_swiglu_fwd: buffers must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  EMI_DISPATCH_DTYPE("emi_swiglu_fwd", dtype, swiglu_fwd_launch<float>(st, a, b, g, n),
                     swiglu_fwd_launch<bf16>(st, a, b, g, n));
}

extern "C" int emi_swiglu_bwd(emi_stream_t stream, const void* a, const void* b, const void* dg, void* da, void* db,
                              int64_t n, int dtype) {
  EMI_REQUIRE(n >= 0, "emi_swiglu_bwd: negative size");
  if (n == 0) return EMI_OK;
  EMI_REQUIRE(a && b && dg && da && db, "emi_swiglu_bwd: null buffer");
  EMI_REQUIRE(aligned16(a) && aligned16(b) && aligned16(dg) && aligned16(da) && aligned16(db),
              "emi_swiglu_bwd: buffers must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  EMI_DISPATCH_DTYPE("emi_swiglu_bwd", dtype, swiglu_bwd_launch<float>(st, a, b, dg, da, db, n),
                     swiglu_bwd_launch<bf16>(st, a, b, dg, da, db, n));
}

extern "C" int emi_add(emi_stream_t stream, const void* a, const void* b, void* y, int64_t n, int dtype) {
  EMI_REQUIRE(n >= 0, "emi_add: negative size");
  if (n == 0) return EMI_OK;
  EMI_REQUIRE(a && b && y, "emi_add: null buffer");
  EMI_REQUIRE(aligned16(a) && aligned16(b) && aligned16(y), "emi_add: buffers must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  EMI_DISPATCH_DTYPE("emi_add", dtype, add_launch<float>(st, a, b, y, n), add_launch<bf16>(st, a, b, y, n));
}

template <typename T>
static int embedding_fwd_launch(hipStream_t st, const int32_t* tokens, const void* table, void* x, int64_t n_tokens,
                                int64_t vocab, int64_t dim) {
  hipLaunchKernelGGL(embedding_fwd_kernel<T>, dim3((unsigned)n_tokens), dim3(256), 0, st, tokens,
                     static_cast<const T*>(table), static_cast<T*>(x), n_tokens, vocab, dim);
  EMI_CHECK_LAUNCH("emi_embedding_fwd");
  return EMI_OK;
}

extern "C" int emi_embedding_fwd(emi_stream_t stream, const int32_t* tokens, const void* table, void* x,
                                 int64_t n_tokens, int64_t vocab, int64_t dim, int dtype) {
  EMI_REQUIRE(n_tokens >= 0 && vocab > 0 && dim > 0, "emi_embedding_fwd: bad shape");
  EMI_REQUIRE(n_tokens <= 0x7fffffff, "emi_embedding_fwd: too many tokens");
  if (n_tokens == 0) return EMI_OK;
  EMI_REQUIRE(tokens && table && x, "emi_embedding_fwd: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  EMI_DISPATCH_DTYPE("emi_embedding_fwd", dtype, embedding_fwd_launch<float>(st, tokens, table, x, n_tokens, vocab, dim),
                     embedding_fwd_launch<bf16>(st, tokens, table, x, n_tokens, vocab, dim));
}

extern "C" size_t emi_embedding_bwd_workspace_bytes(int64_t vocab, int64_t dim, int dtype) {
  if (vocab <= 0 || dim <= 0) return 0;
  return dtype == EMI_BF16 ? (size_t)vocab * (size_t)dim * sizeof(float) : 0;
}

extern "C" int emi_embedding_bwd(emi_stream_t stream, const int32_t* tokens, const void* dx, void* dtable,
                                 void* workspace, size_t workspace_bytes, int64_t n_tokens, int64_t vocab, int64_t dim,
                                 int dtype) {
  EMI_REQUIRE(n_tokens >= 0 && vocab > 0 && dim > 0, "emi_embedding_bwd: bad shape");
  EMI_REQUIRE(n_tokens <= 0x7fffffff, "emi_embedding_bwd: too many tokens");
  EMI_REQUIRE(dtable != nullptr && (n_tokens == 0 || (tokens && dx)), "emi_embedding_bwd: null buffer");
  EMI_REQUIRE(dtype == EMI_F32 || dtype == EMI_BF16, "emi_embedding_bwd: unsupported dtype code %d", dtype);
  const size_t need = emi_embedding_bwd_workspace_bytes(vocab, dim, dtype);
  EMI_REQUIRE(need == 0 || (workspace != nullptr && workspace_bytes >= need),
              "emi_embedding_bwd: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  float* acc = dtype == EMI_BF16 ? static_cast<float*>(workspace) : static_cast<float*>(dtable);
  const int64_t total = vocab * dim;
  hipLaunchKernelGGL(fill_zero_kernel, dim3(2048), dim3(256), 0, st, acc, total);
  EMI_CHECK_LAUNCH("emi_embedding_bwd(zero)");
  if (n_tokens > 0) {
    if (dtype == EMI_BF16)
      hipLaunchKernelGGL(embedding_bwd_kernel<bf16>, dim3((unsigned)n_tokens), dim3(256), 0, st, tokens,
                         static_cast<const bf16*>(dx), acc, n_tokens, vocab, dim);
    else
      hipLaunchKernelGGL(embedding_bwd_kernel<float>, dim3((unsigned)n_tokens), dim3(256), 0, st, tokens,
                         static_cast<const float*>(dx), acc, n_tokens, vocab, dim);
    EMI_CHECK_LAUNCH("emi_embedding_bwd");
  }
  if (dtype == EMI_BF16) {
    hipLaunchKernelGGL(f32_to_bf16_kernel, dim3(2048), dim3(256), 0, st, acc, static_cast<bf16*>(dtable), total);
    EMI_CHECK_LAUNCH("emi_embedding_bwd(convert)");
  }
  return EMI_OK;
}

template <typename T> static int transpose_launch(hipStream_t st, const void* in, void* out, int64_t rows, int64_t cols) {
  const int vec_ok = (aligned16(in) && aligned16(out) && rows % 8 == 0 && cols % 8 == 0) ? 1 : 0;
  constexpr int V = 16 / sizeof(T);
  if (vec_ok && (rows + 16 * V - 1) / (16 * V) <= 65535) {
    const dim3 gridb(blocks_for(cols, 16 * V), blocks_for(rows, 16 * V));
    if (rows * cols * (int64_t)sizeof(T) > (int64_t)(128 << 20))
      hipLaunchKernelGGL((transpose_blocks_kernel<T, true>), gridb, dim3(256), 0, st, static_cast<const T*>(in), static_cast<T*>(out),
                         rows, cols);
    else
      hipLaunchKernelGGL((transpose_blocks_kernel<T, false>), gridb, dim3(256), 0, st, static_cast<const T*>(in), static_cast<T*>(out),
                         rows, cols);
    EMI_CHECK_LAUNCH("emi_transpose");
    return EMI_OK;
  }
  const dim3 grid(blocks_for(cols, 64), blocks_for(rows, 64));
  hipLaunchKernelGGL(transpose_kernel<T>, grid, dim3(256), 0, st, static_cast<const T*>(in), static_cast<T*>(out), rows, cols,
                     vec_ok);
  EMI_CHECK_LAUNCH("emi_transpose");
  return EMI_OK;
}

extern "C" int emi_transpose(emi_stream_t stream, const void* in, void* out, int64_t rows, int64_t cols, int dtype) {
  EMI_REQUIRE(rows >= 0 && cols >= 0, "emi_transpose: negative size");
  if (rows == 0 || cols == 0) return EMI_OK;
  EMI_REQUIRE(in && out && in != out, "emi_transpose: null or aliased buffer");
  EMI_REQUIRE((rows + 63) / 64 <= 65535, "emi_transpose: more than 65535*64 rows");
  hipStream_t st = static_cast<hipStream_t>(stream);
  EMI_DISPATCH_DTYPE("emi_transpose", dtype, transpose_launch<float>(st, in, out, rows, cols),
                     transpose_launch<bf16>(st, in, out, rows, cols));
}
