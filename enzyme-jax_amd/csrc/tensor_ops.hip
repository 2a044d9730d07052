// Generic tensor operators for graphs that reach the library as StableHLO text
// (hlo_call, src/enzyme_ad/jax/primitives.py:1052-1108): the elementwise, data-movement
// and reduction operators that are left once the llama clusters (RMSNorm, SwiGLU, attention,
// projections) have been matched to their fused kernels.  All of them are HBM-bound: they
// move 16-byte chunks per lane where the layout allows, and compute in fp32.
#include "emi_device.h"

namespace emi {
namespace {

constexpr int kBlock = 256;
constexpr int kMaxRank = 8;

inline bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
// one lane per group of eight elements plus one per leftover element (VEC), or per element
inline unsigned map_grid(int64_t n, bool vec) {
  const int64_t lanes = vec ? (n >> 3) + (n & 7) : n;
  return (unsigned)((lanes + kBlock - 1) / kBlock);
}
// The elementwise kernels' vector form: a block covers `per_thread` elements per thread as 16-byte pieces, all of a
// thread's loads in flight together; piece p of thread t is piece p * kBlock + t of the block's range, so every access
// instruction of a wavefront covers consecutive memory.  The elements past the last whole piece go to the first threads
// of block 0.  Measured at [32768, 4096]: four pieces per operand serve fp32 best (multiply 0.76 -> 0.78 of the HBM peak,
// exponential 0.72 -> 0.77) and one piece bf16 (0.82 against 0.79 with two); the kernels with a byte mask next to the
// operands take 16 elements per thread in both types (compare 0.68 -> 0.79 fp32, 0.75 -> 0.80 bf16; select 0.75 -> 0.84,
// 0.86 -> 0.89).
template <typename T> constexpr int map_pieces() { return sizeof(T) == 4 ? 4 : 1; }
template <typename T> constexpr int mask_pieces() { return 16 / Chunk<T>::N; }
inline unsigned piece_grid(int64_t n, bool vec, int per_thread) {
  const int64_t per_block = (int64_t)kBlock * (vec ? per_thread : 1);
  return (unsigned)((n + per_block - 1) / per_block);
}
inline unsigned grid_for(int64_t items, int per_block) {
  int64_t g = (items + per_block - 1) / per_block;
  const int64_t cap = 256 * 32;  // 32 blocks per CU: grid-stride loops cover the rest
  return (unsigned)(g < 1 ? 1 : (g > cap ? cap : g));
}

// ---------------------------------------------------------------------------
// elementwise maps
// ---------------------------------------------------------------------------
template <int OP> __device__ __forceinline__ float apply_binary(float a, float b) {
  switch (OP) {
    case EMI_OP_ADD: return a + b;
    case EMI_OP_SUB: return a - b;
    case EMI_OP_MUL: return a * b;
    case EMI_OP_DIV: return a / b;
    case EMI_OP_MAX: return (a != a || b != b) ? (a + b) : fmaxf(a, b);   // NaN propagates
    case EMI_OP_MIN: return (a != a || b != b) ? (a + b) : fminf(a, b);
    case EMI_OP_GE: return a >= b ? 1.0f : 0.0f;
    case EMI_OP_EQ: return a == b ? 1.0f : 0.0f;
    case EMI_OP_NMUL: return -(a * b);
    case EMI_OP_POW: return powf(a, b);
    // derivative factors: a = incoming cotangent / tangent, b = the operator's input or result
    case EMI_OP_D_SQRT: return b == 0.0f ? 0.0f : a / (2.0f * b);          // b = sqrt(x)
    case EMI_OP_D_RSQRT: return -0.5f * a * b * b * b;                     // b = rsqrt(x)
    case EMI_OP_D_LOGISTIC: return a * b * (1.0f - b);                     // b = logistic(x)
    case EMI_OP_D_TANH: return a * (1.0f - b * b);                         // b = tanh(x)
    case EMI_OP_D_SIN: return a * cosf(b);                                 // b = x
    case EMI_OP_D_COS: return -a * sinf(b);                                // b = x
    case EMI_OP_D_POW_A: return b * powf(a, b - 1.0f);
    case EMI_OP_D_POW_B: return powf(a, b) * logf(a);
    case EMI_OP_D_ABS: return b >= 0.0f ? a : -a;                           // b = x
    case EMI_OP_D_LOG1P: return a / (b + 1.0f);                            // b = x
    case EMI_OP_D_EXPM1: return a * expf(b);                               // b = x
    case EMI_OP_D_CBRT: return a / (3.0f * b * b);                         // b = cbrt(x)
    case EMI_OP_ATAN2: return atan2f(a, b);
    default: return 0.0f;
  }
}

template <int OP> __device__ __forceinline__ float apply_unary(float a) {
  switch (OP) {
    case EMI_OP_NEG: return -a;
    case EMI_OP_EXP: return expf(a);
    case EMI_OP_LOG: return logf(a);
    case EMI_OP_SQRT: return sqrtf(a);
    case EMI_OP_RSQRT: return 1.0f / sqrtf(a);
    case EMI_OP_LOGISTIC: return 1.0f / (1.0f + expf(-a));
    case EMI_OP_TANH: return tanhf(a);
    case EMI_OP_SIN: return sinf(a);
    case EMI_OP_COS: return cosf(a);
    case EMI_OP_ABS: return fabsf(a);
    case EMI_OP_COPY: return a;
    case EMI_OP_LOG1P: return log1pf(a);
    case EMI_OP_EXPM1: return expm1f(a);
    case EMI_OP_CBRT: return cbrtf(a);
    default: return 0.0f;
  }
}

// y[i] = op(a[i * sa], b[i * sb]); sa, sb in {0, 1} (0: the operand is one element).
// VEC: one group of eight elements per lane (16 bytes of bf16, 2 x 16 bytes of fp32), enough
// workgroups to cover the tensor; the last n % 8 elements go to the lanes after the groups.
template <typename T, bool VEC, int OP>
__global__ void __launch_bounds__(kBlock) map_binary_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                            T* __restrict__ y, int64_t n, int sa, int sb) {
  if (VEC) {                                            // see piece_grid
    constexpr int N = Chunk<T>::N, P = map_pieces<T>();
    const int64_t npieces = n / N, first = (int64_t)blockIdx.x * (kBlock * P) + threadIdx.x;
    typename Chunk<T>::Raw ra[P], rb[P];
#pragma unroll
    for (int p = 0; p < P; p++) {
      const int64_t c = first + p * kBlock;
      if (c < npieces) {
        if (sa) ra[p] = Chunk<T>::load_raw(a + c * N);
        if (sb) rb[p] = Chunk<T>::load_raw(b + c * N);
      }
    }
    const float va = sa ? 0.f : to_f32(a[0]), vb = sb ? 0.f : to_f32(b[0]);
#pragma unroll
    for (int p = 0; p < P; p++) {
      const int64_t c = first + p * kBlock;
      if (c < npieces) {
        float fa[N], fb[N];
        if (sa) Chunk<T>::unpack(ra[p], fa);
        if (sb) Chunk<T>::unpack(rb[p], fb);
#pragma unroll
        for (int j = 0; j < N; j++) fa[j] = apply_binary<OP>(sa ? fa[j] : va, sb ? fb[j] : vb);
        Chunk<T>::store(y + c * N, fa);
      }
    }
    if (blockIdx.x == 0 && threadIdx.x < n - npieces * N) {
      const int64_t e = npieces * N + threadIdx.x;
      y[e] = from_f32<T>(apply_binary<OP>(to_f32(a[sa ? e : 0]), to_f32(b[sb ? e : 0])));
    }
  } else {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) y[i] = from_f32<T>(apply_binary<OP>(to_f32(a[sa ? i : 0]), to_f32(b[sb ? i : 0])));
  }
}

template <typename T, bool VEC, int OP>
__global__ void __launch_bounds__(kBlock) map_unary_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n) {
  if (VEC) {                                            // see piece_grid
    constexpr int N = Chunk<T>::N, P = map_pieces<T>();
    const int64_t npieces = n / N, first = (int64_t)blockIdx.x * (kBlock * P) + threadIdx.x;
    typename Chunk<T>::Raw r[P];
#pragma unroll
    for (int p = 0; p < P; p++)
      if (first + p * kBlock < npieces) r[p] = Chunk<T>::load_raw(x + (first + p * kBlock) * N);
#pragma unroll
    for (int p = 0; p < P; p++) {
      const int64_t c = first + p * kBlock;
      if (c < npieces) {
        float f[N];
        Chunk<T>::unpack(r[p], f);
#pragma unroll
        for (int j = 0; j < N; j++) f[j] = apply_unary<OP>(f[j]);
        Chunk<T>::store(y + c * N, f);
      }
    }
    if (blockIdx.x == 0 && threadIdx.x < n - npieces * N) {
      const int64_t e = npieces * N + threadIdx.x;
      y[e] = from_f32<T>(apply_unary<OP>(to_f32(x[e])));
    }
  } else {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) y[i] = from_f32<T>(apply_unary<OP>(to_f32(x[i])));
  }
}

template <typename TI, typename TO, bool VEC>
__global__ void __launch_bounds__(kBlock) convert_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (VEC) {
    const int64_t ngroups = n >> 3;
    if (i < ngroups) {
      float v[8];
      Vec8<TI>::load(x + i * 8, v);
      Vec8<TO>::store(y + i * 8, v);
    } else if (i - ngroups < (n & 7)) {
      const int64_t e = (ngroups << 3) + (i - ngroups);
      y[e] = from_f32<TO>(to_f32(x[e]));
    }
  } else if (i < n) {
    y[i] = from_f32<TO>(to_f32(x[i]));
  }
}

// compare: mask[i] = dir(a[i * sa], b[i * sb]) as one byte (0 / 1); select: y[i] = mask ? a : b.
__device__ __forceinline__ bool cmp(int dir, float a, float b) {
  switch (dir) {
    case EMI_CMP_EQ: return a == b;
    case EMI_CMP_NE: return a != b;
    case EMI_CMP_GE: return a >= b;
    case EMI_CMP_GT: return a > b;
    case EMI_CMP_LE: return a <= b;
    default: return a < b;
  }
}

template <typename T, bool VEC>
__global__ void __launch_bounds__(kBlock) compare_kernel(int dir, const T* __restrict__ a, const T* __restrict__ b,
                                                         uint8_t* __restrict__ mask, int64_t n, int sa, int sb) {
  if (VEC) {                                            // see piece_grid
    constexpr int N = Chunk<T>::N, P = mask_pieces<T>();
    const int64_t npieces = n / N, first = (int64_t)blockIdx.x * (kBlock * P) + threadIdx.x;
    typename Chunk<T>::Raw ra[P], rb[P];
#pragma unroll
    for (int p = 0; p < P; p++) {
      const int64_t c = first + p * kBlock;
      if (c < npieces) {
        if (sa) ra[p] = Chunk<T>::load_raw(a + c * N);
        if (sb) rb[p] = Chunk<T>::load_raw(b + c * N);
      }
    }
    const float va = sa ? 0.f : to_f32(a[0]), vb = sb ? 0.f : to_f32(b[0]);
#pragma unroll
    for (int p = 0; p < P; p++) {
      const int64_t c = first + p * kBlock;
      if (c < npieces) {
        float fa[N], fb[N];
        if (sa) Chunk<T>::unpack(ra[p], fa);
        if (sb) Chunk<T>::unpack(rb[p], fb);
        uint32_t w[N / 4];
#pragma unroll
        for (int q = 0; q < N / 4; q++) w[q] = 0u;
#pragma unroll
        for (int j = 0; j < N; j++) w[j >> 2] |= (uint32_t)cmp(dir, sa ? fa[j] : va, sb ? fb[j] : vb) << (8 * (j & 3));
        if constexpr (N == 4) *reinterpret_cast<uint32_t*>(mask + c * N) = w[0];
        else *reinterpret_cast<uint2*>(mask + c * N) = make_uint2(w[0], w[1]);
      }
    }
    if (blockIdx.x == 0 && threadIdx.x < n - npieces * N) {
      const int64_t e = npieces * N + threadIdx.x;
      mask[e] = cmp(dir, to_f32(a[sa ? e : 0]), to_f32(b[sb ? e : 0]));
    }
  } else {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) mask[i] = cmp(dir, to_f32(a[sa ? i : 0]), to_f32(b[sb ? i : 0]));
  }
}

template <typename T, bool VEC>
__global__ void __launch_bounds__(kBlock) select_kernel(const uint8_t* __restrict__ mask, const T* __restrict__ a,
                                                        const T* __restrict__ b, T* __restrict__ y, int64_t n, int sm, int sa,
                                                        int sb) {
  if (VEC) {                                            // see piece_grid
    constexpr int N = Chunk<T>::N, P = mask_pieces<T>();
    const int64_t npieces = n / N, first = (int64_t)blockIdx.x * (kBlock * P) + threadIdx.x;
    typename Chunk<T>::Raw ra[P], rb[P];
    uint32_t m[P][N / 4];
    const uint32_t mall = sm ? 0u : (mask[0] ? 0x01010101u : 0u);
#pragma unroll
    for (int p = 0; p < P; p++) {
      const int64_t c = first + p * kBlock;
      if (c < npieces) {
        if (sa) ra[p] = Chunk<T>::load_raw(a + c * N);
        if (sb) rb[p] = Chunk<T>::load_raw(b + c * N);
#pragma unroll
        for (int q = 0; q < N / 4; q++) m[p][q] = sm ? reinterpret_cast<const uint32_t*>(mask + c * N)[q] : mall;
      }
    }
    const float va = sa ? 0.f : to_f32(a[0]), vb = sb ? 0.f : to_f32(b[0]);
#pragma unroll
    for (int p = 0; p < P; p++) {
      const int64_t c = first + p * kBlock;
      if (c < npieces) {
        float fa[N], fb[N];
        if (sa) Chunk<T>::unpack(ra[p], fa);
        if (sb) Chunk<T>::unpack(rb[p], fb);
#pragma unroll
        for (int j = 0; j < N; j++) fa[j] = ((m[p][j >> 2] >> (8 * (j & 3))) & 0xff) ? (sa ? fa[j] : va) : (sb ? fb[j] : vb);
        Chunk<T>::store(y + c * N, fa);
      }
    }
    if (blockIdx.x == 0 && threadIdx.x < n - npieces * N) {
      const int64_t e = npieces * N + threadIdx.x;
      y[e] = mask[sm ? e : 0] ? a[sa ? e : 0] : b[sb ? e : 0];
    }
  } else {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) y[i] = mask[sm ? i : 0] ? a[sa ? i : 0] : b[sb ? i : 0];
  }
}

// ---------------------------------------------------------------------------
// strided copy: out[o0 + sum_d i_d * os_d] = in[i0 + sum_d i_d * is_d] over the index box
// dims[0..rank).  Covers transpose (permuted strides), broadcast_in_dim (zero strides),
// slice (offset + strides) and concatenate (a sub-box of the result).
// ---------------------------------------------------------------------------
struct CopyPlan {
  int rank;
  int64_t total;
  int64_t dims[kMaxRank];
  int64_t is[kMaxRank];
  int64_t os[kMaxRank];
};

template <typename E>
__global__ void __launch_bounds__(kBlock) strided_copy_kernel(const E* __restrict__ in, E* __restrict__ out, CopyPlan p) {
  const int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * kBlock;
  for (int64_t i = tid; i < p.total; i += nthreads) {
    int64_t rem = i, io = 0, oo = 0;
#pragma unroll
    for (int d = kMaxRank - 1; d >= 0; d--) {
      if (d < p.rank) {
        const int64_t q = rem / p.dims[d];
        const int64_t r = rem - q * p.dims[d];
        io += r * p.is[d];
        oo += r * p.os[d];
        rem = q;
      }
    }
    out[oo] = in[io];
  }
}

// 32-bit index arithmetic for boxes below 2^31 elements (the usual case).
template <typename E>
__global__ void __launch_bounds__(kBlock) strided_copy32_kernel(const E* __restrict__ in, E* __restrict__ out, CopyPlan p) {
  const uint32_t tid = blockIdx.x * kBlock + threadIdx.x;
  const uint32_t nthreads = gridDim.x * kBlock;
  const uint32_t total = (uint32_t)p.total;
  for (uint32_t i = tid; i < total; i += nthreads) {
    uint32_t rem = i;
    int64_t io = 0, oo = 0;
#pragma unroll
    for (int d = kMaxRank - 1; d >= 0; d--) {
      if (d < p.rank) {
        const uint32_t dim = (uint32_t)p.dims[d];
        const uint32_t q = rem / dim;
        const uint32_t r = rem - q * dim;
        io += (int64_t)r * p.is[d];
        oo += (int64_t)r * p.os[d];
        rem = q;
      }
    }
    out[oo] = in[io];
  }
}

// A permutation whose innermost result index is not the innermost source index: 64 x 64
// tiles over (dt = the index that is contiguous in the source, last = the index that is
// contiguous in the result) staged through LDS so that both sides move whole rows; the other
// indices are enumerated by blockIdx.z.
struct TilePlan {
  int nouter;                  // indices other than dt and last
  int64_t n_dt, n_last, is_last, os_dt;
  int64_t dims[kMaxRank], is[kMaxRank], os[kMaxRank];
};

template <typename E>
__global__ void __launch_bounds__(kBlock) tiled_permute_kernel(const E* __restrict__ in, E* __restrict__ out, TilePlan p,
                                                               int vec_ok) {
  constexpr int TS = 64, PADW = TS + (sizeof(E) == 1 ? 4 : sizeof(E) == 2 ? 2 : 1);
  __shared__ E tile[TS][PADW];
  int64_t rem = blockIdx.z, ib = 0, ob = 0;
#pragma unroll
  for (int d = kMaxRank - 1; d >= 0; d--) {
    if (d < p.nouter) {
      const int64_t q = rem / p.dims[d], r = rem - q * p.dims[d];
      ib += r * p.is[d];
      ob += r * p.os[d];
      rem = q;
    }
  }
  in += ib;
  out += ob;
  const int64_t r0 = (int64_t)blockIdx.y * TS, c0 = (int64_t)blockIdx.x * TS;   // r: last index, c: dt index
  const int t = threadIdx.x;
  if (vec_ok && r0 + TS <= p.n_last && c0 + TS <= p.n_dt) {
    constexpr int V = 16 / sizeof(E);
    constexpr int CPR = TS / V;
#pragma unroll
    for (int i = 0; i < TS * CPR / kBlock; i++) {
      const int idx = t + i * kBlock, r = idx / CPR, c = (idx % CPR) * V;
      const uint4 v = *reinterpret_cast<const uint4*>(in + (r0 + r) * p.is_last + c0 + c);
      const E* e = reinterpret_cast<const E*>(&v);
#pragma unroll
      for (int j = 0; j < V; j++) tile[r][c + j] = e[j];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TS * CPR / kBlock; i++) {
      const int idx = t + i * kBlock, c = idx / CPR, r = (idx % CPR) * V;
      uint4 v;
      E* e = reinterpret_cast<E*>(&v);
#pragma unroll
      for (int j = 0; j < V; j++) e[j] = tile[r + j][c];
      *reinterpret_cast<uint4*>(out + (c0 + c) * p.os_dt + r0 + r) = v;
    }
  } else {
    for (int idx = t; idx < TS * TS; idx += kBlock) {
      const int r = idx / TS, c = idx % TS;
      if (r0 + r < p.n_last && c0 + c < p.n_dt) tile[r][c] = in[(r0 + r) * p.is_last + c0 + c];
    }
    __syncthreads();
    for (int idx = t; idx < TS * TS; idx += kBlock) {
      const int c = idx / TS, r = idx % TS;
      if (r0 + r < p.n_last && c0 + c < p.n_dt) out[(c0 + c) * p.os_dt + r0 + r] = tile[r][c];
    }
  }
}

// The same permutation on whole 16-byte pieces (2- and 4-byte elements, n_dt and n_last multiples of V = 16 /
// sizeof(E)) without LDS: a thread owns a V x V block over (last, dt), reads V pieces, transposes the block in
// registers and writes V pieces; the lanes of a wavefront form an 8 x 8 grid of blocks, so every access
// instruction covers whole 128-byte lines.
template <typename E, bool STREAM>
__global__ void __launch_bounds__(kBlock) block_permute_kernel(const E* __restrict__ in, E* __restrict__ out, TilePlan p) {
  constexpr int V = 16 / sizeof(E);
  static_assert(V == 4 || V == 8, "2- or 4-byte elements");
  int64_t rem = blockIdx.z, ib = 0, ob = 0;
#pragma unroll
  for (int d = kMaxRank - 1; d >= 0; d--) {
    if (d < p.nouter) {
      const int64_t q = rem / p.dims[d], r = rem - q * p.dims[d];
      ib += r * p.is[d];
      ob += r * p.os[d];
      rem = q;
    }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // blocks that run at the same time differ in both block coordinates, so that with power-of-two row lengths their
  // reads and their writes do not all fall on the same few memory channels
  const unsigned by = (blockIdx.y + blockIdx.x) % gridDim.y;
  const int64_t r = ((int64_t)by * 2 + (wave >> 1)) * 8 * V + (lane >> 3) * V;      // r: last index, c: dt index
  const int64_t c = ((int64_t)blockIdx.x * 2 + (wave & 1)) * 8 * V + (lane & 7) * V;
  if (r >= p.n_last || c >= p.n_dt) return;
  in += ib;
  out += ob;
  uint32_t x[V][4], y[V][4];
#pragma unroll
  for (int i = 0; i < V; i++) {
    const uint4 v = STREAM ? stream_load(reinterpret_cast<const uint4*>(in + (r + i) * p.is_last + c))
                           : *reinterpret_cast<const uint4*>(in + (r + i) * p.is_last + c);
    x[i][0] = v.x; x[i][1] = v.y; x[i][2] = v.z; x[i][3] = v.w;
  }
  if constexpr (V == 4) {
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int i = 0; i < 4; i++) y[j][i] = x[i][j];
  } else {
    // 16-bit elements: dword k of output row j holds source rows 2k and 2k + 1 at column j
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
    if (STREAM) stream_store(reinterpret_cast<uint4*>(out + (c + j) * p.os_dt + r), make_uint4(y[j][0], y[j][1], y[j][2], y[j][3]));
    else *reinterpret_cast<uint4*>(out + (c + j) * p.os_dt + r) = make_uint4(y[j][0], y[j][1], y[j][2], y[j][3]);
  }
}

// Tries the tiled form; returns false when the plan does not have it (then the generic
// kernel runs).
template <typename E>
bool launch_tiled(hipStream_t st, const void* in, void* out, const CopyPlan& p, int* status) {
  const int l = p.rank - 1;
  if (p.rank < 2 || p.os[l] != 1 || p.is[l] == 1 || p.is[l] == 0) return false;
  int dt = -1;
  for (int d = 0; d < l; d++)
    if (p.is[d] == 1 && p.dims[d] >= 16) dt = d;
  if (dt < 0 || p.dims[l] < 16) return false;
  TilePlan t;
  t.nouter = 0;
  t.n_dt = p.dims[dt];
  t.n_last = p.dims[l];
  t.is_last = p.is[l];
  t.os_dt = p.os[dt];
  int64_t nz = 1;
  for (int d = 0; d < l; d++) {
    if (d == dt) continue;
    t.dims[t.nouter] = p.dims[d];
    t.is[t.nouter] = p.is[d];
    t.os[t.nouter] = p.os[d];
    t.nouter++;
    nz *= p.dims[d];
  }
  for (int d = t.nouter; d < kMaxRank; d++) { t.dims[d] = 1; t.is[d] = 0; t.os[d] = 0; }
  const int64_t gx = (t.n_dt + 63) / 64, gy = (t.n_last + 63) / 64;
  if (nz > 65535 || gy > 65535) return false;
  constexpr int V = 16 / sizeof(E);
  int vec_ok = sizeof(E) <= 4 && al16(in) && al16(out) && t.is_last % V == 0 && t.os_dt % V == 0;
  for (int d = 0; d < t.nouter && vec_ok; d++) vec_ok = t.is[d] % V == 0 && t.os[d] % V == 0;
  if constexpr (sizeof(E) == 2 || sizeof(E) == 4) {
    if (vec_ok && t.n_dt % V == 0 && t.n_last % V == 0 && kBlock == 256) {
      const int64_t bx = (t.n_dt + 16 * V - 1) / (16 * V), by = (t.n_last + 16 * V - 1) / (16 * V);
      // operands beyond 128 MiB stream through (non-temporal accesses); smaller ones (weights) are read again soon
      if (p.total * (int64_t)sizeof(E) > (int64_t)(128 << 20))
        hipLaunchKernelGGL((block_permute_kernel<E, true>), dim3((unsigned)bx, (unsigned)by, (unsigned)nz), dim3(kBlock), 0, st,
                           static_cast<const E*>(in), static_cast<E*>(out), t);
      else
        hipLaunchKernelGGL((block_permute_kernel<E, false>), dim3((unsigned)bx, (unsigned)by, (unsigned)nz), dim3(kBlock), 0, st,
                           static_cast<const E*>(in), static_cast<E*>(out), t);
      hipError_t eb = hipGetLastError();
      *status = eb == hipSuccess ? EMI_OK : emi_fail(EMI_INTERNAL, "emi_strided_copy: launch failed: %s", hipGetErrorString(eb));
      return true;
    }
  }
  hipLaunchKernelGGL(tiled_permute_kernel<E>, dim3((unsigned)gx, (unsigned)gy, (unsigned)nz), dim3(kBlock), 0, st,
                     static_cast<const E*>(in), static_cast<E*>(out), t, vec_ok);
  hipError_t e = hipGetLastError();
  *status = e == hipSuccess ? EMI_OK : emi_fail(EMI_INTERNAL, "emi_strided_copy: launch failed: %s", hipGetErrorString(e));
  return true;
}

// Rows of whole 16-byte chunks, contiguous on both sides (row broadcast: source row stride 0; slices and
// concatenations along the slow index): one chunk per thread, blockIdx.y = row, no index divisions.  The result
// is written with streaming stores; a broadcast source is read through the cache (every row reads it again).
__global__ void __launch_bounds__(kBlock) row_copy_kernel(const uint4* __restrict__ in, uint4* __restrict__ out, int64_t chunks,
                                                          int64_t is_row, int64_t os_row) {
  const int64_t c = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (c >= chunks) return;
  const uint4* src = in + (int64_t)blockIdx.y * is_row + c;
  const uint4 v = is_row == 0 ? *src : stream_load(src);
  stream_store(out + (int64_t)blockIdx.y * os_row + c, v);
}

template <typename E>
int launch_copy(hipStream_t st, const void* in, void* out, const CopyPlan& p) {
  int status = EMI_OK;
  if constexpr (sizeof(E) == 16) {
    if (p.rank == 2 && p.is[1] == 1 && p.os[1] == 1 && p.dims[1] >= 64 && p.dims[0] <= 65535) {
      hipLaunchKernelGGL(row_copy_kernel, dim3((unsigned)((p.dims[1] + kBlock - 1) / kBlock), (unsigned)p.dims[0]), dim3(kBlock), 0, st,
                         static_cast<const uint4*>(in), static_cast<uint4*>(out), p.dims[1], p.is[0], p.os[0]);
      EMI_CHECK_LAUNCH("emi_strided_copy");
      return EMI_OK;
    }
  }
  if constexpr (sizeof(E) <= 8) {
    if (launch_tiled<E>(st, in, out, p, &status)) return status;
  }
  const unsigned grid = grid_for(p.total, kBlock);
  if (p.total < 0x7fffffffLL)
    hipLaunchKernelGGL(strided_copy32_kernel<E>, dim3(grid), dim3(kBlock), 0, st, static_cast<const E*>(in),
                       static_cast<E*>(out), p);
  else
    hipLaunchKernelGGL(strided_copy_kernel<E>, dim3(grid), dim3(kBlock), 0, st, static_cast<const E*>(in),
                       static_cast<E*>(out), p);
  EMI_CHECK_LAUNCH("emi_strided_copy");
  return EMI_OK;
}

// ---------------------------------------------------------------------------
// reductions over the middle index of x[outer, red, inner] (sum or max, fp32 accumulate)
// ---------------------------------------------------------------------------
template <int OP> __device__ __forceinline__ float red_init() { return OP == EMI_OP_ADD ? 0.0f : -INFINITY; }
template <int OP> __device__ __forceinline__ float red_op(float a, float b) {
  if (OP == EMI_OP_ADD) return a + b;
  return (a != a || b != b) ? (a + b) : fmaxf(a, b);
}
template <int OP> __device__ __forceinline__ float wave_red(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = red_op<OP>(v, __shfl_xor(v, o, kWave));
  return v;
}

// inner == 1.  Row `row` of x is split into `nsplit` segments of `seg` elements; workgroup
// (row, s) reduces segment s with WAVES waves, lanes striding over 16-byte chunks (VEC: the
// segments start 16-byte aligned) or elements, and writes either the result (nsplit == 1,
// TO = T) or an fp32 partial [row, s] for the second stage.
template <typename T, typename TO, int OP, int WAVES, bool VEC>
__global__ void __launch_bounds__(WAVES * kWave) reduce_rows_kernel(const T* __restrict__ x, TO* __restrict__ y,
                                                                    int64_t rows, int64_t red, int64_t seg, int nsplit) {
  constexpr int N = Chunk<T>::N;
  __shared__ float part[WAVES];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int64_t item = blockIdx.x; item < rows * nsplit; item += gridDim.x) {
    const int64_t row = item / nsplit, sidx = item - row * nsplit;
    const int64_t lo = sidx * seg, hi = lo + seg < red ? lo + seg : red;
    const T* xr = x + row * red + lo;
    const int64_t len = hi - lo;
    float a0 = red_init<OP>(), a1 = a0;
    if (VEC) {
      const int64_t nchunks = len / N;
      typename Chunk<T>::Raw r0, r1;
      float v[N];
      int64_t c = threadIdx.x;
      for (; c + WAVES * kWave < nchunks; c += 2 * WAVES * kWave) {       // two loads in flight
        r0 = Chunk<T>::load_raw(xr + c * N);
        r1 = Chunk<T>::load_raw(xr + (c + WAVES * kWave) * N);
        Chunk<T>::unpack(r0, v);
#pragma unroll
        for (int j = 0; j < N; j++) a0 = red_op<OP>(a0, v[j]);
        Chunk<T>::unpack(r1, v);
#pragma unroll
        for (int j = 0; j < N; j++) a1 = red_op<OP>(a1, v[j]);
      }
      if (c < nchunks) {
        Chunk<T>::load(xr + c * N, v);
#pragma unroll
        for (int j = 0; j < N; j++) a0 = red_op<OP>(a0, v[j]);
      }
      for (int64_t i = nchunks * N + threadIdx.x; i < len; i += WAVES * kWave) a1 = red_op<OP>(a1, to_f32(xr[i]));
    } else {
      for (int64_t i = threadIdx.x; i < len; i += WAVES * kWave) a0 = red_op<OP>(a0, to_f32(xr[i]));
    }
    float acc = wave_red<OP>(red_op<OP>(a0, a1));
    if (WAVES > 1) {
      __syncthreads();
      if (lane == 0) part[wave] = acc;
      __syncthreads();
      acc = part[0];
#pragma unroll
      for (int w = 1; w < WAVES; w++) acc = red_op<OP>(acc, part[w]);
    }
    if (threadIdx.x == 0) y[item] = from_f32<TO>(acc);
  }
}

// inner > 1: x [outer, red, inner].  Lane = one 16-byte chunk of columns (VEC) or one column;
// blockIdx.y = band of `band` rows, blockIdx.z = outer.  Writes the result (nsplit == 1) or
// an fp32 partial [band, outer, inner].
template <typename T, typename TO, int OP, bool VEC>
__global__ void __launch_bounds__(kBlock) reduce_cols_kernel(const T* __restrict__ x, TO* __restrict__ y, int64_t outer,
                                                             int64_t red, int64_t inner, int64_t band) {
  constexpr int N = VEC ? Chunk<T>::N : 1;
  const int64_t col = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * N;
  if (col >= inner) return;
  const int64_t o = blockIdx.z, r0 = (int64_t)blockIdx.y * band, r1 = r0 + band < red ? r0 + band : red;
  const T* p = x + (o * red + r0) * inner + col;
  float acc[N], acc2[N];
#pragma unroll
  for (int j = 0; j < N; j++) acc[j] = acc2[j] = red_init<OP>();
  int64_t r = r0;
  if (VEC) {
    float v[Chunk<T>::N];
    constexpr int UN = 8;                                   // row loads in flight per lane
    for (; r + UN <= r1; r += UN) {
      typename Chunk<T>::Raw q[UN];
#pragma unroll
      for (int u = 0; u < UN; u++) q[u] = Chunk<T>::load_raw(p + u * inner);
      p += UN * inner;
#pragma unroll
      for (int u = 0; u < UN; u++) {
        Chunk<T>::unpack(q[u], v);
        if (u & 1) {
#pragma unroll
          for (int j = 0; j < N; j++) acc2[j] = red_op<OP>(acc2[j], v[j]);
        } else {
#pragma unroll
          for (int j = 0; j < N; j++) acc[j] = red_op<OP>(acc[j], v[j]);
        }
      }
    }
    for (; r < r1; r++, p += inner) {
      Chunk<T>::load(p, v);
#pragma unroll
      for (int j = 0; j < N; j++) acc[j] = red_op<OP>(acc[j], v[j]);
    }
  } else {
    for (; r < r1; r++, p += inner) acc[0] = red_op<OP>(acc[0], to_f32(*p));
  }
  TO* yp = y + ((int64_t)blockIdx.y * outer + o) * inner + col;
#pragma unroll
  for (int j = 0; j < N; j++) yp[j] = from_f32<TO>(red_op<OP>(acc[j], acc2[j]));
}

// second stage of the column form: y[m] = reduce over s of part[s, m].  A workgroup owns 64
// columns; its 16 waves take the partial rows s = wave, wave + 16, ... with eight loads in
// flight each and meet in LDS, so the pass costs a few round trips to memory, not nsplit.
template <typename T, int OP>
__global__ void __launch_bounds__(1024) reduce_partials_kernel(const float* __restrict__ part, T* __restrict__ y,
                                                               int64_t m, int nsplit) {
  __shared__ float sh[16][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t i = (int64_t)blockIdx.x * 64 + lane;
  float acc = red_init<OP>();
  if (i < m) {
    int s = wave;
    for (; s + 7 * 16 < nsplit; s += 8 * 16) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = part[(int64_t)(s + u * 16) * m + i];
#pragma unroll
      for (int u = 0; u < 8; u++) acc = red_op<OP>(acc, v[u]);
    }
    for (; s < nsplit; s += 16) acc = red_op<OP>(acc, part[(int64_t)s * m + i]);
  }
  sh[wave][lane] = acc;
  __syncthreads();
  if (wave == 0 && i < m) {
#pragma unroll
    for (int w = 1; w < 16; w++) acc = red_op<OP>(acc, sh[w][lane]);
    y[i] = from_f32<T>(acc);
  }
}

struct ReducePlan {
  int nsplit;          // 1: single pass
  int64_t seg;         // rows form: elements per segment; column form: rows per band
};

// Enough workgroups to fill 256 CUs a few times over; segments keep 16-byte alignment.
template <typename T>
ReducePlan reduce_plan(int64_t outer, int64_t red, int64_t inner) {
  ReducePlan p{1, red};
  const int64_t want = 2048;
  if (inner == 1) {
    if (outer >= want / 2 || red < 16384) return p;
    int64_t ns = (want + outer - 1) / outer;
    int64_t seg = (red + ns - 1) / ns;
    seg = (seg + 1023) / 1024 * 1024;                       // multiple of every chunk size
    if (seg < 8192) seg = 8192;
    ns = (red + seg - 1) / seg;
    if (ns > 1) { p.nsplit = (int)ns; p.seg = seg; }
  } else {
    // Bands of rows, one block each per 256-lane strip of columns: as many blocks as CUs (long bands: a band's fixed
    // costs are paid once per 256+ rows; one more block than CUs would double the time), times four where a strip has
    // a single wavefront of columns, times two where it has two.
    const int64_t lanes = (inner + Chunk<T>::N - 1) / Chunk<T>::N;
    const int64_t blocks = ((lanes + kBlock - 1) / kBlock) * outer;
    const int64_t strip_waves = ((lanes < kBlock ? lanes : kBlock) + 63) / 64;
    const int64_t target = 256 * ((4 + strip_waves - 1) / strip_waves);
    if (2 * blocks > target || red < 64) return p;
    int64_t ns = target / blocks;
    int64_t band = (red + ns - 1) / ns;
    if (band < 64) band = 64;
    ns = (red + band - 1) / band;
    if (ns > 1) { p.nsplit = (int)ns; p.seg = band; }
  }
  return p;
}

template <typename T>
size_t reduce_workspace(int64_t outer, int64_t red, int64_t inner) {
  const ReducePlan p = reduce_plan<T>(outer, red, inner);
  return p.nsplit == 1 ? 0 : (size_t)p.nsplit * (size_t)outer * (size_t)inner * sizeof(float);
}

template <typename T, typename TO, int OP>
void launch_rows(hipStream_t st, const T* x, TO* y, int64_t rows, int64_t red, int64_t seg, int nsplit) {
  const int64_t items = rows * nsplit;
  const unsigned grid = (unsigned)(items < 262144 ? items : 262144);
  const bool vec = al16(x) && red % Chunk<T>::N == 0 && seg % Chunk<T>::N == 0;
  const int64_t chunks = seg / Chunk<T>::N;
#define EMI_ROWS(W)                                                                                              \
  do {                                                                                                           \
    if (vec) hipLaunchKernelGGL((reduce_rows_kernel<T, TO, OP, W, true>), dim3(grid), dim3(W * 64), 0, st, x, y, rows, red, seg, nsplit); \
    else hipLaunchKernelGGL((reduce_rows_kernel<T, TO, OP, W, false>), dim3(grid), dim3(W * 64), 0, st, x, y, rows, red, seg, nsplit);   \
  } while (0)
  if (chunks <= 128) EMI_ROWS(1);
  else if (chunks <= 1024) EMI_ROWS(4);
  else EMI_ROWS(16);
#undef EMI_ROWS
}

template <typename T, int OP>
int launch_reduce(hipStream_t st, const void* x, void* y, void* ws, size_t ws_bytes, int64_t outer, int64_t red,
                  int64_t inner) {
  const T* xp = static_cast<const T*>(x);
  T* yp = static_cast<T*>(y);
  ReducePlan p = reduce_plan<T>(outer, red, inner);
  if (p.nsplit > 1 && (ws == nullptr || ws_bytes < reduce_workspace<T>(outer, red, inner))) p = ReducePlan{1, red};
  float* part = static_cast<float*>(ws);
  if (inner == 1) {
    if (p.nsplit == 1) {
      launch_rows<T, T, OP>(st, xp, yp, outer, red, red, 1);
    } else {
      launch_rows<T, float, OP>(st, xp, part, outer, red, p.seg, p.nsplit);
      EMI_CHECK_LAUNCH("emi_reduce");
      launch_rows<float, T, OP>(st, part, yp, outer, p.nsplit, p.nsplit, 1);
    }
  } else {
    const bool vec = al16(x) && inner % Chunk<T>::N == 0;
    const int64_t lanes = vec ? inner / Chunk<T>::N : inner;
    const dim3 grid((unsigned)((lanes + kBlock - 1) / kBlock), (unsigned)p.nsplit, (unsigned)outer);
    if (p.nsplit == 1) {
      if (vec) hipLaunchKernelGGL((reduce_cols_kernel<T, T, OP, true>), grid, dim3(kBlock), 0, st, xp, yp, outer, red, inner, red);
      else hipLaunchKernelGGL((reduce_cols_kernel<T, T, OP, false>), grid, dim3(kBlock), 0, st, xp, yp, outer, red, inner, red);
    } else {
      if (vec) hipLaunchKernelGGL((reduce_cols_kernel<T, float, OP, true>), grid, dim3(kBlock), 0, st, xp, part, outer, red, inner, p.seg);
      else hipLaunchKernelGGL((reduce_cols_kernel<T, float, OP, false>), grid, dim3(kBlock), 0, st, xp, part, outer, red, inner, p.seg);
      EMI_CHECK_LAUNCH("emi_reduce");
      const int64_t m = outer * inner;
      hipLaunchKernelGGL((reduce_partials_kernel<T, OP>), dim3((unsigned)((m + 63) / 64)), dim3(1024), 0, st, part, yp, m,
                         p.nsplit);
    }
  }
  EMI_CHECK_LAUNCH("emi_reduce");
  return EMI_OK;
}

template <typename T, bool VEC>
int launch_binary_op(hipStream_t st, int op, unsigned grid, const T* a, const T* b, T* y, int64_t n, int sa, int sb) {
#define EMI_BIN(OP)                                                                                              \
  case OP:                                                                                                       \
    hipLaunchKernelGGL((map_binary_kernel<T, VEC, OP>), dim3(grid), dim3(kBlock), 0, st, a, b, y, n, sa, sb);  \
    break;
  switch (op) {
    EMI_BIN(EMI_OP_ADD) EMI_BIN(EMI_OP_SUB) EMI_BIN(EMI_OP_MUL) EMI_BIN(EMI_OP_DIV) EMI_BIN(EMI_OP_MAX)
    EMI_BIN(EMI_OP_MIN) EMI_BIN(EMI_OP_GE) EMI_BIN(EMI_OP_EQ) EMI_BIN(EMI_OP_NMUL) EMI_BIN(EMI_OP_POW)
    EMI_BIN(EMI_OP_D_SQRT) EMI_BIN(EMI_OP_D_RSQRT) EMI_BIN(EMI_OP_D_LOGISTIC) EMI_BIN(EMI_OP_D_TANH)
    EMI_BIN(EMI_OP_D_SIN) EMI_BIN(EMI_OP_D_COS) EMI_BIN(EMI_OP_D_POW_A) EMI_BIN(EMI_OP_D_POW_B)
    EMI_BIN(EMI_OP_D_ABS) EMI_BIN(EMI_OP_D_LOG1P) EMI_BIN(EMI_OP_D_EXPM1) EMI_BIN(EMI_OP_D_CBRT) EMI_BIN(EMI_OP_ATAN2)
    default: return emi_fail(EMI_INVALID_ARGUMENT, "emi_map_binary: unknown operator code %d", op);
  }
#undef EMI_BIN
  EMI_CHECK_LAUNCH("emi_map_binary");
  return EMI_OK;
}

template <typename T>
int launch_binary(hipStream_t st, int op, const void* a, const void* b, void* y, int64_t n, int sa, int sb) {
  const bool vec = al16(a) && al16(b) && al16(y);
  const unsigned grid = piece_grid(n, vec, map_pieces<T>() * Chunk<T>::N);
  const T* ap = static_cast<const T*>(a);
  const T* bp = static_cast<const T*>(b);
  T* yp = static_cast<T*>(y);
  return vec ? launch_binary_op<T, true>(st, op, grid, ap, bp, yp, n, sa, sb)
             : launch_binary_op<T, false>(st, op, grid, ap, bp, yp, n, sa, sb);
}

template <typename T, bool VEC>
int launch_unary_op(hipStream_t st, int op, unsigned grid, const T* x, T* y, int64_t n) {
#define EMI_UN(OP)                                                                                  \
  case OP:                                                                                          \
    hipLaunchKernelGGL((map_unary_kernel<T, VEC, OP>), dim3(grid), dim3(kBlock), 0, st, x, y, n); \
    break;
  switch (op) {
    EMI_UN(EMI_OP_NEG) EMI_UN(EMI_OP_EXP) EMI_UN(EMI_OP_LOG) EMI_UN(EMI_OP_SQRT) EMI_UN(EMI_OP_RSQRT)
    EMI_UN(EMI_OP_LOGISTIC) EMI_UN(EMI_OP_TANH) EMI_UN(EMI_OP_SIN) EMI_UN(EMI_OP_COS) EMI_UN(EMI_OP_ABS)
    EMI_UN(EMI_OP_COPY) EMI_UN(EMI_OP_LOG1P) EMI_UN(EMI_OP_EXPM1) EMI_UN(EMI_OP_CBRT)
    default: return emi_fail(EMI_INVALID_ARGUMENT, "emi_map_unary: unknown operator code %d", op);
  }
#undef EMI_UN
  EMI_CHECK_LAUNCH("emi_map_unary");
  return EMI_OK;
}

template <typename T>
int launch_unary(hipStream_t st, int op, const void* x, void* y, int64_t n) {
  const bool vec = al16(x) && al16(y);
  const unsigned grid = piece_grid(n, vec, map_pieces<T>() * Chunk<T>::N);
  const T* xp = static_cast<const T*>(x);
  T* yp = static_cast<T*>(y);
  return vec ? launch_unary_op<T, true>(st, op, grid, xp, yp, n) : launch_unary_op<T, false>(st, op, grid, xp, yp, n);
}

template <typename TI, typename TO>
int launch_convert(hipStream_t st, const void* x, void* y, int64_t n) {
  const bool vec = al16(x) && al16(y);
  const unsigned grid = map_grid(n, vec);
  if (vec)
    hipLaunchKernelGGL((convert_kernel<TI, TO, true>), dim3(grid), dim3(kBlock), 0, st, static_cast<const TI*>(x),
                       static_cast<TO*>(y), n);
  else
    hipLaunchKernelGGL((convert_kernel<TI, TO, false>), dim3(grid), dim3(kBlock), 0, st, static_cast<const TI*>(x),
                       static_cast<TO*>(y), n);
  EMI_CHECK_LAUNCH("emi_convert");
  return EMI_OK;
}

}  // namespace
}  // namespace emi

using namespace emi;

extern "C" int emi_map_binary(emi_stream_t stream, int op, const void* a, const void* b, void* y, int64_t n,
                              int a_is_scalar, int b_is_scalar, int dtype) {
  EMI_REQUIRE(op >= EMI_OP_ADD && op <= EMI_OP_ATAN2, "emi_map_binary: unknown operator code %d", op);
  EMI_REQUIRE(n >= 0 && n < (int64_t)1 << 39, "emi_map_binary: size out of range");
  if (n == 0) return EMI_OK;
  EMI_REQUIRE(a && b && y, "emi_map_binary: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int sa = a_is_scalar ? 0 : 1, sb = b_is_scalar ? 0 : 1;
  switch (dtype) {
    case EMI_F32: return launch_binary<float>(st, op, a, b, y, n, sa, sb);
    case EMI_BF16: return launch_binary<bf16>(st, op, a, b, y, n, sa, sb);
    default: return emi_fail(EMI_INVALID_ARGUMENT, "emi_map_binary: unsupported dtype code %d", dtype);
  }
}

extern "C" int emi_map_unary(emi_stream_t stream, int op, const void* x, void* y, int64_t n, int dtype) {
  EMI_REQUIRE(op >= EMI_OP_NEG && op <= EMI_OP_CBRT, "emi_map_unary: unknown operator code %d", op);
  EMI_REQUIRE(n >= 0 && n < (int64_t)1 << 39, "emi_map_unary: size out of range");
  if (n == 0) return EMI_OK;
  EMI_REQUIRE(x && y, "emi_map_unary: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case EMI_F32: return launch_unary<float>(st, op, x, y, n);
    case EMI_BF16: return launch_unary<bf16>(st, op, x, y, n);
    default: return emi_fail(EMI_INVALID_ARGUMENT, "emi_map_unary: unsupported dtype code %d", dtype);
  }
}

extern "C" int emi_convert(emi_stream_t stream, const void* x, void* y, int64_t n, int from_dtype, int to_dtype) {
  EMI_REQUIRE(n >= 0 && n < (int64_t)1 << 39, "emi_convert: size out of range");
  if (n == 0) return EMI_OK;
  EMI_REQUIRE(x && y, "emi_convert: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (from_dtype == EMI_F32 && to_dtype == EMI_BF16) return launch_convert<float, bf16>(st, x, y, n);
  if (from_dtype == EMI_BF16 && to_dtype == EMI_F32) return launch_convert<bf16, float>(st, x, y, n);
  if (from_dtype == EMI_F32 && to_dtype == EMI_F32) return launch_convert<float, float>(st, x, y, n);
  if (from_dtype == EMI_BF16 && to_dtype == EMI_BF16) return launch_convert<bf16, bf16>(st, x, y, n);
  return emi_fail(EMI_INVALID_ARGUMENT, "emi_convert: unsupported dtype codes %d -> %d", from_dtype, to_dtype);
}

extern "C" int emi_strided_copy(emi_stream_t stream, const void* in, void* out, int rank, const int64_t* dims,
                                const int64_t* in_strides, int64_t in_offset, const int64_t* out_strides,
                                int64_t out_offset, int elem_bytes) {
  EMI_REQUIRE(rank >= 0 && rank <= kMaxRank, "emi_strided_copy: rank %d (at most %d)", rank, kMaxRank);
  EMI_REQUIRE(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8, "emi_strided_copy: element size %d",
              elem_bytes);
  EMI_REQUIRE(rank == 0 || (dims && in_strides && out_strides), "emi_strided_copy: null shape");
  EMI_REQUIRE(in_offset >= 0 && out_offset >= 0, "emi_strided_copy: negative offset");
  int64_t total = 1;
  for (int d = 0; d < rank; d++) {
    EMI_REQUIRE(dims[d] >= 0 && in_strides[d] >= 0 && out_strides[d] >= 0, "emi_strided_copy: negative size or stride");
    total *= dims[d];
  }
  if (total == 0) return EMI_OK;
  EMI_REQUIRE(in && out, "emi_strided_copy: null buffer");
  // drop unit dimensions, merge neighbours that are contiguous on both sides
  CopyPlan p;
  p.rank = 0;
  p.total = total;
  for (int d = 0; d < rank; d++) {
    if (dims[d] == 1) continue;
    if (p.rank > 0 && p.is[p.rank - 1] == in_strides[d] * dims[d] && p.os[p.rank - 1] == out_strides[d] * dims[d]) {
      p.dims[p.rank - 1] *= dims[d];
      p.is[p.rank - 1] = in_strides[d];
      p.os[p.rank - 1] = out_strides[d];
    } else {
      p.dims[p.rank] = dims[d];
      p.is[p.rank] = in_strides[d];
      p.os[p.rank] = out_strides[d];
      p.rank++;
    }
  }
  for (int d = p.rank; d < kMaxRank; d++) { p.dims[d] = 1; p.is[d] = 0; p.os[d] = 0; }
  if (p.rank == 0) { p.rank = 1; }
  const char* ip = static_cast<const char*>(in) + in_offset * elem_bytes;
  char* op = static_cast<char*>(out) + out_offset * elem_bytes;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // 16-byte chunks when the innermost index is contiguous on both sides and everything
  // else is a multiple of the chunk
  const int N = 16 / elem_bytes;
  const int l = p.rank - 1;
  bool vec = p.is[l] == 1 && p.os[l] == 1 && p.dims[l] % N == 0 && al16(ip) && al16(op);
  for (int d = 0; d < l && vec; d++) vec = p.is[d] % N == 0 && p.os[d] % N == 0;
  if (vec) {
    CopyPlan q = p;
    q.dims[l] /= N;
    q.total /= N;
    for (int d = 0; d < l; d++) { q.is[d] /= N; q.os[d] /= N; }
    return launch_copy<uint4>(st, ip, op, q);
  }
  if (elem_bytes == 1) return launch_copy<uint8_t>(st, ip, op, p);
  if (elem_bytes == 2) return launch_copy<uint16_t>(st, ip, op, p);
  if (elem_bytes == 4) return launch_copy<uint32_t>(st, ip, op, p);
  return launch_copy<uint64_t>(st, ip, op, p);
}

extern "C" size_t emi_reduce_workspace_bytes(int64_t outer, int64_t red, int64_t inner, int dtype) {
  if (outer <= 0 || red <= 0 || inner <= 0) return 0;
  return dtype == EMI_BF16 ? reduce_workspace<bf16>(outer, red, inner) : reduce_workspace<float>(outer, red, inner);
}

extern "C" int emi_reduce(emi_stream_t stream, int op, const void* x, void* y, void* workspace, size_t workspace_bytes,
                          int64_t outer, int64_t red, int64_t inner, int dtype) {
  EMI_REQUIRE(op == EMI_OP_ADD || op == EMI_OP_MAX, "emi_reduce: operator code %d (want add or max)", op);
  EMI_REQUIRE(outer >= 0 && red > 0 && inner > 0, "emi_reduce: bad shape [%lld, %lld, %lld]", (long long)outer,
              (long long)red, (long long)inner);
  EMI_REQUIRE(outer <= 65535 || inner == 1, "emi_reduce: more than 65535 outer slices with inner > 1");
  if (outer == 0) return EMI_OK;
  EMI_REQUIRE(x && y, "emi_reduce: null buffer");
  EMI_REQUIRE(workspace == nullptr || al16(workspace), "emi_reduce: workspace must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == EMI_F32)
    return op == EMI_OP_ADD ? launch_reduce<float, EMI_OP_ADD>(st, x, y, workspace, workspace_bytes, outer, red, inner)
                            : launch_reduce<float, EMI_OP_MAX>(st, x, y, workspace, workspace_bytes, outer, red, inner);
  if (dtype == EMI_BF16)
    return op == EMI_OP_ADD ? launch_reduce<bf16, EMI_OP_ADD>(st, x, y, workspace, workspace_bytes, outer, red, inner)
                            : launch_reduce<bf16, EMI_OP_MAX>(st, x, y, workspace, workspace_bytes, outer, red, inner);
  return emi_fail(EMI_INVALID_ARGUMENT, "emi_reduce: unsupported dtype code %d", dtype);
}

extern "C" int emi_compare(emi_stream_t stream, int direction, const void* a, const void* b, void* mask, int64_t n,
                           int a_is_scalar, int b_is_scalar, int dtype) {
  EMI_REQUIRE(direction >= EMI_CMP_EQ && direction <= EMI_CMP_LT, "emi_compare: unknown direction code %d", direction);
  EMI_REQUIRE(n >= 0 && n < (int64_t)1 << 39, "emi_compare: size out of range");
  if (n == 0) return EMI_OK;
  EMI_REQUIRE(a && b && mask, "emi_compare: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int sa = a_is_scalar ? 0 : 1, sb = b_is_scalar ? 0 : 1;
  const bool vec = al16(a) && al16(b) && (reinterpret_cast<uintptr_t>(mask) & 7) == 0;
  const unsigned grid = piece_grid(n, vec, 16);
#define EMI_CMP_LAUNCH(T)                                                                                             \
  do {                                                                                                                 \
    if (vec) hipLaunchKernelGGL((compare_kernel<T, true>), dim3(grid), dim3(kBlock), 0, st, direction, (const T*)a, (const T*)b, (uint8_t*)mask, n, sa, sb); \
    else hipLaunchKernelGGL((compare_kernel<T, false>), dim3(grid), dim3(kBlock), 0, st, direction, (const T*)a, (const T*)b, (uint8_t*)mask, n, sa, sb);    \
  } while (0)
  if (dtype == EMI_F32) EMI_CMP_LAUNCH(float);
  else if (dtype == EMI_BF16) EMI_CMP_LAUNCH(bf16);
  else return emi_fail(EMI_INVALID_ARGUMENT, "emi_compare: unsupported dtype code %d", dtype);
#undef EMI_CMP_LAUNCH
  EMI_CHECK_LAUNCH("emi_compare");
  return EMI_OK;
}

extern "C" int emi_select(emi_stream_t stream, const void* mask, const void* a, const void* b, void* y, int64_t n,
                          int mask_is_scalar, int a_is_scalar, int b_is_scalar, int dtype) {
  EMI_REQUIRE(n >= 0 && n < (int64_t)1 << 39, "emi_select: size out of range");
  if (n == 0) return EMI_OK;
  EMI_REQUIRE(mask && a && b && y, "emi_select: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int sm = mask_is_scalar ? 0 : 1, sa = a_is_scalar ? 0 : 1, sb = b_is_scalar ? 0 : 1;
  const bool vec = al16(a) && al16(b) && al16(y) && (reinterpret_cast<uintptr_t>(mask) & 7) == 0;
  const unsigned grid = piece_grid(n, vec, 16);
#define EMI_SEL_LAUNCH(T)                                                                                             \
  do {                                                                                                                 \
    if (vec) hipLaunchKernelGGL((select_kernel<T, true>), dim3(grid), dim3(kBlock), 0, st, (const uint8_t*)mask, (const T*)a, (const T*)b, (T*)y, n, sm, sa, sb); \
    else hipLaunchKernelGGL((select_kernel<T, false>), dim3(grid), dim3(kBlock), 0, st, (const uint8_t*)mask, (const T*)a, (const T*)b, (T*)y, n, sm, sa, sb);    \
  } while (0)
  if (dtype == EMI_F32) EMI_SEL_LAUNCH(float);
  else if (dtype == EMI_BF16) EMI_SEL_LAUNCH(bf16);
  else return emi_fail(EMI_INVALID_ARGUMENT, "emi_select: unsupported dtype code %d", dtype);
#undef EMI_SEL_LAUNCH
  EMI_CHECK_LAUNCH("emi_select");
  return EMI_OK;
}
