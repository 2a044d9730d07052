// Skinny GEMMs of the single-token (decode) form of the llama step, all HBM-bound on
// the weight matrix, which is read (or written) exactly once:
//   mat-vec        y = W x            test/llama.py:149-157,211,224-233  (NT, M <= 8)
//   its adjoints   dx = dy W          HLODerivatives.td:1166-1170        (NN, M <= 8)
//                  dW = dy^T x                                           (TN, K <= 8)
// emi_gemm routes here when the token dimension is at most 8; fp32 accumulation,
// one rounding, optional residual like the large kernels.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "emi_device.h"

namespace emi {
namespace {

// y[m][n] = sum_k A[m][k] B[n][k] (+ R[m][n]).  A row n of B streams through in batches of UN 16-byte chunks per lane
// (8 KB of a bf16 row); SPLIT wavefronts of a block share a row (batch b goes to wavefront b mod SPLIT) and meet in LDS,
// so that a matrix of few long rows still puts thousands of wavefronts' loads in flight.  A wavefront issues the loads
// of its next batch before it sums the current one.  The loads are unconditional (a chunk past the end of the row is
// read from the row's start and multiplied by zero): guarded loads made the compiler wait for all earlier ones before
// each.  A (M x K, a few KB) comes from cache; AREG: one row of A and K of one batch, A stays in registers.
// STREAM: B is read with streaming loads (a weight that is larger than the caches).
template <typename T, int MT, int SPLIT, bool AREG, bool STREAM>
__global__ __launch_bounds__(256) void gemv_nt_kernel(const T* __restrict__ A, const T* __restrict__ B, const T* R, T* C, int M,
                                                      int N, int K, int64_t lda, int64_t ldb, int64_t ldr, int64_t ldc) {
  using BC = std::conditional_t<STREAM, Chunk<T>, ChunkCached<T>>;
  using Raw = typename ChunkCached<T>::Raw;
  constexpr int V = ChunkCached<T>::N;
  constexpr int UN = 8;                      // 16-byte loads of a row in flight per lane and batch
  constexpr int BATCH = 64 * V * UN;         // elements of a row per batch
  static_assert(!AREG || (MT == 1 && SPLIT == 1), "A in registers: one row of A, one batch");
  __shared__ float red[4][MT];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = wave % SPLIT;
  const int row = blockIdx.x * (4 / SPLIT) + wave / SPLIT;
  const bool live = row < N;
  const int nb = (K + BATCH - 1) / BATCH;
  float acc[MT];
#pragma unroll
  for (int m = 0; m < MT; m++) acc[m] = 0.f;
  if (live) {
    const T* brow = B + (int64_t)row * ldb;
    Raw areg[AREG ? UN : 1];
    if constexpr (AREG) {
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int k = lane * V + u * 64 * V;
        areg[u] = ChunkCached<T>::load_raw(A + (k < K ? k : 0));
      }
    }
    auto issue = [&](int b, Raw(&r)[UN]) {
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int k = b * BATCH + lane * V + u * 64 * V;
        r[u] = BC::load_raw(brow + (k < K ? k : 0));
      }
    };
    // one row of A: its chunks of a batch are requested before the loads of the next batch of B, whose arrival
    // (the memory counter is in order) the sum would otherwise wait for
    auto load_a = [&](int b, Raw(&ra)[UN]) {
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int k = b * BATCH + lane * V + u * 64 * V;
        ra[u] = ChunkCached<T>::load_raw(A + (k < K ? k : 0));
      }
    };
    constexpr bool APRE = MT == 1 && !AREG;
    Raw ra[APRE ? UN : 1];
    auto consume = [&](int b, const Raw(&r)[UN]) {
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int k = b * BATCH + lane * V + u * 64 * V;
        const bool ok = k < K;
        float bv[V];
        ChunkCached<T>::unpack(r[u], bv);
#pragma unroll
        for (int e = 0; e < V; e++) bv[e] = ok ? bv[e] : 0.f;
#pragma unroll
        for (int m = 0; m < MT; m++) {
          if (m < M) {
            float a[V];
            if constexpr (AREG) ChunkCached<T>::unpack(areg[u], a);
            else if constexpr (APRE) ChunkCached<T>::unpack(ra[u], a);
            else ChunkCached<T>::load(A + (int64_t)m * lda + (ok ? k : 0), a);
#pragma unroll
            for (int e = 0; e < V; e++) acc[m] = fmaf(ok ? a[e] : 0.f, bv[e], acc[m]);
          }
        }
      }
    };
    Raw r0[UN], r1[UN];
    int b = sub;
    if (b < nb) issue(b, r0);
    while (b < nb) {
      const int b1 = b + SPLIT;
      if constexpr (APRE) load_a(b, ra);
      if (b1 < nb) issue(b1, r1);
      consume(b, r0);
      if (b1 >= nb) break;
      b = b1 + SPLIT;
      if constexpr (APRE) load_a(b1, ra);
      if (b < nb) issue(b, r0);
      consume(b1, r1);
    }
#pragma unroll
    for (int m = 0; m < MT; m++) acc[m] = wave_sum(acc[m]);
  }
  if constexpr (SPLIT > 1) {
    if (lane == 0) {
#pragma unroll
      for (int m = 0; m < MT; m++) red[wave][m] = acc[m];
    }
    __syncthreads();
    if (sub == 0 && lane == 0) {
#pragma unroll
      for (int m = 0; m < MT; m++) {
        acc[m] = 0.f;
#pragma unroll
        for (int w = 0; w < SPLIT; w++) acc[m] += red[wave + w][m];      // in wavefront order: the result does not depend on timing
      }
    }
  }
  if (live && sub == 0 && lane == 0) {
#pragma unroll
    for (int m = 0; m < MT; m++)
      if (m < M) {
        float v = acc[m];
        if (R != nullptr) v += to_f32(R[(int64_t)m * ldr + row]);
        C[(int64_t)m * ldc + row] = from_f32<T>(v);
      }
  }
}

// y[m][n] = sum_k A[m][k] B[k][n] (+ R): a block owns 8 chunks = 128 bytes of every row of B
// (8 lanes side by side) and its 128 row-lanes walk down the K rows with UN loads in flight
// each (a block must keep tens of KB in flight: there are only N / 64 of them); the partial
// sums meet through lane shuffles and LDS.  No atomics: the result does not depend on the
// launch.
template <typename T, int MT>
__global__ __launch_bounds__(1024) void gemv_nn_kernel(const T* __restrict__ A, const T* __restrict__ B, const T* R, T* C, int M,
                                                       int N, int K, int64_t lda, int64_t ldb, int64_t ldr, int64_t ldc) {
  constexpr int V = ChunkCached<T>::N, UN = MT * V > 32 ? 4 : 8, ROWS = 128;
  __shared__ float part[16][MT][8 * V];
  const int cl = threadIdx.x & 7, rl = threadIdx.x >> 3;           // chunk lane, row lane (0..127)
  const int n = (blockIdx.x * 8 + cl) * V;
  float acc[MT][V];
#pragma unroll
  for (int m = 0; m < MT; m++)
#pragma unroll
    for (int e = 0; e < V; e++) acc[m][e] = 0.f;
  if (n < N) {
    for (int k0 = rl; k0 < K; k0 += ROWS * UN) {
      float b[UN][V];
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int k = k0 + u * ROWS;
        if (k < K) ChunkCached<T>::load(B + (int64_t)k * ldb + n, b[u]);
      }
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int k = k0 + u * ROWS;
        if (k < K) {
#pragma unroll
          for (int m = 0; m < MT; m++) {
            if (m < M) {
              const float a = to_f32(A[(int64_t)m * lda + k]);
#pragma unroll
              for (int e = 0; e < V; e++) acc[m][e] = fmaf(a, b[u][e], acc[m][e]);
            }
          }
        }
      }
    }
  }
  // the 8 row lanes of a wavefront differ in lane bits 3..5; then the 16 wavefronts meet in LDS
#pragma unroll
  for (int m = 0; m < MT; m++)
#pragma unroll
    for (int e = 0; e < V; e++) {
      float v = acc[m][e];
      v += __shfl_xor(v, 8, kWave);
      v += __shfl_xor(v, 16, kWave);
      v += __shfl_xor(v, 32, kWave);
      if ((threadIdx.x & 63) < 8) part[threadIdx.x >> 6][m][cl * V + e] = v;
    }
  __syncthreads();
  for (int idx = threadIdx.x; idx < MT * 8 * V; idx += 1024) {
    const int m = idx / (8 * V), c = idx % (8 * V);
    const int col = blockIdx.x * 8 * V + c;
    if (m < M && col < N) {
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < 16; w++) v += part[w][m][c];
      if (R != nullptr) v += to_f32(R[(int64_t)m * ldr + col]);
      C[(int64_t)m * ldc + col] = from_f32<T>(v);
    }
  }
}

// The same product with a workspace: the K rows are cut into bands, a block sums one band
// for 256 chunks of columns (every row it reads is one contiguous run), writes fp32
// partials [band][m][n], and a second kernel adds the bands in order.  Hundreds of blocks
// instead of N / 64, and no 8 KB strides inside a wavefront.
template <typename T, int MT>
__global__ __launch_bounds__(256) void gemv_nn_bands_kernel(const T* __restrict__ A, const T* __restrict__ B,
                                                            float* __restrict__ part, int M, int N, int K, int64_t lda,
                                                            int64_t ldb, int rows_per_band) {
  using Raw = typename ChunkCached<T>::Raw;
  constexpr int V = ChunkCached<T>::N, UN = 8, AR = 256;
  __shared__ float sa[MT][AR + 2 * UN];                           // A values of the rows being processed, then zeros
  const int n = (blockIdx.x * 256 + threadIdx.x) * V;
  const int k_begin = blockIdx.y * rows_per_band;
  const int k_end = k_begin + rows_per_band < K ? k_begin + rows_per_band : K;
  const bool live = n < N;
  const T* bcol = B + (live ? n : 0);
  float acc[MT][V];
#pragma unroll
  for (int m = 0; m < MT; m++)
#pragma unroll
    for (int e = 0; e < V; e++) acc[m][e] = 0.f;
  // Unconditional loads (a row past the band is read from the band's last row and meets a zero of A): guarded
  // loads made the compiler wait for all earlier ones before each.  The next UN rows are requested before the
  // current ones are summed.
  auto issue = [&](int k0, Raw(&r)[UN]) {
#pragma unroll
    for (int u = 0; u < UN; u++) {
      const int k = k0 + u < k_end ? k0 + u : k_end - 1;
      r[u] = Chunk<T>::load_raw(bcol + (int64_t)k * ldb);
    }
  };
  auto consume = [&](int j0, const Raw(&r)[UN]) {                 // j0: index of the first row within sa
#pragma unroll
    for (int u = 0; u < UN; u++) {
      float bf[V];
      ChunkCached<T>::unpack(r[u], bf);
#pragma unroll
      for (int m = 0; m < MT; m++)
        if (m < M) {
          const float a = sa[m][j0 + u];
#pragma unroll
          for (int e = 0; e < V; e++) acc[m][e] = fmaf(a, bf[e], acc[m][e]);
        }
    }
  };
  for (int kc = k_begin; kc < k_end; kc += AR) {
    __syncthreads();
    for (int j = threadIdx.x; j < AR + 2 * UN; j += 256)
#pragma unroll
      for (int m = 0; m < MT; m++)
        if (m < M) sa[m][j] = (j < AR && kc + j < k_end) ? to_f32(A[(int64_t)m * lda + kc + j]) : 0.f;
    __syncthreads();
    const int kce = kc + AR < k_end ? kc + AR : k_end;
    Raw r0[UN], r1[UN];
    int k0 = kc;
    issue(k0, r0);
    while (k0 < kce) {
      const int k1 = k0 + UN;
      if (k1 < kce) issue(k1, r1);
      consume(k0 - kc, r0);
      if (k1 >= kce) break;
      k0 = k1 + UN;
      if (k0 < kce) issue(k0, r0);
      consume(k1 - kc, r1);
    }
  }
  if (!live) return;
#pragma unroll
  for (int m = 0; m < MT; m++)
    if (m < M) {
      float* dst = part + ((int64_t)blockIdx.y * M + m) * N + n;
#pragma unroll
      for (int e = 0; e < V; e += 4) *reinterpret_cast<float4*>(dst + e) = make_float4(acc[m][e], acc[m][e + 1], acc[m][e + 2], acc[m][e + 3]);
    }
}

// C[m][n] = sum over bands (in a fixed order) + R: 16 columns (64 bytes of a partial row) per block, 16 band
// lanes with up to 16 loads in flight each, so 256 bands are one round trip; the lanes meet through LDS.
template <typename T>
__global__ __launch_bounds__(256) void gemv_bands_reduce_kernel(const float* __restrict__ part, const T* R, T* C, int M, int N,
                                                                int bands, int64_t ldr, int64_t ldc) {
  constexpr int BL = 16, UN = 16;
  __shared__ float red[BL][16];
  const int col = threadIdx.x & 15, bl = threadIdx.x >> 4;
  const int64_t i = blockIdx.x * (int64_t)16 + col;               // index into [M][N]
  const bool live = i < (int64_t)M * N;
  float v = 0.f;
  if (live) {
    const float* p = part + i;
    const int64_t bstride = (int64_t)M * N;
    for (int b0 = bl; b0 < bands; b0 += BL * UN) {
      float t[UN];
#pragma unroll
      for (int u = 0; u < UN; u++) t[u] = b0 + BL * u < bands ? p[(int64_t)(b0 + BL * u) * bstride] : 0.f;
#pragma unroll
      for (int u = 0; u < UN; u++) v += t[u];
    }
  }
  red[bl][col] = v;
  __syncthreads();
  if (bl == 0 && live) {
    const int m = (int)(i / N), n = (int)(i % N);
    v = 0.f;
#pragma unroll
    for (int b = 0; b < BL; b++) v += red[b][col];
    if (R != nullptr) v += to_f32(R[(int64_t)m * ldr + n]);
    C[(int64_t)m * ldc + n] = from_f32<T>(v);
  }
}

// Number of row bands for the workspace form (the same in the size query and the launch).
int nn_bands(int64_t N, int64_t K, int V) {
  const int64_t colgroups = (N / V + 255) / 256;
  int64_t bands = (256 + colgroups - 1) / colgroups;             // one block per CU measured best (19.5 us against 21.3 and 25.1
  if (bands > 256) bands = 256;                                  // for two and four on [11008, 4096])
  if (bands > (K + 7) / 8) bands = (K + 7) / 8;
  return (int)(bands < 1 ? 1 : bands);
}

// C[m][n] = sum_{k < K <= 8} A[k][m] B[k][n] (+ R): a sum of K outer products, one 16-byte
// store per thread; bound by the write of C.
template <typename T, bool STREAM>
__global__ __launch_bounds__(256) void outer_tn_kernel(const T* __restrict__ A, const T* __restrict__ B, const T* R, T* C, int M,
                                                       int N, int K, int64_t lda, int64_t ldb, int64_t ldr, int64_t ldc) {
  constexpr int V = ChunkCached<T>::N;
  const int chunks = N / V;
  const int64_t total = (int64_t)M * chunks;
  for (int64_t i = blockIdx.x * (int64_t)256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int m = (int)(i / chunks), n = (int)(i % chunks) * V;
    float acc[V];
    if (R != nullptr) ChunkCached<T>::load(R + (int64_t)m * ldr + n, acc);
    else {
#pragma unroll
      for (int e = 0; e < V; e++) acc[e] = 0.f;
    }
    for (int k = 0; k < K; k++) {
      const float a = to_f32(A[(int64_t)k * lda + m]);
      float b[V];
      ChunkCached<T>::load(B + (int64_t)k * ldb + n, b);
#pragma unroll
      for (int e = 0; e < V; e++) acc[e] = fmaf(a, b[e], acc[e]);
    }
    if constexpr (STREAM) Chunk<T>::store(C + (int64_t)m * ldc + n, acc);
    else ChunkCached<T>::store(C + (int64_t)m * ldc + n, acc);
  }
}

bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T>
int launch_skinny_t(hipStream_t st, const void* A_, const void* B_, const void* R_, void* C_, void* workspace,
                    size_t workspace_bytes, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldr, int64_t ldc,
                    int trans_a, int trans_b) {
  constexpr int V = ChunkCached<T>::N;
  const T* A = static_cast<const T*>(A_);
  const T* B = static_cast<const T*>(B_);
  const T* R = static_cast<const T*>(R_);
  T* C = static_cast<T*>(C_);
#define EMI_SKINNY_MT(KERNEL, GRID, BLOCK)                                                                              \
  do {                                                                                                                  \
    if (M <= 1) hipLaunchKernelGGL((KERNEL<T, 1>), GRID, dim3(BLOCK), 0, st, A, B, R, C, (int)M, (int)N, (int)K, lda, ldb, ldr, ldc); \
    else if (M <= 2) hipLaunchKernelGGL((KERNEL<T, 2>), GRID, dim3(BLOCK), 0, st, A, B, R, C, (int)M, (int)N, (int)K, lda, ldb, ldr, ldc); \
    else if (M <= 4) hipLaunchKernelGGL((KERNEL<T, 4>), GRID, dim3(BLOCK), 0, st, A, B, R, C, (int)M, (int)N, (int)K, lda, ldb, ldr, ldc); \
    else hipLaunchKernelGGL((KERNEL<T, 8>), GRID, dim3(BLOCK), 0, st, A, B, R, C, (int)M, (int)N, (int)K, lda, ldb, ldr, ldc); \
  } while (0)
  if (!trans_a && trans_b) {                 // mat-vec: 16-byte chunks along K of both operands
    if (M > 8 || K % V || lda % V || ldb % V || !al16(A) || !al16(B)) return -1;
    // wavefronts per row: enough of them that about 8192 are in flight, at most one per batch of the row
    constexpr int kBatch = 64 * V * 8;
    const int64_t nbat = (K + kBatch - 1) / kBatch;
    int split = 1;
    while (split < 4 && N * split < 8192 && split < nbat) split *= 2;
    const dim3 grid((unsigned)((N * split + 3) / 4));
    const bool stream = (size_t)N * (size_t)K * sizeof(T) > ((size_t)32 << 20);
#define EMI_GEMV_NT_L(MT, SPLIT, AREG)                                                                                         \
  do {                                                                                                                         \
    if (stream)                                                                                                                \
      hipLaunchKernelGGL((gemv_nt_kernel<T, MT, SPLIT, AREG, true>), grid, dim3(256), 0, st, A, B, R, C, (int)M, (int)N, (int)K, lda, \
                         ldb, ldr, ldc);                                                                                       \
    else                                                                                                                       \
      hipLaunchKernelGGL((gemv_nt_kernel<T, MT, SPLIT, AREG, false>), grid, dim3(256), 0, st, A, B, R, C, (int)M, (int)N, (int)K, lda, \
                         ldb, ldr, ldc);                                                                                       \
  } while (0)
#define EMI_GEMV_NT(MT)                                    \
  do {                                                     \
    if (split == 4) EMI_GEMV_NT_L(MT, 4, false);           \
    else if (split == 2) EMI_GEMV_NT_L(MT, 2, false);      \
    else EMI_GEMV_NT_L(MT, 1, false);                      \
  } while (0)
    // (a variant that kept the vector in registers over several rows per wavefront measured the same: 17.5-18.8 us
    // for 1 to 11 rows against 17.8 us on [11008, 4096])
    if (M <= 1 && split == 1 && nbat == 1) EMI_GEMV_NT_L(1, 1, true);
    else if (M <= 1) EMI_GEMV_NT(1);
    else if (M <= 2) EMI_GEMV_NT(2);
    else if (M <= 4) EMI_GEMV_NT(4);
    else EMI_GEMV_NT(8);
#undef EMI_GEMV_NT
#undef EMI_GEMV_NT_L
  } else if (!trans_a && !trans_b) {         // 16-byte chunks along N of B
    if (M > 8 || N % V || ldb % V || !al16(B)) return -1;
    const int bands = nn_bands(N, K, V);
    if (workspace != nullptr && al16(workspace) && workspace_bytes >= (size_t)bands * M * N * sizeof(float) && bands > 1) {
      const int rpb = (int)((K + bands - 1) / bands);
      const dim3 grid((unsigned)((N / V + 255) / 256), (unsigned)bands);
      float* part = static_cast<float*>(workspace);
#define EMI_BANDS(MT)                                                                                                   \
  hipLaunchKernelGGL((gemv_nn_bands_kernel<T, MT>), grid, dim3(256), 0, st, A, B, part, (int)M, (int)N, (int)K, lda, ldb, rpb)
      if (M <= 1) EMI_BANDS(1);
      else if (M <= 2) EMI_BANDS(2);
      else if (M <= 4) EMI_BANDS(4);
      else EMI_BANDS(8);
#undef EMI_BANDS
      EMI_CHECK_LAUNCH("emi_gemm(skinny bands)");
      hipLaunchKernelGGL(gemv_bands_reduce_kernel<T>, dim3((unsigned)((M * N + 15) / 16)), dim3(256), 0, st, part, R, C, (int)M,
                         (int)N, bands, ldr, ldc);
    } else {
      EMI_SKINNY_MT(gemv_nn_kernel, dim3((unsigned)((N / V + 7) / 8)), 1024);
    }
  } else if (trans_a && !trans_b) {          // outer products: 16-byte chunks along N of B, C (and R)
    if (K > 8 || N % V || ldb % V || ldc % V || !al16(B) || !al16(C) || (R != nullptr && (ldr % V || !al16(R)))) return -1;
    const int64_t total = M * (N / V);
    const unsigned grid = (unsigned)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
    if ((size_t)M * (size_t)N * sizeof(T) > ((size_t)32 << 20))       // a result larger than the caches: streaming stores
      hipLaunchKernelGGL((outer_tn_kernel<T, true>), dim3(grid), dim3(256), 0, st, A, B, R, C, (int)M, (int)N, (int)K, lda, ldb, ldr, ldc);
    else
      hipLaunchKernelGGL((outer_tn_kernel<T, false>), dim3(grid), dim3(256), 0, st, A, B, R, C, (int)M, (int)N, (int)K, lda, ldb, ldr, ldc);
  } else {
    return -1;
  }
#undef EMI_SKINNY_MT
  EMI_CHECK_LAUNCH("emi_gemm(skinny)");
  return EMI_OK;
}

}  // namespace

// Returns -1 when the shape is not one of the skinny forms (the caller then takes the tiled
// kernels), otherwise a status code.
int launch_skinny(hipStream_t st, const void* A, const void* B, const void* R, void* C, void* workspace, size_t workspace_bytes,
                  int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldr, int64_t ldc, int trans_a, int trans_b,
                  int dtype) {
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return -1;
  if (dtype == EMI_BF16)
    return launch_skinny_t<bf16>(st, A, B, R, C, workspace, workspace_bytes, M, N, K, lda, ldb, ldr, ldc, trans_a, trans_b);
  return launch_skinny_t<float>(st, A, B, R, C, workspace, workspace_bytes, M, N, K, lda, ldb, ldr, ldc, trans_a, trans_b);
}

// Bytes of workspace with which the skinny NN form runs its banded kernel (0: none useful).
size_t skinny_workspace_bytes(int64_t M, int64_t N, int64_t K, int trans_a, int trans_b, int dtype) {
  if (trans_a || trans_b || M < 1 || M > 8 || N < 1 || K < 1) return 0;
  const int V = dtype == EMI_BF16 ? 8 : 4;
  if (N % V) return 0;
  const int bands = nn_bands(N, K, V);
  return bands > 1 ? (size_t)bands * M * N * sizeof(float) : 0;
}

}  // namespace emi
