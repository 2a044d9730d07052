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
    default: return 0.0f;
  }
}

// y[i] = op(a[i * sa], b[i * sb]); sa, sb in {0, 1} (0: the operand is one element).
// VEC: chunks of 16 bytes per lane over the first n - n % N elements, lane-serial tail.
template <typename T, bool VEC, int OP>
__global__ void __launch_bounds__(kBlock) map_binary_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                            T* __restrict__ y, int64_t n, int sa, int sb) {
  constexpr int N = Chunk<T>::N;
  const int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * kBlock;
  if (VEC) {
    const int64_t nchunks = n / N;
    float fa[N], fb[N], fy[N];
    if (!sa) { const float s = to_f32(a[0]);
#pragma unroll
      for (int j = 0; j < N; j++) fa[j] = s; }
    if (!sb) { const float s = to_f32(b[0]);
#pragma unroll
      for (int j = 0; j < N; j++) fb[j] = s; }
    for (int64_t c = tid; c < nchunks; c += nthreads) {
      if (sa) Chunk<T>::load(a + c * N, fa);
      if (sb) Chunk<T>::load(b + c * N, fb);
#pragma unroll
      for (int j = 0; j < N; j++) fy[j] = apply_binary<OP>(fa[j], fb[j]);
      Chunk<T>::store(y + c * N, fy);
    }
    const int64_t i = nchunks * N + tid;
    if (i < n) y[i] = from_f32<T>(apply_binary<OP>(to_f32(a[sa ? i : 0]), to_f32(b[sb ? i : 0])));
  } else {
    for (int64_t i = tid; i < n; i += nthreads)
      y[i] = from_f32<T>(apply_binary<OP>(to_f32(a[sa ? i : 0]), to_f32(b[sb ? i : 0])));
  }
}

template <typename T, bool VEC, int OP>
__global__ void __launch_bounds__(kBlock) map_unary_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n) {
  constexpr int N = Chunk<T>::N;
  const int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * kBlock;
  if (VEC) {
    const int64_t nchunks = n / N;
    float fx[N], fy[N];
    for (int64_t c = tid; c < nchunks; c += nthreads) {
      Chunk<T>::load(x + c * N, fx);
#pragma unroll
      for (int j = 0; j < N; j++) fy[j] = apply_unary<OP>(fx[j]);
      Chunk<T>::store(y + c * N, fy);
    }
    const int64_t i = nchunks * N + tid;
    if (i < n) y[i] = from_f32<T>(apply_unary<OP>(to_f32(x[i])));
  } else {
    for (int64_t i = tid; i < n; i += nthreads) y[i] = from_f32<T>(apply_unary<OP>(to_f32(x[i])));
  }
}

template <typename TI, typename TO>
__global__ void __launch_bounds__(kBlock) convert_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t n) {
  const int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * kBlock;
  const int64_t nchunks = n / 8;
  float v[8];
  for (int64_t c = tid; c < nchunks; c += nthreads) {
    Vec8<TI>::load(x + c * 8, v);
    Vec8<TO>::store(y + c * 8, v);
  }
  const int64_t i = nchunks * 8 + tid;
  if (i < n) y[i] = from_f32<TO>(to_f32(x[i]));
}

template <typename TI, typename TO>
__global__ void __launch_bounds__(kBlock) convert_scalar_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t n) {
  const int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  for (int64_t i = tid; i < n; i += (int64_t)gridDim.x * kBlock) y[i] = from_f32<TO>(to_f32(x[i]));
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

template <typename E>
int launch_copy(hipStream_t st, const void* in, void* out, const CopyPlan& p) {
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

// inner == 1: one workgroup of WAVES waves per row; lanes stride over 16-byte chunks when the
// rows are 16-byte aligned (VEC), elements otherwise.
template <typename T, int OP, int WAVES, bool VEC>
__global__ void __launch_bounds__(WAVES * kWave) reduce_rows_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                    int64_t rows, int64_t red) {
  constexpr int N = Chunk<T>::N;
  __shared__ float part[WAVES];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const T* xr = x + row * red;
    float acc = red_init<OP>();
    if (VEC) {
      const int64_t nchunks = red / N;
      float v[N];
      for (int64_t c = threadIdx.x; c < nchunks; c += WAVES * kWave) {
        Chunk<T>::load(xr + c * N, v);
#pragma unroll
        for (int j = 0; j < N; j++) acc = red_op<OP>(acc, v[j]);
      }
    } else {
      for (int64_t i = threadIdx.x; i < red; i += WAVES * kWave) acc = red_op<OP>(acc, to_f32(xr[i]));
    }
    acc = wave_red<OP>(acc);
    if (WAVES > 1) {
      __syncthreads();
      if (lane == 0) part[wave] = acc;
      __syncthreads();
      acc = part[0];
#pragma unroll
      for (int w = 1; w < WAVES; w++) acc = red_op<OP>(acc, part[w]);
    }
    if (threadIdx.x == 0) y[row] = from_f32<T>(acc);
  }
}

// inner > 1: one lane per (outer, inner) result, coalesced over inner.
template <typename T, int OP>
__global__ void __launch_bounds__(kBlock) reduce_cols_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t outer,
                                                             int64_t red, int64_t inner) {
  const int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t total = outer * inner;
  for (int64_t i = tid; i < total; i += (int64_t)gridDim.x * kBlock) {
    const int64_t o = i / inner, c = i - o * inner;
    const T* p = x + o * red * inner + c;
    float a0 = red_init<OP>(), a1 = a0, a2 = a0, a3 = a0;
    int64_t r = 0;
    for (; r + 4 <= red; r += 4) {
      a0 = red_op<OP>(a0, to_f32(p[(r + 0) * inner]));
      a1 = red_op<OP>(a1, to_f32(p[(r + 1) * inner]));
      a2 = red_op<OP>(a2, to_f32(p[(r + 2) * inner]));
      a3 = red_op<OP>(a3, to_f32(p[(r + 3) * inner]));
    }
    for (; r < red; r++) a0 = red_op<OP>(a0, to_f32(p[r * inner]));
    y[i] = from_f32<T>(red_op<OP>(red_op<OP>(a0, a1), red_op<OP>(a2, a3)));
  }
}

template <typename T, int OP>
int launch_reduce(hipStream_t st, const void* x, void* y, int64_t outer, int64_t red, int64_t inner) {
  const T* xp = static_cast<const T*>(x);
  T* yp = static_cast<T*>(y);
  if (inner == 1) {
    const bool vec = al16(x) && red % Chunk<T>::N == 0;
    const unsigned grid = (unsigned)(outer < 65536 ? outer : 65536);
    if (red <= 2048) {
      if (vec) hipLaunchKernelGGL((reduce_rows_kernel<T, OP, 1, true>), dim3(grid), dim3(64), 0, st, xp, yp, outer, red);
      else hipLaunchKernelGGL((reduce_rows_kernel<T, OP, 1, false>), dim3(grid), dim3(64), 0, st, xp, yp, outer, red);
    } else {
      if (vec) hipLaunchKernelGGL((reduce_rows_kernel<T, OP, 16, true>), dim3(grid), dim3(1024), 0, st, xp, yp, outer, red);
      else hipLaunchKernelGGL((reduce_rows_kernel<T, OP, 16, false>), dim3(grid), dim3(1024), 0, st, xp, yp, outer, red);
    }
  } else {
    hipLaunchKernelGGL((reduce_cols_kernel<T, OP>), dim3(grid_for(outer * inner, kBlock)), dim3(kBlock), 0, st, xp, yp,
                       outer, red, inner);
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
    default: return emi_fail(EMI_INVALID_ARGUMENT, "emi_map_binary: unknown operator code %d", op);
  }
#undef EMI_BIN
  EMI_CHECK_LAUNCH("emi_map_binary");
  return EMI_OK;
}

template <typename T>
int launch_binary(hipStream_t st, int op, const void* a, const void* b, void* y, int64_t n, int sa, int sb) {
  const bool vec = al16(a) && al16(b) && al16(y) && n >= Chunk<T>::N;
  const unsigned grid = grid_for(vec ? n / Chunk<T>::N : n, kBlock);
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
    EMI_UN(EMI_OP_COPY)
    default: return emi_fail(EMI_INVALID_ARGUMENT, "emi_map_unary: unknown operator code %d", op);
  }
#undef EMI_UN
  EMI_CHECK_LAUNCH("emi_map_unary");
  return EMI_OK;
}

template <typename T>
int launch_unary(hipStream_t st, int op, const void* x, void* y, int64_t n) {
  const bool vec = al16(x) && al16(y) && n >= Chunk<T>::N;
  const unsigned grid = grid_for(vec ? n / Chunk<T>::N : n, kBlock);
  const T* xp = static_cast<const T*>(x);
  T* yp = static_cast<T*>(y);
  return vec ? launch_unary_op<T, true>(st, op, grid, xp, yp, n) : launch_unary_op<T, false>(st, op, grid, xp, yp, n);
}

template <typename TI, typename TO>
int launch_convert(hipStream_t st, const void* x, void* y, int64_t n) {
  const bool vec = al16(x) && al16(y) && n >= 8;
  if (vec)
    hipLaunchKernelGGL((convert_kernel<TI, TO>), dim3(grid_for(n / 8, kBlock)), dim3(kBlock), 0, st,
                       static_cast<const TI*>(x), static_cast<TO*>(y), n);
  else
    hipLaunchKernelGGL((convert_scalar_kernel<TI, TO>), dim3(grid_for(n, kBlock)), dim3(kBlock), 0, st,
                       static_cast<const TI*>(x), static_cast<TO*>(y), n);
  EMI_CHECK_LAUNCH("emi_convert");
  return EMI_OK;
}

}  // namespace
}  // namespace emi

using namespace emi;

extern "C" int emi_map_binary(emi_stream_t stream, int op, const void* a, const void* b, void* y, int64_t n,
                              int a_is_scalar, int b_is_scalar, int dtype) {
  EMI_REQUIRE(op >= EMI_OP_ADD && op <= EMI_OP_D_POW_B, "emi_map_binary: unknown operator code %d", op);
  EMI_REQUIRE(n >= 0, "emi_map_binary: negative size");
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
  EMI_REQUIRE(op >= EMI_OP_NEG && op <= EMI_OP_COPY, "emi_map_unary: unknown operator code %d", op);
  EMI_REQUIRE(n >= 0, "emi_map_unary: negative size");
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
  EMI_REQUIRE(n >= 0, "emi_convert: negative size");
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
  EMI_REQUIRE(elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8, "emi_strided_copy: element size %d", elem_bytes);
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
  if (elem_bytes == 2) return launch_copy<uint16_t>(st, ip, op, p);
  if (elem_bytes == 4) return launch_copy<uint32_t>(st, ip, op, p);
  return launch_copy<uint64_t>(st, ip, op, p);
}

extern "C" int emi_reduce(emi_stream_t stream, int op, const void* x, void* y, int64_t outer, int64_t red,
                          int64_t inner, int dtype) {
  EMI_REQUIRE(op == EMI_OP_ADD || op == EMI_OP_MAX, "emi_reduce: operator code %d (want add or max)", op);
  EMI_REQUIRE(outer >= 0 && red > 0 && inner > 0, "emi_reduce: bad shape [%lld, %lld, %lld]", (long long)outer,
              (long long)red, (long long)inner);
  if (outer == 0) return EMI_OK;
  EMI_REQUIRE(x && y, "emi_reduce: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == EMI_F32)
    return op == EMI_OP_ADD ? launch_reduce<float, EMI_OP_ADD>(st, x, y, outer, red, inner)
                            : launch_reduce<float, EMI_OP_MAX>(st, x, y, outer, red, inner);
  if (dtype == EMI_BF16)
    return op == EMI_OP_ADD ? launch_reduce<bf16, EMI_OP_ADD>(st, x, y, outer, red, inner)
                            : launch_reduce<bf16, EMI_OP_MAX>(st, x, y, outer, red, inner);
  return emi_fail(EMI_INVALID_ARGUMENT, "emi_reduce: unsupported dtype code %d", dtype);
}
