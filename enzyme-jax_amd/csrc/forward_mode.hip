// Forward-mode (tangent) kernels of the operators that are not linear in their
// inputs: RMSNorm, SwiGLU and softmax attention.  The linear ones (projections, RoPE,
// residual adds, gather) push tangents through their own forward kernels.  The reference
// selects forward mode by rewriting the pass pipeline (enzyme_jvp,
// src/enzyme_ad/jax/primitives.py:1147-1245); the per-op tangent rules are the forward halves
// of the HLODerivatives.td entries cited at each kernel.  A null tangent pointer means zero.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "emi_device.h"

namespace emi {
namespace {

__device__ __forceinline__ float block_sum256(float v, float* scratch) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  return scratch[0] + scratch[1] + scratch[2] + scratch[3];
}

// y = gamma * x * r, r = rsqrt(mean(x^2) + eps)  (test/llama.py:6-10; Mul :1221, Rsqrt :1283,
// reduce-add StableHLOAutoDiffOpInterfaceImpl.cpp:1865-1879):
//   ty = gamma * (r tx - x r^3 mean(x tx)) + tgamma * x * r
// One 256-thread block per row; the second sweep over the row comes from cache.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void rmsnorm_jvp_kernel(const T* __restrict__ x, const T* __restrict__ gamma,
                                                          const T* __restrict__ tx, const T* __restrict__ tgamma,
                                                          T* __restrict__ ty, int64_t dim, float eps) {
  __shared__ float scratch[4];
  constexpr int V = VEC ? 8 : 1;
  const int64_t row = blockIdx.x;
  const T* xr = x + row * dim;
  const T* txr = tx ? tx + row * dim : nullptr;
  float ss = 0.f, sxt = 0.f;
  for (int64_t c = (int64_t)threadIdx.x * V; c < dim; c += 256 * V) {
    float xv[8], tv[8];
    if constexpr (VEC) {
      Vec8<T>::load(xr + c, xv);
      if (txr) Vec8<T>::load(txr + c, tv);
    } else {
      xv[0] = to_f32(xr[c]);
      if (txr) tv[0] = to_f32(txr[c]);
    }
#pragma unroll
    for (int e = 0; e < V; e++) {
      ss = fmaf(xv[e], xv[e], ss);
      if (txr) sxt = fmaf(xv[e], tv[e], sxt);
    }
  }
  ss = block_sum256(ss, scratch);
  sxt = block_sum256(sxt, scratch);
  const float r = 1.0f / sqrtf(ss / (float)dim + eps);
  const float coef = r * r * r * (sxt / (float)dim);
  for (int64_t c = (int64_t)threadIdx.x * V; c < dim; c += 256 * V) {
    float xv[8], tv[8], gv[8], tg[8], out[8];
    if constexpr (VEC) {
      Vec8<T>::load(xr + c, xv);
      Vec8<T>::load(gamma + c, gv);
      if (txr) Vec8<T>::load(txr + c, tv);
      if (tgamma) Vec8<T>::load(tgamma + c, tg);
    } else {
      xv[0] = to_f32(xr[c]);
      gv[0] = to_f32(gamma[c]);
      if (txr) tv[0] = to_f32(txr[c]);
      if (tgamma) tg[0] = to_f32(tgamma[c]);
    }
#pragma unroll
    for (int e = 0; e < V; e++) {
      float o = 0.f;
      if (txr) o = gv[e] * (r * tv[e] - xv[e] * coef);
      if (tgamma) o = fmaf(tg[e], xv[e] * r, o);
      out[e] = o;
    }
    if constexpr (VEC) Vec8<T>::store(ty + row * dim + c, out);
    else ty[row * dim + c] = from_f32<T>(out[0]);
  }
}

// Same tangent with the row held in registers: every lane loads its NCH groups of eight
// elements of x and tx up front (all loads in flight together), the two row sums follow, and
// the result is written from the registers: x and tx are read from memory once.
// Needs dim % 8 == 0, dim <= 256 * 8 * NCH, 16-byte aligned rows.
template <typename T, int NCH>
__global__ __launch_bounds__(256) void rmsnorm_jvp_rows_kernel(const T* __restrict__ x, const T* __restrict__ gamma,
                                                               const T* __restrict__ tx, const T* __restrict__ tgamma,
                                                               T* __restrict__ ty, int dim, float eps) {
  __shared__ float scratch[4];
  const int64_t row = blockIdx.x;
  const T* xr = x + row * dim;
  const T* txr = tx ? tx + row * dim : nullptr;
  typename Vec8<T>::Raw xraw[NCH], traw[NCH];
#pragma unroll
  for (int c = 0; c < NCH; c++) {
    const int col = (threadIdx.x + c * 256) * 8;
    xraw[c] = col < dim ? Vec8<T>::load_raw(xr + col) : Vec8<T>::zero_raw();
    traw[c] = (txr && col < dim) ? Vec8<T>::load_raw(txr + col) : Vec8<T>::zero_raw();
  }
  float ss = 0.f, sxt = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; c++) {
    float xv[8], tv[8];
    Vec8<T>::unpack(xraw[c], xv);
    Vec8<T>::unpack(traw[c], tv);
#pragma unroll
    for (int e = 0; e < 8; e++) {
      ss = fmaf(xv[e], xv[e], ss);
      sxt = fmaf(xv[e], tv[e], sxt);
    }
  }
  ss = block_sum256(ss, scratch);
  sxt = block_sum256(sxt, scratch);
  const float r = 1.0f / sqrtf(ss / (float)dim + eps);
  const float coef = r * r * r * (sxt / (float)dim);
#pragma unroll
  for (int c = 0; c < NCH; c++) {
    const int col = (threadIdx.x + c * 256) * 8;
    if (col < dim) {
      float xv[8], tv[8], gv[8], tg[8], out[8];
      Vec8<T>::unpack(xraw[c], xv);
      Vec8<T>::unpack(traw[c], tv);
      Vec8<T>::load(gamma + col, gv);
      if (tgamma) Vec8<T>::load(tgamma + col, tg);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        float o = gv[e] * (r * tv[e] - xv[e] * coef);          // tv = 0 without tx: the term vanishes
        if (tgamma) o = fmaf(tg[e], xv[e] * r, o);
        out[e] = o;
      }
      Vec8<T>::store(ty + row * dim + col, out);
    }
  }
}

// g = a sigmoid(a) b  (test/llama.py:21-28,227-229; Mul :1221, Div :1133, Exp :1182):
//   tg = ta b s (1 + a (1 - s)) + tb a s,  s = sigmoid(a)
template <typename T>
__global__ __launch_bounds__(256) void swiglu_jvp_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                         const T* __restrict__ ta, const T* __restrict__ tb, T* __restrict__ tg,
                                                         int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t nchunks = n >> 3;
  auto one = [](float av, float bv, float tav, float tbv) {
    const float s = 1.0f / (1.0f + __expf(-av));
    return tav * bv * s * (1.0f + av * (1.0f - s)) + tbv * av * s;
  };
  if (i < nchunks) {
    float av[8], bv[8], tav[8], tbv[8], o[8];
    Vec8<T>::load(a + i * 8, av);
    Vec8<T>::load(b + i * 8, bv);
#pragma unroll
    for (int e = 0; e < 8; e++) tav[e] = 0.f, tbv[e] = 0.f;
    if (ta) Vec8<T>::load(ta + i * 8, tav);
    if (tb) Vec8<T>::load(tb + i * 8, tbv);
#pragma unroll
    for (int e = 0; e < 8; e++) o[e] = one(av[e], bv[e], tav[e], tbv[e]);
    Vec8<T>::store(tg + i * 8, o);
  } else if (i - nchunks < (n & 7)) {
    const int64_t e = (nchunks << 3) + (i - nchunks);
    tg[e] = from_f32<T>(one(to_f32(a[e]), to_f32(b[e]), ta ? to_f32(ta[e]) : 0.f, tb ? to_f32(tb[e]) : 0.f));
  }
}

struct JvpShape {
  int seq, heads;
  int64_t sb, sh, ss;
};

// o = P v, P = softmax(scale q k^T + causal mask)  (test/llama.py:13-18,178-206; DotGeneral :1166,
// Exp :1182, Div :1133, Sub :1312, reduce max/add StableHLOAutoDiffOpInterfaceImpl.cpp:1833-1916):
//   tS = scale (tq k^T + q tk^T);  tP = P (tS - rowsum(P tS));  to = tP v + P tv
//      = sum_j p_j tS_j v_j - (sum_j p_j tS_j) o + sum_j p_j tv_j,   p_j = exp(S_j - lse)
// One wavefront per query row, one key per lane and 64 keys per sweep; head_dim <= 256.
template <typename T>
__global__ __launch_bounds__(256) void attn_jvp_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                                                       const float* __restrict__ lse, const T* __restrict__ tq,
                                                       const T* __restrict__ tk, const T* __restrict__ tv, T* __restrict__ to,
                                                       JvpShape sh, int d, float scale, int causal) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int qi = blockIdx.x * 4 + wave;
  const int bh = blockIdx.y;
  if (qi >= sh.seq) return;
  const int64_t base = (int64_t)(bh / sh.heads) * sh.sb + (int64_t)(bh % sh.heads) * sh.sh;
  const T* qr = q + base + (int64_t)qi * sh.ss;
  const T* tqr = tq ? tq + base + (int64_t)qi * sh.ss : nullptr;
  const int nkeys = causal ? qi + 1 : sh.seq;
  const float L = lse[(int64_t)bh * sh.seq + qi];
  float mu = 0.f;
  float acc_w[4] = {0.f, 0.f, 0.f, 0.f}, acc_o[4] = {0.f, 0.f, 0.f, 0.f}, acc_t[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < nkeys; k0 += 64) {
    const int key = k0 + lane;
    float p = 0.f, w = 0.f;
    if (key < nkeys) {
      const T* kr = k + base + (int64_t)key * sh.ss;
      const T* tkr = tk ? tk + base + (int64_t)key * sh.ss : nullptr;
      float s = 0.f, ts = 0.f;
      for (int i = 0; i < d; i++) {
        const float qv = to_f32(qr[i]), kv = to_f32(kr[i]);
        s = fmaf(qv, kv, s);
        if (tqr) ts = fmaf(to_f32(tqr[i]), kv, ts);
        if (tkr) ts = fmaf(qv, to_f32(tkr[i]), ts);
      }
      p = expf(s * scale - L);
      w = p * ts * scale;
    }
    mu += wave_sum(w);
    const int cnt = nkeys - k0 < 64 ? nkeys - k0 : 64;
    for (int j = 0; j < cnt; j++) {
      const float pj = __shfl(p, j, 64), wj = __shfl(w, j, 64);
      const T* vr = v + base + (int64_t)(k0 + j) * sh.ss;
      const T* tvr = tv ? tv + base + (int64_t)(k0 + j) * sh.ss : nullptr;
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const int i = lane + c * 64;
        if (i < d) {
          const float vv = to_f32(vr[i]);
          acc_w[c] = fmaf(wj, vv, acc_w[c]);
          acc_o[c] = fmaf(pj, vv, acc_o[c]);
          if (tvr) acc_t[c] = fmaf(pj, to_f32(tvr[i]), acc_t[c]);
        }
      }
    }
  }
  T* out = to + base + (int64_t)qi * sh.ss;
#pragma unroll
  for (int c = 0; c < 4; c++) {
    const int i = lane + c * 64;
    if (i < d) out[i] = from_f32<T>(acc_w[c] - mu * acc_o[c] + acc_t[c]);
  }
}

bool al16(const void* p) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

// attention.hip
int launch_attn_jvp_mfma(hipStream_t st, const void* q, const void* k, const void* v, const float* lse, const void* tq,
                         const void* tk, const void* tv, void* to, int64_t batch, int64_t heads, int64_t seq, int64_t head_dim,
                         int64_t sb, int64_t shh, int64_t ss, float scale, int causal, int dtype);
}  // namespace emi

using namespace emi;

extern "C" int emi_rmsnorm_jvp(emi_stream_t stream, const void* x, const void* gamma, const void* tx, const void* tgamma,
                               void* ty, int64_t rows, int64_t dim, float eps, int dtype) {
  EMI_REQUIRE(rows >= 0 && dim > 0, "emi_rmsnorm_jvp: bad shape rows=%lld dim=%lld", (long long)rows, (long long)dim);
  EMI_REQUIRE(dtype == EMI_F32 || dtype == EMI_BF16, "emi_rmsnorm_jvp: unsupported dtype code %d (want 11=f32 or 16=bf16)", dtype);
  if (rows == 0) return EMI_OK;
  EMI_REQUIRE(x && gamma && ty, "emi_rmsnorm_jvp: null buffer");
  EMI_REQUIRE(rows <= 0x7fffffff, "emi_rmsnorm_jvp: too many rows");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec = dim % 8 == 0 && al16(x) && al16(gamma) && al16(tx) && al16(tgamma) && al16(ty);
#define EMI_RMS_JVP(T, VEC)                                                                                          \
  hipLaunchKernelGGL((rmsnorm_jvp_kernel<T, VEC>), dim3((unsigned)rows), dim3(256), 0, st, (const T*)x, (const T*)gamma, \
                     (const T*)tx, (const T*)tgamma, (T*)ty, dim, eps)
#define EMI_RMS_JVP_ROWS(T, NCH)                                                                                     \
  hipLaunchKernelGGL((rmsnorm_jvp_rows_kernel<T, NCH>), dim3((unsigned)rows), dim3(256), 0, st, (const T*)x, (const T*)gamma, \
                     (const T*)tx, (const T*)tgamma, (T*)ty, (int)dim, eps)
#define EMI_RMS_JVP_T(T)                                   \
  do {                                                     \
    if (!vec) EMI_RMS_JVP(T, false);                       \
    else if (dim <= 2048) EMI_RMS_JVP_ROWS(T, 1);          \
    else if (dim <= 4096) EMI_RMS_JVP_ROWS(T, 2);          \
    else if (dim <= 8192) EMI_RMS_JVP_ROWS(T, 4);          \
    else EMI_RMS_JVP(T, true);                             \
  } while (0)
  if (dtype == EMI_BF16) EMI_RMS_JVP_T(bf16);
  else EMI_RMS_JVP_T(float);
#undef EMI_RMS_JVP_T
#undef EMI_RMS_JVP_ROWS
#undef EMI_RMS_JVP
  EMI_CHECK_LAUNCH("emi_rmsnorm_jvp");
  return EMI_OK;
}

extern "C" int emi_swiglu_jvp(emi_stream_t stream, const void* a, const void* b, const void* ta, const void* tb, void* tg,
                              int64_t n, int dtype) {
  EMI_REQUIRE(n >= 0, "emi_swiglu_jvp: negative size");
  EMI_REQUIRE(dtype == EMI_F32 || dtype == EMI_BF16, "emi_swiglu_jvp: unsupported dtype code %d (want 11=f32 or 16=bf16)", dtype);
  if (n == 0) return EMI_OK;
  EMI_REQUIRE(a && b && tg, "emi_swiglu_jvp: null buffer");
  EMI_REQUIRE(al16(a) && al16(b) && al16(ta) && al16(tb) && al16(tg), "emi_swiglu_jvp: buffers must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)(((n >> 3) + (n & 7) + 255) / 256));
  if (dtype == EMI_BF16)
    hipLaunchKernelGGL(swiglu_jvp_kernel<bf16>, grid, dim3(256), 0, st, (const bf16*)a, (const bf16*)b, (const bf16*)ta,
                       (const bf16*)tb, (bf16*)tg, n);
  else
    hipLaunchKernelGGL(swiglu_jvp_kernel<float>, grid, dim3(256), 0, st, (const float*)a, (const float*)b, (const float*)ta,
                       (const float*)tb, (float*)tg, n);
  EMI_CHECK_LAUNCH("emi_swiglu_jvp");
  return EMI_OK;
}

extern "C" int emi_attn_jvp(emi_stream_t stream, const void* q, const void* k, const void* v, const float* lse, const void* tq,
                            const void* tk, const void* tv, void* to, int64_t batch, int64_t heads, int64_t seq,
                            int64_t head_dim, int64_t stride_b, int64_t stride_h, int64_t stride_s, float scale, int causal,
                            int dtype) {
  EMI_REQUIRE(batch >= 0 && heads > 0 && seq > 0 && head_dim > 0, "emi_attn_jvp: bad shape [%lld,%lld,%lld,%lld]",
              (long long)batch, (long long)heads, (long long)seq, (long long)head_dim);
  EMI_REQUIRE(dtype == EMI_F32 || dtype == EMI_BF16, "emi_attn_jvp: unsupported dtype code %d (want 11=f32 or 16=bf16)", dtype);
  EMI_REQUIRE(head_dim <= 256, "emi_attn_jvp: head_dim %lld > 256 is not supported", (long long)head_dim);
  EMI_REQUIRE(stride_s >= head_dim && stride_h > 0 && stride_b > 0, "emi_attn_jvp: bad strides");
  EMI_REQUIRE(seq <= 0x7fffffff / 4 && batch * heads <= 65535, "emi_attn_jvp: seq or batch*heads too large");
  if (batch == 0) return EMI_OK;
  EMI_REQUIRE(q && k && v && lse && to, "emi_attn_jvp: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  {
    const int rc = launch_attn_jvp_mfma(st, q, k, v, lse, tq, tk, tv, to, batch, heads, seq, head_dim, stride_b, stride_h,
                                        stride_s, scale, causal, dtype);
    if (rc >= 0) return rc;
  }
  const JvpShape sh{(int)seq, (int)heads, stride_b, stride_h, stride_s};
  const dim3 grid((unsigned)((seq + 3) / 4), (unsigned)(batch * heads));
  if (dtype == EMI_BF16)
    hipLaunchKernelGGL(attn_jvp_kernel<bf16>, grid, dim3(256), 0, st, (const bf16*)q, (const bf16*)k, (const bf16*)v, lse,
                       (const bf16*)tq, (const bf16*)tk, (const bf16*)tv, (bf16*)to, sh, (int)head_dim, scale, causal);
  else
    hipLaunchKernelGGL(attn_jvp_kernel<float>, grid, dim3(256), 0, st, (const float*)q, (const float*)k, (const float*)v, lse,
                       (const float*)tq, (const float*)tk, (const float*)tv, (float*)to, sh, (int)head_dim, scale, causal);
  EMI_CHECK_LAUNCH("emi_attn_jvp");
  return EMI_OK;
}
