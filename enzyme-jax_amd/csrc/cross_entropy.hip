// Softmax cross-entropy over the logits of the llama path for gfx950 (the loss that
// follows the classifier commented out at test/llama.py:236): per token
//   loss = logsumexp(z) - z[target],   dz = (softmax(z) - onehot(target)) * dloss,
//   tloss = sum_v softmax(z)_v tz_v - tz[target].
// All three kernels are HBM streams (the logits are read once, the adjoint writes them
// once): 16-byte chunks, every load of a pass issued before the first use, exponentials
// as exp2 with log2(e) folded into one multiply-add, fp32 arithmetic whatever the storage
// type.  A token whose target lies outside [0, vocab) is masked: zero loss, zero gradient.
#include "emi_device.h"

namespace emi {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Chunk c of a row as fp32.  VEC: one 16-byte load (rows are 16-byte aligned and hold
// whole chunks); otherwise scalar loads, elements past the row end reading as `fill`.
template <typename T, bool VEC>
__device__ __forceinline__ void load_row_chunk(const T* row, int64_t c, int64_t vocab, float fill,
                                               float (&v)[Chunk<T>::N]) {
  constexpr int N = Chunk<T>::N;
  if constexpr (VEC) {
    Chunk<T>::load(row + c * N, v);
  } else {
#pragma unroll
    for (int e = 0; e < N; e++) v[e] = c * N + e < vocab ? to_f32(row[c * N + e]) : fill;
  }
}

// Sum of `a` over the block's four wavefronts.
__device__ __forceinline__ float block_sum(float a, float* red) {
  a = wave_sum(a);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) red[wave] = a;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

// One block per token.  Each thread keeps a running (max, sum of 2^(z log2e - max)) over
// its chunks, UN chunks per pass in flight.
template <typename T, bool VEC, int UN>
__global__ __launch_bounds__(256) void xent_fwd_kernel(const T* __restrict__ logits, const int32_t* __restrict__ targets,
                                                       float* __restrict__ loss, float* __restrict__ lse,
                                                       int64_t vocab) {
  constexpr int N = Chunk<T>::N;
  __shared__ float red[8];
  const int64_t row = blockIdx.x;
  const T* z = logits + row * vocab;
  const int64_t nchunk = (vocab + N - 1) / N;
  float m = -INFINITY, s = 0.f;
  for (int64_t c0 = threadIdx.x; c0 < nchunk; c0 += 256 * UN) {
    if constexpr (VEC) {
      // chunks stay in storage format (16 bytes each) and are unpacked for the maximum and again for the sum
      typename Chunk<T>::Raw raw[UN];
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int64_t c = c0 + 256 * u;
        raw[u] = Chunk<T>::load_raw(z + (c < nchunk ? c : c0) * N);      // past the end: this thread's first chunk again
      }
      float top = -INFINITY;
#pragma unroll
      for (int u = 0; u < UN; u++) {
        float v[N];
        Chunk<T>::unpack(raw[u], v);
#pragma unroll
        for (int e = 0; e < N; e++) top = fmaxf(top, v[e]);
      }
      const float mx = fmaxf(m, top * kLog2e);
      if (mx > -INFINITY) {                       // at least one finite logit so far
        float t = 0.f;
#pragma unroll
        for (int u = 0; u < UN; u++) {
          if (c0 + 256 * u < nchunk) {
            float v[N];
            Chunk<T>::unpack(raw[u], v);
#pragma unroll
            for (int e = 0; e < N; e++) t += __builtin_amdgcn_exp2f(fmaf(v[e], kLog2e, -mx));
          }
        }
        s = s * __builtin_amdgcn_exp2f(m - mx) + t;
        m = mx;
      }
    } else {
      float v[UN][N];
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int64_t c = c0 + 256 * u;
        if (c < nchunk) {
          load_row_chunk<T, VEC>(z, c, vocab, -INFINITY, v[u]);
        } else {
#pragma unroll
          for (int e = 0; e < N; e++) v[u][e] = -INFINITY;
        }
      }
      float top = -INFINITY;
#pragma unroll
      for (int u = 0; u < UN; u++)
#pragma unroll
        for (int e = 0; e < N; e++) top = fmaxf(top, v[u][e]);
      const float mx = fmaxf(m, top * kLog2e);
      if (mx > -INFINITY) {                       // at least one finite logit so far
        float t = 0.f;
#pragma unroll
        for (int u = 0; u < UN; u++)
#pragma unroll
          for (int e = 0; e < N; e++) t += __builtin_amdgcn_exp2f(fmaf(v[u][e], kLog2e, -mx));
        s = s * __builtin_amdgcn_exp2f(m - mx) + t;
        m = mx;
      }
    }
  }
  // block reduction of (m, s)
  const float mw = wave_max(m);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) red[4 + wave] = mw;
  __syncthreads();
  const float mb = fmaxf(fmaxf(red[4], red[5]), fmaxf(red[6], red[7]));
  const float sc = m > -INFINITY ? s * __builtin_amdgcn_exp2f(m - mb) : 0.f;
  const float sb = block_sum(sc, red);
  if (threadIdx.x == 0) {
    const float l = (mb + __builtin_amdgcn_logf(sb)) * kLn2;        // v_log_f32 is log2
    const int32_t t = targets[row];
    const bool live = t >= 0 && t < vocab;
    lse[row] = l;
    loss[row] = live ? l - to_f32(z[t]) : 0.f;
  }
}

// dz = (2^(z log2e - lse log2e) - [v == target]) * dloss.  A block owns 256*UN chunks of one row; consecutive
// blocks walk along a row, then to the next row, so that the blocks in flight cover one contiguous range.
template <typename T, bool VEC, int UN>
__global__ __launch_bounds__(256) void xent_bwd_kernel(const T* __restrict__ logits, const int32_t* __restrict__ targets,
                                                       const float* __restrict__ lse, const float* __restrict__ dloss,
                                                       T* __restrict__ dlogits, int vocab, int blocks_per_row) {
  constexpr int N = Chunk<T>::N;
  const int64_t row = blockIdx.x / blocks_per_row;
  const T* z = logits + row * vocab;
  T* dz = dlogits + row * vocab;
  const int nchunk = (vocab + N - 1) / N;
  const int c0 = (blockIdx.x % blocks_per_row) * (256 * UN) + threadIdx.x;
  float v[UN][N];
#pragma unroll
  for (int u = 0; u < UN; u++) {
    const int c = c0 + 256 * u;
    if (c < nchunk) load_row_chunk<T, VEC>(z, c, vocab, 0.f, v[u]);
  }
  const int32_t t = targets[row];
  const bool live = t >= 0 && t < vocab;
  const float g = live ? dloss[row] : 0.f;
  const float l2 = lse[row] * kLog2e;
#pragma unroll
  for (int u = 0; u < UN; u++) {
    const int c = c0 + 256 * u;
    if (c < nchunk) {
      float o[N];
#pragma unroll
      for (int e = 0; e < N; e++) o[e] = __builtin_amdgcn_exp2f(fmaf(v[u][e], kLog2e, -l2)) * g;
      const int rel = t - c * N;                  // the target's place in this chunk, if it is here
      if (rel >= 0 && rel < N) {
#pragma unroll
        for (int e = 0; e < N; e++)
          if (e == rel) o[e] -= g;
      }
      if constexpr (VEC) {
        Chunk<T>::store(dz + (int64_t)c * N, o);
      } else {
#pragma unroll
        for (int e = 0; e < N; e++)
          if (c * N + e < vocab) dz[c * N + e] = from_f32<T>(o[e]);
      }
    }
  }
}

// tloss = sum_v p_v tz_v - tz[target], p from lse; one block per token.
template <typename T, bool VEC, int UN>
__global__ __launch_bounds__(256) void xent_jvp_kernel(const T* __restrict__ logits, const int32_t* __restrict__ targets,
                                                       const float* __restrict__ lse, const T* __restrict__ tlogits,
                                                       float* __restrict__ tloss, int64_t vocab) {
  constexpr int N = Chunk<T>::N;
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const T* z = logits + row * vocab;
  const T* tz = tlogits + row * vocab;
  const int64_t nchunk = (vocab + N - 1) / N;
  const float l2 = lse[row] * kLog2e;
  float acc = 0.f;
  for (int64_t c0 = threadIdx.x; c0 < nchunk; c0 += 256 * UN) {
    if constexpr (VEC) {
      typename Chunk<T>::Raw rz[UN], rt[UN];                 // storage format until used
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int64_t c = c0 + 256 * u;
        if (c < nchunk) {
          rz[u] = Chunk<T>::load_raw(z + c * N);
          rt[u] = Chunk<T>::load_raw(tz + c * N);
        }
      }
#pragma unroll
      for (int u = 0; u < UN; u++) {
        if (c0 + 256 * u < nchunk) {
          float v[N], w[N];
          Chunk<T>::unpack(rz[u], v);
          Chunk<T>::unpack(rt[u], w);
#pragma unroll
          for (int e = 0; e < N; e++) acc += __builtin_amdgcn_exp2f(fmaf(v[e], kLog2e, -l2)) * w[e];
        }
      }
    } else {
      float v[UN][N], w[UN][N];
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int64_t c = c0 + 256 * u;
        if (c < nchunk) {
          load_row_chunk<T, VEC>(z, c, vocab, -INFINITY, v[u]);
          load_row_chunk<T, VEC>(tz, c, vocab, 0.f, w[u]);
        } else {
#pragma unroll
          for (int e = 0; e < N; e++) v[u][e] = -INFINITY, w[u][e] = 0.f;
        }
      }
#pragma unroll
      for (int u = 0; u < UN; u++)
#pragma unroll
        for (int e = 0; e < N; e++) acc += __builtin_amdgcn_exp2f(fmaf(v[u][e], kLog2e, -l2)) * w[u][e];
    }
  }
  const float tot = block_sum(acc, red);
  if (threadIdx.x == 0) {
    const int32_t t = targets[row];
    const bool live = t >= 0 && t < vocab;
    tloss[row] = live ? tot - to_f32(tz[t]) : 0.f;
  }
}

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T> static inline bool row_chunks(int64_t vocab, const void* a, const void* b) {
  return vocab % Chunk<T>::N == 0 && aligned16(a) && aligned16(b);
}

template <typename T>
static int xent_fwd_launch(hipStream_t st, const void* logits, const int32_t* targets, float* loss, float* lse,
                           int64_t tokens, int64_t vocab) {
  const T* z = static_cast<const T*>(logits);
  if (row_chunks<T>(vocab, logits, nullptr))
    hipLaunchKernelGGL((xent_fwd_kernel<T, true, 16>), dim3((unsigned)tokens), dim3(256), 0, st, z, targets, loss, lse, vocab);
  else
    hipLaunchKernelGGL((xent_fwd_kernel<T, false, 2>), dim3((unsigned)tokens), dim3(256), 0, st, z, targets, loss, lse, vocab);
  EMI_CHECK_LAUNCH("emi_cross_entropy_fwd");
  return EMI_OK;
}

template <typename T>
static int xent_bwd_launch(hipStream_t st, const void* logits, const int32_t* targets, const float* lse,
                           const float* dloss, void* dlogits, int64_t tokens, int64_t vocab) {
  const T* z = static_cast<const T*>(logits);
  T* dz = static_cast<T*>(dlogits);
  constexpr int N = Chunk<T>::N;
  const int64_t nchunk = (vocab + N - 1) / N;
  const bool vec = row_chunks<T>(vocab, logits, dlogits);
  constexpr int UNV = 8 / N;                                 // eight elements per lane
  const int64_t per_row = vec ? (nchunk + 256 * UNV - 1) / (256 * UNV) : (nchunk + 256 * 2 - 1) / (256 * 2);
  EMI_REQUIRE(tokens * per_row <= 0x7fffffffLL, "emi_cross_entropy_bwd: %lld tokens x %lld blocks per row exceed the grid",
              (long long)tokens, (long long)per_row);
  const unsigned grid = (unsigned)(tokens * per_row);
  if (vec)
    hipLaunchKernelGGL((xent_bwd_kernel<T, true, UNV>), dim3(grid), dim3(256), 0, st, z, targets, lse, dloss, dz, (int)vocab, (int)per_row);
  else
    hipLaunchKernelGGL((xent_bwd_kernel<T, false, 2>), dim3(grid), dim3(256), 0, st, z, targets, lse, dloss, dz, (int)vocab, (int)per_row);
  EMI_CHECK_LAUNCH("emi_cross_entropy_bwd");
  return EMI_OK;
}

template <typename T>
static int xent_jvp_launch(hipStream_t st, const void* logits, const int32_t* targets, const float* lse,
                           const void* tlogits, float* tloss, int64_t tokens, int64_t vocab) {
  const T* z = static_cast<const T*>(logits);
  const T* tz = static_cast<const T*>(tlogits);
  if (row_chunks<T>(vocab, logits, tlogits))
    hipLaunchKernelGGL((xent_jvp_kernel<T, true, 8>), dim3((unsigned)tokens), dim3(256), 0, st, z, targets, lse, tz, tloss, vocab);
  else
    hipLaunchKernelGGL((xent_jvp_kernel<T, false, 2>), dim3((unsigned)tokens), dim3(256), 0, st, z, targets, lse, tz, tloss, vocab);
  EMI_CHECK_LAUNCH("emi_cross_entropy_jvp");
  return EMI_OK;
}

}  // namespace emi

using namespace emi;

#define EMI_XENT_SHAPE(name)                                                                                          \
  EMI_REQUIRE(tokens >= 0 && vocab > 0, name ": bad shape tokens=%lld vocab=%lld", (long long)tokens, (long long)vocab); \
  EMI_REQUIRE(tokens <= 0x7fffffffLL, name ": tokens=%lld too large", (long long)tokens);                              \
  EMI_REQUIRE(vocab <= (1LL << 24), name ": vocab=%lld too large (at most 2^24)", (long long)vocab);                   \
  if (tokens == 0) return EMI_OK;

extern "C" int emi_cross_entropy_fwd(emi_stream_t stream, const void* logits, const int32_t* targets, float* loss,
                                     float* lse, int64_t tokens, int64_t vocab, int dtype) {
  EMI_XENT_SHAPE("emi_cross_entropy_fwd")
  EMI_REQUIRE(logits && targets && loss && lse, "emi_cross_entropy_fwd: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case EMI_F32: return xent_fwd_launch<float>(st, logits, targets, loss, lse, tokens, vocab);
    case EMI_BF16: return xent_fwd_launch<bf16>(st, logits, targets, loss, lse, tokens, vocab);
    default: return emi_fail(EMI_INVALID_ARGUMENT, "emi_cross_entropy_fwd: unsupported dtype code %d (want 11=f32 or 16=bf16)", dtype);
  }
}

extern "C" int emi_cross_entropy_bwd(emi_stream_t stream, const void* logits, const int32_t* targets, const float* lse,
                                     const float* dloss, void* dlogits, int64_t tokens, int64_t vocab, int dtype) {
  EMI_XENT_SHAPE("emi_cross_entropy_bwd")
  EMI_REQUIRE(logits && targets && lse && dloss && dlogits, "emi_cross_entropy_bwd: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case EMI_F32: return xent_bwd_launch<float>(st, logits, targets, lse, dloss, dlogits, tokens, vocab);
    case EMI_BF16: return xent_bwd_launch<bf16>(st, logits, targets, lse, dloss, dlogits, tokens, vocab);
    default: return emi_fail(EMI_INVALID_ARGUMENT, "emi_cross_entropy_bwd: unsupported dtype code %d (want 11=f32 or 16=bf16)", dtype);
  }
}

extern "C" int emi_cross_entropy_jvp(emi_stream_t stream, const void* logits, const int32_t* targets, const float* lse,
                                     const void* tlogits, float* tloss, int64_t tokens, int64_t vocab, int dtype) {
  EMI_XENT_SHAPE("emi_cross_entropy_jvp")
  EMI_REQUIRE(logits && targets && lse && tlogits && tloss, "emi_cross_entropy_jvp: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case EMI_F32: return xent_jvp_launch<float>(st, logits, targets, lse, tlogits, tloss, tokens, vocab);
    case EMI_BF16: return xent_jvp_launch<bf16>(st, logits, targets, lse, tlogits, tloss, tokens, vocab);
    default: return emi_fail(EMI_INVALID_ARGUMENT, "emi_cross_entropy_jvp: unsupported dtype code %d (want 11=f32 or 16=bf16)", dtype);
  }
}
