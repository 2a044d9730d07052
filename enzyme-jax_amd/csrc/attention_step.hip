// Attention of the single-token (decode) step: one query per (batch, head) against the
// seq_kv rows of that head's key/value cache, test/llama.py:178-206 with the softmax of
// :13-18 (scale applied after the dot, max-subtracted).  HBM-bound: every cache row is read
// once (forward and backward) and dK, dV are written once.  The keys of a head are split
// over blocks of kKeysPerBlock (there are only batch*heads queries, far too few to fill
// the chip); each block leaves a partial result (max, sum, unnormalised output; or its
// share of dQ) in the workspace and a second small kernel combines them in a fixed order.
// Inside a block 16 lanes share a key, each lane owning 16-byte chunks of the head
// dimension, and every lane keeps four keys in flight.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "emi_device.h"

namespace emi {
namespace {

constexpr int kRedFloats = 2048;                 // LDS floats for the reduction over key slots
constexpr int kKeysPerBlock = 512;

template <typename T> struct Vec16;              // 16 raw bytes of T, unpacked on use
template <> struct Vec16<float> {
  typedef float4 type;
  static __device__ __forceinline__ float4 zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
  static __device__ __forceinline__ void unpack(const float4& r, float (&v)[4]) { v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w; }
};
template <> struct Vec16<bf16> {
  typedef uint4 type;
  static __device__ __forceinline__ uint4 zero() { return make_uint4(0, 0, 0, 0); }
  static __device__ __forceinline__ void unpack(const uint4& r, float (&v)[8]) { Vec8<bf16>::unpack(r, v); }
};

template <typename T, bool VEC> struct Elems {   // VEC: 16-byte chunks; else single elements (any head_dim / alignment)
  static constexpr int N = VEC ? Chunk<T>::N : 1;
  // the same piece as it sits in memory (a streaming load: the cache rows are read once), unpacked on use
  typedef std::conditional_t<VEC, typename Vec16<T>::type, T> Raw;
  static __device__ __forceinline__ Raw load_raw(const T* p) {
    if constexpr (VEC) return stream_load(reinterpret_cast<const Raw*>(p));
    else return p[0];
  }
  static __device__ __forceinline__ Raw zero_raw() {
    if constexpr (VEC) return Vec16<T>::zero();
    else return from_f32<T>(0.f);
  }
  static __device__ __forceinline__ void unpack(const Raw& r, float (&v)[N]) {
    if constexpr (VEC) Vec16<T>::unpack(r, v);
    else v[0] = to_f32(r);
  }
  static __device__ __forceinline__ void load(const T* p, float (&v)[N]) {
    if constexpr (VEC) Chunk<T>::load(p, v);
    else v[0] = to_f32(p[0]);
  }
  static __device__ __forceinline__ void store(T* p, const float (&v)[N]) {
    if constexpr (VEC) Chunk<T>::store(p, v);
    else p[0] = from_f32<T>(v[0]);
  }
};

struct StepShape {
  int heads, seq_kv, head_dim;
  int64_t q_sb, q_sh, kv_sb, kv_sh, kv_ss;
};

__device__ __forceinline__ float sum16(float v) {          // over the 16 lanes that share a key
  v += __shfl_xor(v, 1, kWave);
  v += __shfl_xor(v, 2, kWave);
  v += __shfl_xor(v, 4, kWave);
  v += __shfl_xor(v, 8, kWave);
  return v;
}

// Block-wide reductions through a 4-float LDS scratch.
__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  return fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
}
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  return scratch[0] + scratch[1] + scratch[2] + scratch[3];
}

// Sum of per-lane chunk accumulators over the 16 key slots of the block (4 per wavefront:
// lane bits 4, 5; then the 4 wavefronts through LDS).  Result valid in threads 0..15.
template <int MAXC, int NE>
__device__ __forceinline__ void reduce_keys(float (&acc)[MAXC][NE], int nch, float* red /* [4][MAXC][16][NE] */) {
  static_assert(4 * MAXC * 16 * NE <= kRedFloats, "reduction scratch");
  const int l16 = threadIdx.x & 15, wave = threadIdx.x >> 6;
  __syncthreads();
#pragma unroll
  for (int c = 0; c < MAXC; c++)
#pragma unroll
    for (int e = 0; e < NE; e++) {
      float v = acc[c][e];
      v += __shfl_xor(v, 16, kWave);
      v += __shfl_xor(v, 32, kWave);
      if ((threadIdx.x & 63) < 16 && c < nch) red[(wave * MAXC + c) * 16 * NE + l16 * NE + e] = v;
    }
  __syncthreads();
  if (threadIdx.x < 16) {
#pragma unroll
    for (int c = 0; c < MAXC; c++)
#pragma unroll
      for (int e = 0; e < NE; e++) {
        float v = 0.f;
        if (c < nch)
          for (int w = 0; w < 4; w++) v += red[(w * MAXC + c) * 16 * NE + l16 * NE + e];
        acc[c][e] = v;
      }
  }
}

// NCH: 16-byte chunks (or single elements) of the head dimension per lane, 1, 2, 4 or 16; a
// lane keeps 16 / NCH (at least 2) keys in flight.
template <typename T, bool VEC, int NCH>
__global__ __launch_bounds__(256) void attn_step_fwd_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                            const T* __restrict__ v, float* __restrict__ part, StepShape sh,
                                                            float scale) {
  constexpr int NE = Elems<T, VEC>::N, MAXC = NCH, kUnroll = NCH >= 8 ? 2 : 16 / NCH;
  __shared__ float scores[kKeysPerBlock];
  __shared__ float scratch[4];
  __shared__ float red[kRedFloats];
  const int bh = blockIdx.y, b = bh / sh.heads, h = bh % sh.heads;
  const int s0 = blockIdx.x * kKeysPerBlock;
  const int s1 = s0 + kKeysPerBlock < sh.seq_kv ? s0 + kKeysPerBlock : sh.seq_kv;
  const int l16 = threadIdx.x & 15, slot = threadIdx.x >> 4;       // 16 key slots per block
  const int nchunks = sh.head_dim / NE;                            // chunks per row
  const int nch = (nchunks - l16 + 15) / 16;                       // chunks of this lane: l16, l16 + 16, ...
  const T* qrow = q + b * sh.q_sb + h * sh.q_sh;
  const T* kbase = k + b * sh.kv_sb + h * sh.kv_sh;
  const T* vbase = v + b * sh.kv_sb + h * sh.kv_sh;

  float qf[MAXC][NE];
#pragma unroll
  for (int c = 0; c < MAXC; c++)
    if (c < nch) Elems<T, VEC>::load(qrow + (l16 + 16 * c) * NE, qf[c]);

  float mx = -INFINITY;
  for (int sb = s0 + slot; sb < s1; sb += 16 * kUnroll) {
    float dot[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      const int s = sb + 16 * u;
      dot[u] = 0.f;
      if (s < s1) {
        const T* krow = kbase + (int64_t)s * sh.kv_ss;
#pragma unroll
        for (int c = 0; c < MAXC; c++)
          if (c < nch) {
            float kf[NE];
            Elems<T, VEC>::load(krow + (l16 + 16 * c) * NE, kf);
#pragma unroll
            for (int e = 0; e < NE; e++) dot[u] = fmaf(qf[c][e], kf[e], dot[u]);
          }
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      const int s = sb + 16 * u;
      const float d = sum16(dot[u]) * scale;
      if (s < s1) {
        if (l16 == 0) scores[s - s0] = d;
        mx = fmaxf(mx, d);
      }
    }
  }
  mx = block_max(mx, scratch);
  float sum = 0.f;
  for (int s = threadIdx.x; s < s1 - s0; s += 256) {
    const float p = __expf(scores[s] - mx);
    scores[s] = p;
    sum += p;
  }
  sum = block_sum(sum, scratch);                          // also orders the writes of p before the reads below

  float acc[MAXC][NE];
#pragma unroll
  for (int c = 0; c < MAXC; c++)
#pragma unroll
    for (int e = 0; e < NE; e++) acc[c][e] = 0.f;
  for (int sb = s0 + slot; sb < s1; sb += 16 * kUnroll) {
    float vf[kUnroll][MAXC][NE];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      const int s = sb + 16 * u;
      if (s < s1) {
        const T* vrow = vbase + (int64_t)s * sh.kv_ss;
#pragma unroll
        for (int c = 0; c < MAXC; c++)
          if (c < nch) Elems<T, VEC>::load(vrow + (l16 + 16 * c) * NE, vf[u][c]);
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      const int s = sb + 16 * u;
      if (s < s1) {
        const float p = scores[s - s0];
#pragma unroll
        for (int c = 0; c < MAXC; c++)
          if (c < nch) {
#pragma unroll
            for (int e = 0; e < NE; e++) acc[c][e] = fmaf(p, vf[u][c][e], acc[c][e]);
          }
      }
    }
  }
  reduce_keys<MAXC, NE>(acc, nch, red);
  if (threadIdx.x < 16) {
    // partial of this block: [head_dim] unnormalised output, then max and sum
    float* out = part + ((int64_t)bh * gridDim.x + blockIdx.x) * (sh.head_dim + 2);
#pragma unroll
    for (int c = 0; c < MAXC; c++)
      if (c < nch) {
#pragma unroll
        for (int e = 0; e < NE; e++) out[(l16 + 16 * c) * NE + e] = acc[c][e];
      }
    if (threadIdx.x == 0) {
      out[sh.head_dim] = mx;
      out[sh.head_dim + 1] = sum;
    }
  }
}

// Forward for one 16-byte chunk per lane (head_dim 128 in bf16, 64 in fp32, and smaller):
// the block loads all its K and V chunks up front (32 keys per slot, 16 loads of each kind
// in flight per lane, kept as raw 16-byte vectors) and then works from registers, so the
// memory system sees the whole request at once.
template <typename T>
__global__ __launch_bounds__(256) void attn_step_fwd1_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                             const T* __restrict__ v, float* __restrict__ part, StepShape sh,
                                                             float scale) {
  constexpr int NE = Chunk<T>::N, KPS = kKeysPerBlock / 16 / 2;      // keys per slot and half
  typedef typename Vec16<T>::type raw_t;
  __shared__ float scratch[4];
  __shared__ float red[kRedFloats];
  const int bh = blockIdx.y, b = bh / sh.heads, h = bh % sh.heads;
  const int l16 = threadIdx.x & 15, slot = threadIdx.x >> 4;
  const bool mine = l16 * NE < sh.head_dim;                         // lanes beyond the head dimension idle
  const T* qrow = q + b * sh.q_sb + h * sh.q_sh + l16 * NE;
  const T* kbase = k + b * sh.kv_sb + h * sh.kv_sh + l16 * NE;
  const T* vbase = v + b * sh.kv_sb + h * sh.kv_sh + l16 * NE;
  float qf[NE];
#pragma unroll
  for (int e = 0; e < NE; e++) qf[e] = 0.f;
  if (mine) Chunk<T>::load(qrow, qf);

  float mx = -INFINITY, sum = 0.f;
  float acc[1][NE];
#pragma unroll
  for (int e = 0; e < NE; e++) acc[0][e] = 0.f;
  // two halves of 16 keys per slot: registers hold 16 K and 16 V chunks at a time
#pragma unroll 1
  for (int half = 0; half < 2; half++) {
    const int s0 = blockIdx.x * kKeysPerBlock + half * (kKeysPerBlock / 2);
    if (s0 >= sh.seq_kv) break;
    raw_t kr[KPS], vr[KPS];
#pragma unroll
    for (int u = 0; u < KPS; u++) {
      const int s = s0 + slot + 16 * u;
      kr[u] = Vec16<T>::zero();
      vr[u] = Vec16<T>::zero();
      if (mine && s < sh.seq_kv) {
        kr[u] = stream_load(reinterpret_cast<const raw_t*>(kbase + (int64_t)s * sh.kv_ss));     // the cache rows are read once
        vr[u] = stream_load(reinterpret_cast<const raw_t*>(vbase + (int64_t)s * sh.kv_ss));
      }
    }
    float sc[KPS];
    float hm = -INFINITY;
#pragma unroll
    for (int u = 0; u < KPS; u++) {
      float kf[NE];
      Vec16<T>::unpack(kr[u], kf);
      float dot = 0.f;
#pragma unroll
      for (int e = 0; e < NE; e++) dot = fmaf(qf[e], kf[e], dot);
      sc[u] = s0 + slot + 16 * u < sh.seq_kv ? sum16(dot) * scale : -INFINITY;
      hm = fmaxf(hm, sc[u]);
    }
    // running maximum per slot (online softmax): rescale what has been accumulated so far
    const float nm = fmaxf(mx, hm);
    const float alpha = mx == -INFINITY ? 0.f : __expf(mx - nm);
    sum *= alpha;
#pragma unroll
    for (int e = 0; e < NE; e++) acc[0][e] *= alpha;
    mx = nm;
#pragma unroll
    for (int u = 0; u < KPS; u++) {
      const float p = sc[u] == -INFINITY ? 0.f : __expf(sc[u] - mx);
      sum += p;
      float vf[NE];
      Vec16<T>::unpack(vr[u], vf);
#pragma unroll
      for (int e = 0; e < NE; e++) acc[0][e] = fmaf(p, vf[e], acc[0][e]);
    }
  }
  // the 16 slots have their own running maxima: bring them to the block maximum, then reduce
  const float bm = block_max(mx, scratch);
  const float w = mx == -INFINITY ? 0.f : __expf(mx - bm);
#pragma unroll
  for (int e = 0; e < NE; e++) acc[0][e] *= w;
  float bsum = block_sum(l16 == 0 ? sum * w : 0.f, scratch);
  reduce_keys<1, NE>(acc, mine ? 1 : 0, red);
  if (threadIdx.x < 16) {
    float* out = part + ((int64_t)bh * gridDim.x + blockIdx.x) * (sh.head_dim + 2);
    if (mine) {
#pragma unroll
      for (int e = 0; e < NE; e++) out[l16 * NE + e] = acc[0][e];
    }
    if (threadIdx.x == 0) {
      out[sh.head_dim] = bm;
      out[sh.head_dim + 1] = bsum;
    }
  }
}

// o = sum_i w_i o_i / sum_i w_i l_i with w_i = exp(m_i - max m); lse = max m + log(sum).  One wavefront per
// (batch, head): lane i holds the statistics and the weight of split c + i and hands the weight round by lane
// index, so the partial rows stream in with independent loads instead of one dependent chain per pass.
template <typename T>
__global__ __launch_bounds__(64) void attn_step_combine_kernel(const float* __restrict__ part, T* __restrict__ o,
                                                               float* __restrict__ lse, StepShape sh, int nsplit) {
  const int bh = blockIdx.x, b = bh / sh.heads, h = bh % sh.heads;
  const int lane = threadIdx.x, hd = sh.head_dim, stride = sh.head_dim + 2;
  const float* p0 = part + (int64_t)bh * nsplit * stride;
  float mx = -INFINITY;
  for (int i = lane; i < nsplit; i += 64) mx = fmaxf(mx, p0[i * stride + hd]);
  mx = wave_max(mx);
  float l = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};                         // head_dim <= 256: up to four columns per lane
  for (int c = 0; c < nsplit; c += 64) {
    const int i = c + lane;
    float w = 0.f;
    if (i < nsplit) {
      w = __expf(p0[i * stride + hd] - mx);
      l += p0[i * stride + hd + 1] * w;
    }
    const int cnt = nsplit - c < 64 ? nsplit - c : 64;
    // eight partial rows requested together (a row past the last is the last again, with weight zero): one round
    // trip to memory per eight splits instead of one per split
    for (int i0 = 0; i0 < cnt; i0 += 8) {
      float r[8][4];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const float* row = p0 + (int64_t)(c + (i0 + u < cnt ? i0 + u : cnt - 1)) * stride;
#pragma unroll
        for (int q = 0; q < 4; q++) r[u][q] = row[lane + 64 * q < hd ? lane + 64 * q : 0];
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const float ws = __shfl(w, (i0 + u) & 63, kWave);
        const float wi = i0 + u < cnt ? ws : 0.f;
#pragma unroll
        for (int q = 0; q < 4; q++) acc[q] = fmaf(r[u][q], wi, acc[q]);
      }
    }
  }
  l = wave_sum(l);
  const float inv = 1.0f / l;
  T* orow = o + b * sh.q_sb + h * sh.q_sh;
#pragma unroll
  for (int q = 0; q < 4; q++)
    if (lane + 64 * q < hd) orow[lane + 64 * q] = from_f32<T>(acc[q] * inv);
  if (lane == 0) lse[bh] = mx + __logf(l);
}

// dV_s = p_s dO; dP_s = dO . V_s; dS_s = p_s (dP_s - dO . O); dQ = scale sum_s dS_s K_s;
// dK_s = scale dS_s Q.  p is recomputed from lse; one pass over the keys of the block.
template <typename T, bool VEC, int NCH>
__global__ __launch_bounds__(256) void attn_step_bwd_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                            const T* __restrict__ v, const T* __restrict__ o,
                                                            const float* __restrict__ lse, const T* __restrict__ d_o,
                                                            float* __restrict__ part, T* __restrict__ dk, T* __restrict__ dv,
                                                            StepShape sh, float scale) {
  using E = Elems<T, VEC>;
  using Raw = typename E::Raw;
  constexpr int NE = E::N, MAXC = NCH, U = NCH >= 4 ? 1 : 4 / NCH;      // keys per slot and batch
  __shared__ float red[kRedFloats];
  const int bh = blockIdx.y, b = bh / sh.heads, h = bh % sh.heads;
  const int s0 = blockIdx.x * kKeysPerBlock;
  const int s1 = s0 + kKeysPerBlock < sh.seq_kv ? s0 + kKeysPerBlock : sh.seq_kv;
  const int l16 = threadIdx.x & 15, slot = threadIdx.x >> 4;
  const int nchunks = sh.head_dim / NE;
  const int nch = (nchunks - l16 + 15) / 16;
  const int64_t qoff = b * sh.q_sb + h * sh.q_sh, kvoff = b * sh.kv_sb + h * sh.kv_sh;
  const float L = lse[bh];

  float qf[MAXC][NE], dof[MAXC][NE];
  int coff[MAXC];                                   // element offset of chunk c inside a row (a lane's idle chunks: 0)
  float delta = 0.f;
#pragma unroll
  for (int c = 0; c < MAXC; c++) {
    coff[c] = c < nch ? (l16 + 16 * c) * NE : 0;
#pragma unroll
    for (int e = 0; e < NE; e++) qf[c][e] = dof[c][e] = 0.f;
    if (c < nch) {
      float of[NE];
      E::load(q + qoff + coff[c], qf[c]);
      E::load(d_o + qoff + coff[c], dof[c]);
      E::load(o + qoff + coff[c], of);
#pragma unroll
      for (int e = 0; e < NE; e++) delta = fmaf(dof[c][e], of[e], delta);
    }
  }
  delta = sum16(delta);

  float acc[MAXC][NE];
#pragma unroll
  for (int c = 0; c < MAXC; c++)
#pragma unroll
    for (int e = 0; e < NE; e++) acc[c][e] = 0.f;
  // Two register sets of U keys: the next batch is requested before the current one is worked on.  The loads are
  // unconditional (a key past the block's range re-reads the last key and gets weight zero; a lane's idle chunks
  // re-read chunk 0 against zero q and dO): guarded loads make the compiler wait for all earlier ones before each.
  auto issue = [&](int sb, Raw(&kr)[U][MAXC], Raw(&vr)[U][MAXC]) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int s = sb + 16 * u < s1 ? sb + 16 * u : s1 - 1;
      const int64_t row = kvoff + (int64_t)s * sh.kv_ss;
#pragma unroll
      for (int c = 0; c < MAXC; c++) {
        kr[u][c] = E::load_raw(k + row + coff[c]);
        vr[u][c] = E::load_raw(v + row + coff[c]);
      }
    }
  };
  auto consume = [&](int sb, const Raw(&kr)[U][MAXC], const Raw(&vr)[U][MAXC]) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int s = sb + 16 * u;
      float kf[MAXC][NE];
      float dot = 0.f, dp = 0.f;
#pragma unroll
      for (int c = 0; c < MAXC; c++) {
        float vf[NE];
        E::unpack(kr[u][c], kf[c]);
        E::unpack(vr[u][c], vf);
#pragma unroll
        for (int e = 0; e < NE; e++) {
          dot = fmaf(qf[c][e], kf[c][e], dot);
          dp = fmaf(dof[c][e], vf[e], dp);
        }
      }
      dot = sum16(dot);
      dp = sum16(dp);
      if (s < s1) {
        const float p = __expf(dot * scale - L);
        const float ds = p * (dp - delta) * scale;
        T* dkrow = dk + kvoff + (int64_t)s * sh.kv_ss;
        T* dvrow = dv + kvoff + (int64_t)s * sh.kv_ss;
#pragma unroll
        for (int c = 0; c < MAXC; c++)
          if (c < nch) {
            float t[NE];
#pragma unroll
            for (int e = 0; e < NE; e++) acc[c][e] = fmaf(ds, kf[c][e], acc[c][e]);
#pragma unroll
            for (int e = 0; e < NE; e++) t[e] = ds * qf[c][e];
            E::store(dkrow + coff[c], t);
#pragma unroll
            for (int e = 0; e < NE; e++) t[e] = p * dof[c][e];
            E::store(dvrow + coff[c], t);
          }
      }
    }
  };
  {
    Raw k0[U][MAXC], v0[U][MAXC], k1[U][MAXC], v1[U][MAXC];
    int sb = s0 + slot;
    issue(sb, k0, v0);
    while (sb < s1) {
      const int sb1 = sb + 16 * U;
      if (sb1 < s1) issue(sb1, k1, v1);
      consume(sb, k0, v0);
      if (sb1 >= s1) break;
      sb = sb1 + 16 * U;
      if (sb < s1) issue(sb, k0, v0);
      consume(sb1, k1, v1);
    }
  }
  reduce_keys<MAXC, NE>(acc, nch, red);
  if (threadIdx.x < 16) {
    float* out = part + ((int64_t)bh * gridDim.x + blockIdx.x) * (sh.head_dim + 2);
#pragma unroll
    for (int c = 0; c < MAXC; c++)
      if (c < nch) {
#pragma unroll
        for (int e = 0; e < NE; e++) out[(l16 + 16 * c) * NE + e] = acc[c][e];
      }
  }
}

template <typename T>
__global__ __launch_bounds__(64) void attn_step_dq_kernel(const float* __restrict__ part, T* __restrict__ dq, StepShape sh,
                                                          int nsplit) {
  const int bh = blockIdx.x, b = bh / sh.heads, h = bh % sh.heads;
  const float* p0 = part + (int64_t)bh * nsplit * (sh.head_dim + 2);
  T* row = dq + b * sh.q_sb + h * sh.q_sh;
  for (int e = threadIdx.x; e < sh.head_dim; e += 64) {
    float acc = 0.f;
    for (int i = 0; i < nsplit; i++) acc += p0[i * (sh.head_dim + 2) + e];
    row[e] = from_f32<T>(acc);
  }
}

// Forward mode of the step: with p_s = exp(scale q.k_s - lse) from the saved lse,
// tS_s = scale (tq.k_s + q.tk_s), mu = sum_s p_s tS_s:
//   to = sum_s p_s (tS_s v_s + tv_s) - mu o.
// One pass over the keys of the block (k, v and the tangent caches read once); the block's
// partial sum and its share of mu go to `part`, the combine kernel finishes.  A null tangent
// pointer is a zero tangent.
template <typename T, bool VEC, int NCH>
__global__ __launch_bounds__(256) void attn_step_jvp_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                            const T* __restrict__ v, const float* __restrict__ lse,
                                                            const T* __restrict__ tq, const T* __restrict__ tk,
                                                            const T* __restrict__ tv, float* __restrict__ part, StepShape sh,
                                                            float scale) {
  using E = Elems<T, VEC>;
  using Raw = typename E::Raw;
  constexpr int NE = E::N, MAXC = NCH, U = NCH >= 2 ? 1 : 2;            // keys per slot and batch (four streams)
  __shared__ float red[kRedFloats];
  __shared__ float scratch[4];
  const int bh = blockIdx.y, b = bh / sh.heads, h = bh % sh.heads;
  const int s0 = blockIdx.x * kKeysPerBlock;
  const int s1 = s0 + kKeysPerBlock < sh.seq_kv ? s0 + kKeysPerBlock : sh.seq_kv;
  const int l16 = threadIdx.x & 15, slot = threadIdx.x >> 4;
  const int nchunks = sh.head_dim / NE;
  const int nch = (nchunks - l16 + 15) / 16;
  const int64_t qoff = b * sh.q_sb + h * sh.q_sh, kvoff = b * sh.kv_sb + h * sh.kv_sh;
  const float L = lse[bh];

  float qf[MAXC][NE], tqf[MAXC][NE];
  int coff[MAXC];
#pragma unroll
  for (int c = 0; c < MAXC; c++) {
    coff[c] = c < nch ? (l16 + 16 * c) * NE : 0;
#pragma unroll
    for (int e = 0; e < NE; e++) qf[c][e] = tqf[c][e] = 0.f;
    if (c < nch) {
      E::load(q + qoff + coff[c], qf[c]);
      if (tq) E::load(tq + qoff + coff[c], tqf[c]);
    }
  }
  float acc[MAXC][NE];
#pragma unroll
  for (int c = 0; c < MAXC; c++)
#pragma unroll
    for (int e = 0; e < NE; e++) acc[c][e] = 0.f;
  float mu = 0.f;
  // as in the adjoint kernel: two register sets, unconditional loads (clamped key, idle chunks against zero q, tq);
  // a null tangent cache is a block-uniform branch around its loads
  struct Set {
    Raw k[U][MAXC], v[U][MAXC], tk[U][MAXC], tv[U][MAXC];
  };
  auto issue = [&](int sb, Set& r) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int s = sb + 16 * u < s1 ? sb + 16 * u : s1 - 1;
      const int64_t row = kvoff + (int64_t)s * sh.kv_ss;
#pragma unroll
      for (int c = 0; c < MAXC; c++) {
        r.k[u][c] = E::load_raw(k + row + coff[c]);
        r.v[u][c] = E::load_raw(v + row + coff[c]);
        r.tk[u][c] = tk ? E::load_raw(tk + row + coff[c]) : E::zero_raw();
        r.tv[u][c] = tv ? E::load_raw(tv + row + coff[c]) : E::zero_raw();
      }
    }
  };
  auto consume = [&](int sb, const Set& r) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int s = sb + 16 * u;
      float dot = 0.f, tdot = 0.f;
#pragma unroll
      for (int c = 0; c < MAXC; c++) {
        float kf[NE], tkf[NE];
        E::unpack(r.k[u][c], kf);
        E::unpack(r.tk[u][c], tkf);
#pragma unroll
        for (int e = 0; e < NE; e++) {
          dot = fmaf(qf[c][e], kf[e], dot);
          tdot = fmaf(tqf[c][e], kf[e], tdot);
          tdot = fmaf(qf[c][e], tkf[e], tdot);
        }
      }
      dot = sum16(dot);
      tdot = sum16(tdot);
      if (s < s1) {
        const float p = __expf(dot * scale - L);
        const float w = p * tdot * scale;
        if (l16 == 0) mu += w;
#pragma unroll
        for (int c = 0; c < MAXC; c++)
          if (c < nch) {
            float vf[NE], tvf[NE];
            E::unpack(r.v[u][c], vf);
            E::unpack(r.tv[u][c], tvf);
#pragma unroll
            for (int e = 0; e < NE; e++) acc[c][e] = fmaf(w, vf[e], fmaf(p, tvf[e], acc[c][e]));
          }
      }
    }
  };
  {
    Set r0, r1;
    int sb = s0 + slot;
    issue(sb, r0);
    while (sb < s1) {
      const int sb1 = sb + 16 * U;
      if (sb1 < s1) issue(sb1, r1);
      consume(sb, r0);
      if (sb1 >= s1) break;
      sb = sb1 + 16 * U;
      if (sb < s1) issue(sb, r0);
      consume(sb1, r1);
    }
  }
  mu = block_sum(mu, scratch);
  reduce_keys<MAXC, NE>(acc, nch, red);
  float* out = part + ((int64_t)bh * gridDim.x + blockIdx.x) * (sh.head_dim + 2);
  if (threadIdx.x < 16) {
#pragma unroll
    for (int c = 0; c < MAXC; c++)
      if (c < nch) {
#pragma unroll
        for (int e = 0; e < NE; e++) out[(l16 + 16 * c) * NE + e] = acc[c][e];
      }
  }
  if (threadIdx.x == 0) out[sh.head_dim] = mu;
}

template <typename T>
__global__ __launch_bounds__(64) void attn_step_jvp_combine_kernel(const float* __restrict__ part, const T* __restrict__ o,
                                                                   T* __restrict__ to, StepShape sh, int nsplit) {
  const int bh = blockIdx.x, b = bh / sh.heads, h = bh % sh.heads;
  const float* p0 = part + (int64_t)bh * nsplit * (sh.head_dim + 2);
  const int64_t off = b * sh.q_sb + h * sh.q_sh;
  float mu = 0.f;
  for (int i = 0; i < nsplit; i++) mu += p0[i * (sh.head_dim + 2) + sh.head_dim];
  for (int e = threadIdx.x; e < sh.head_dim; e += 64) {
    float acc = 0.f;
    for (int i = 0; i < nsplit; i++) acc += p0[i * (sh.head_dim + 2) + e];
    to[off + e] = from_f32<T>(acc - mu * to_f32(o[off + e]));
  }
}

bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int check_step(const char* name, int64_t batch, int64_t heads, int64_t seq_kv, int64_t head_dim, int64_t q_sb, int64_t q_sh,
               int64_t kv_sb, int64_t kv_sh, int64_t kv_ss, int dtype) {
  EMI_REQUIRE(batch >= 0 && heads > 0 && seq_kv > 0 && head_dim > 0, "%s: bad shape [%lld,%lld,%lld,%lld]", name, (long long)batch,
              (long long)heads, (long long)seq_kv, (long long)head_dim);
  EMI_REQUIRE(dtype == EMI_F32 || dtype == EMI_BF16, "%s: unsupported dtype code %d (want 11=f32 or 16=bf16)", name, dtype);
  EMI_REQUIRE(head_dim <= 256, "%s: head_dim %lld > 256 is not supported", name, (long long)head_dim);
  EMI_REQUIRE(q_sh >= head_dim && q_sb > 0 && kv_ss >= head_dim && kv_sh > 0 && kv_sb > 0, "%s: bad strides", name);
  EMI_REQUIRE(batch * heads <= 65535 && seq_kv <= 0x7fffffff / 2, "%s: batch*heads or seq_kv too large", name);
  return EMI_OK;
}

}  // namespace
}  // namespace emi

using namespace emi;

extern "C" size_t emi_attn_step_workspace_bytes(int64_t batch, int64_t heads, int64_t seq_kv, int64_t head_dim) {
  if (batch <= 0 || heads <= 0 || seq_kv <= 0 || head_dim <= 0) return 0;
  const int64_t nsplit = (seq_kv + kKeysPerBlock - 1) / kKeysPerBlock;
  return (size_t)(batch * heads * nsplit * (head_dim + 2)) * sizeof(float);
}

extern "C" int emi_attn_step_fwd(emi_stream_t stream, const void* q, const void* k, const void* v, void* o, float* lse,
                                 void* workspace, size_t workspace_bytes, int64_t batch, int64_t heads, int64_t seq_kv,
                                 int64_t head_dim, int64_t q_stride_b, int64_t q_stride_h, int64_t kv_stride_b,
                                 int64_t kv_stride_h, int64_t kv_stride_s, float scale, int dtype) {
  if (int rc = check_step("emi_attn_step_fwd", batch, heads, seq_kv, head_dim, q_stride_b, q_stride_h, kv_stride_b, kv_stride_h,
                          kv_stride_s, dtype))
    return rc;
  if (batch == 0) return EMI_OK;
  EMI_REQUIRE(q && k && v && o && lse, "emi_attn_step_fwd: null buffer");
  const size_t need = emi_attn_step_workspace_bytes(batch, heads, seq_kv, head_dim);
  EMI_REQUIRE(workspace != nullptr && workspace_bytes >= need, "emi_attn_step_fwd: workspace of %zu bytes needed, got %zu", need,
              workspace_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const StepShape sh{(int)heads, (int)seq_kv, (int)head_dim, q_stride_b, q_stride_h, kv_stride_b, kv_stride_h, kv_stride_s};
  const int ne = dtype == EMI_BF16 ? 8 : 4;
  const bool vec = head_dim % ne == 0 && q_stride_b % ne == 0 && q_stride_h % ne == 0 && kv_stride_b % ne == 0 &&
                   kv_stride_h % ne == 0 && kv_stride_s % ne == 0 && al16(q) && al16(k) && al16(v);
  const int nsplit = (int)((seq_kv + kKeysPerBlock - 1) / kKeysPerBlock);
  const dim3 grid((unsigned)nsplit, (unsigned)(batch * heads));
  float* part = static_cast<float*>(workspace);
#define EMI_STEP_FWD(T, VEC, NCH)                                                                                       \
  do {                                                                                                                   \
    hipLaunchKernelGGL((attn_step_fwd_kernel<T, VEC, NCH>), grid, dim3(256), 0, st, (const T*)q, (const T*)k,            \
                       (const T*)v, part, sh, scale);                                                                    \
    EMI_CHECK_LAUNCH("emi_attn_step_fwd");                                                                               \
    hipLaunchKernelGGL(attn_step_combine_kernel<T>, dim3((unsigned)(batch * heads)), dim3(64), 0, st, part, (T*)o, lse,  \
                       sh, nsplit);                                                                                      \
  } while (0)
#define EMI_STEP_FWD1(T)                                                                                                \
  do {                                                                                                                   \
    hipLaunchKernelGGL(attn_step_fwd1_kernel<T>, grid, dim3(256), 0, st, (const T*)q, (const T*)k, (const T*)v, part,    \
                       sh, scale);                                                                                       \
    EMI_CHECK_LAUNCH("emi_attn_step_fwd");                                                                               \
    hipLaunchKernelGGL(attn_step_combine_kernel<T>, dim3((unsigned)(batch * heads)), dim3(64), 0, st, part, (T*)o, lse,  \
                       sh, nsplit);                                                                                      \
  } while (0)
#define EMI_STEP_FWD_T(T)                                              \
  do {                                                                 \
    if (!vec) EMI_STEP_FWD(T, false, 16);                              \
    else if (nch <= 1) EMI_STEP_FWD1(T);                               \
    else if (nch <= 2) EMI_STEP_FWD(T, true, 2);                       \
    else EMI_STEP_FWD(T, true, 4);                                     \
  } while (0)
  const int nch = (int)((head_dim / ne + 15) / 16);      // 16-byte chunks per lane
  if (dtype == EMI_BF16) EMI_STEP_FWD_T(bf16);
  else EMI_STEP_FWD_T(float);
#undef EMI_STEP_FWD_T
#undef EMI_STEP_FWD1
#undef EMI_STEP_FWD
  EMI_CHECK_LAUNCH("emi_attn_step_fwd(combine)");
  return EMI_OK;
}

extern "C" int emi_attn_step_bwd(emi_stream_t stream, const void* q, const void* k, const void* v, const void* o,
                                 const float* lse, const void* d_o, void* dq, void* dk, void* dv, void* workspace,
                                 size_t workspace_bytes, int64_t batch, int64_t heads, int64_t seq_kv, int64_t head_dim,
                                 int64_t q_stride_b, int64_t q_stride_h, int64_t kv_stride_b, int64_t kv_stride_h,
                                 int64_t kv_stride_s, float scale, int dtype) {
  if (int rc = check_step("emi_attn_step_bwd", batch, heads, seq_kv, head_dim, q_stride_b, q_stride_h, kv_stride_b, kv_stride_h,
                          kv_stride_s, dtype))
    return rc;
  if (batch == 0) return EMI_OK;
  EMI_REQUIRE(q && k && v && o && lse && d_o && dq && dk && dv, "emi_attn_step_bwd: null buffer");
  const size_t need = emi_attn_step_workspace_bytes(batch, heads, seq_kv, head_dim);
  EMI_REQUIRE(workspace != nullptr && workspace_bytes >= need, "emi_attn_step_bwd: workspace of %zu bytes needed, got %zu", need,
              workspace_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const StepShape sh{(int)heads, (int)seq_kv, (int)head_dim, q_stride_b, q_stride_h, kv_stride_b, kv_stride_h, kv_stride_s};
  const int ne = dtype == EMI_BF16 ? 8 : 4;
  const bool vec = head_dim % ne == 0 && q_stride_b % ne == 0 && q_stride_h % ne == 0 && kv_stride_b % ne == 0 &&
                   kv_stride_h % ne == 0 && kv_stride_s % ne == 0 && al16(q) && al16(k) && al16(v) && al16(o) && al16(d_o) &&
                   al16(dk) && al16(dv);
  const int nsplit = (int)((seq_kv + kKeysPerBlock - 1) / kKeysPerBlock);
  const dim3 grid((unsigned)nsplit, (unsigned)(batch * heads));
  float* part = static_cast<float*>(workspace);
#define EMI_STEP_BWD(T, VEC, NCH)                                                                                       \
  do {                                                                                                                   \
    hipLaunchKernelGGL((attn_step_bwd_kernel<T, VEC, NCH>), grid, dim3(256), 0, st, (const T*)q, (const T*)k,            \
                       (const T*)v, (const T*)o, lse, (const T*)d_o, part, (T*)dk, (T*)dv, sh, scale);                   \
    EMI_CHECK_LAUNCH("emi_attn_step_bwd");                                                                               \
    hipLaunchKernelGGL(attn_step_dq_kernel<T>, dim3((unsigned)(batch * heads)), dim3(64), 0, st, part, (T*)dq, sh,       \
                       nsplit);                                                                                          \
  } while (0)
#define EMI_STEP_BWD_T(T)                                              \
  do {                                                                 \
    if (!vec) EMI_STEP_BWD(T, false, 16);                              \
    else if (nch <= 1) EMI_STEP_BWD(T, true, 1);                       \
    else if (nch <= 2) EMI_STEP_BWD(T, true, 2);                       \
    else EMI_STEP_BWD(T, true, 4);                                     \
  } while (0)
  const int nch = (int)((head_dim / ne + 15) / 16);      // 16-byte chunks per lane
  if (dtype == EMI_BF16) EMI_STEP_BWD_T(bf16);
  else EMI_STEP_BWD_T(float);
#undef EMI_STEP_BWD_T
#undef EMI_STEP_BWD
  EMI_CHECK_LAUNCH("emi_attn_step_bwd(dq)");
  return EMI_OK;
}

extern "C" int emi_attn_step_jvp(emi_stream_t stream, const void* q, const void* k, const void* v, const void* o,
                                 const float* lse, const void* tq, const void* tk, const void* tv, void* to, void* workspace,
                                 size_t workspace_bytes, int64_t batch, int64_t heads, int64_t seq_kv, int64_t head_dim,
                                 int64_t q_stride_b, int64_t q_stride_h, int64_t kv_stride_b, int64_t kv_stride_h,
                                 int64_t kv_stride_s, float scale, int dtype) {
  if (int rc = check_step("emi_attn_step_jvp", batch, heads, seq_kv, head_dim, q_stride_b, q_stride_h, kv_stride_b, kv_stride_h,
                          kv_stride_s, dtype))
    return rc;
  if (batch == 0) return EMI_OK;
  EMI_REQUIRE(q && k && v && o && lse && to, "emi_attn_step_jvp: null buffer");
  const size_t need = emi_attn_step_workspace_bytes(batch, heads, seq_kv, head_dim);
  EMI_REQUIRE(workspace != nullptr && workspace_bytes >= need, "emi_attn_step_jvp: workspace of %zu bytes needed, got %zu", need,
              workspace_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const StepShape sh{(int)heads, (int)seq_kv, (int)head_dim, q_stride_b, q_stride_h, kv_stride_b, kv_stride_h, kv_stride_s};
  const int ne = dtype == EMI_BF16 ? 8 : 4;
  const bool vec = head_dim % ne == 0 && q_stride_b % ne == 0 && q_stride_h % ne == 0 && kv_stride_b % ne == 0 &&
                   kv_stride_h % ne == 0 && kv_stride_s % ne == 0 && al16(q) && al16(k) && al16(v) && al16(tq) && al16(tk) &&
                   al16(tv);
  const int nsplit = (int)((seq_kv + kKeysPerBlock - 1) / kKeysPerBlock);
  const dim3 grid((unsigned)nsplit, (unsigned)(batch * heads));
  float* part = static_cast<float*>(workspace);
#define EMI_STEP_JVP(T, VEC, NCH)                                                                                       \
  do {                                                                                                                   \
    hipLaunchKernelGGL((attn_step_jvp_kernel<T, VEC, NCH>), grid, dim3(256), 0, st, (const T*)q, (const T*)k,            \
                       (const T*)v, lse, (const T*)tq, (const T*)tk, (const T*)tv, part, sh, scale);                     \
    EMI_CHECK_LAUNCH("emi_attn_step_jvp");                                                                               \
    hipLaunchKernelGGL(attn_step_jvp_combine_kernel<T>, dim3((unsigned)(batch * heads)), dim3(64), 0, st, part,          \
                       (const T*)o, (T*)to, sh, nsplit);                                                                 \
  } while (0)
#define EMI_STEP_JVP_T(T)                                              \
  do {                                                                 \
    if (!vec) EMI_STEP_JVP(T, false, 16);                              \
    else if (nch <= 1) EMI_STEP_JVP(T, true, 1);                       \
    else if (nch <= 2) EMI_STEP_JVP(T, true, 2);                       \
    else EMI_STEP_JVP(T, true, 4);                                     \
  } while (0)
  const int nch = (int)((head_dim / ne + 15) / 16);      // 16-byte chunks per lane
  if (dtype == EMI_BF16) EMI_STEP_JVP_T(bf16);
  else EMI_STEP_JVP_T(float);
#undef EMI_STEP_JVP_T
#undef EMI_STEP_JVP
  EMI_CHECK_LAUNCH("emi_attn_step_jvp(combine)");
  return EMI_OK;
}
