// Causal softmax attention in fp32 on the matrix cores, forward and adjoint, for gfx950:
// v_mfma_f32_16x16x4_f32 with fp32 operands and fp32 accumulation (no narrower arithmetic anywhere),
// for head_dim a multiple of 16 up to 128 and rows that start on 16-byte boundaries.  Replaces the per-head
// loop of test/llama.py:178-206 with the softmax of :13-18 for the fp32 configurations (stories15M: 6 heads x 48).
//
// One wavefront owns 16 queries (forward, dQ) or 16 keys (dK/dV) and walks the other sequence axis 64 rows
// at a time; operands come straight from global memory (L1/L2 serve the reuse between wavefronts), so there is
// no LDS and no barrier.  As on the bf16 path everything is computed transposed: the score tile is
// S^T[other row, own row], so lane l owns row l % 16 for its whole life, its softmax statistics are per-lane
// scalars, and the probabilities leave the accumulator already in the B-operand layout of the second product.
//
// Operand layouts of v_mfma_f32_16x16x4_f32 (D = A . B, A 16x4, B 4x16): lane l supplies A[l % 16][l / 16] and
// B[l / 16][l % 16]; register r of lane l receives D[4 (l / 16) + r][l % 16].  The contraction index of one
// instruction is the lane group g = l / 16; which four columns (or rows) of the operand tensors the four
// groups stand for is free as long as A and B agree:
//   * products over head_dim (scores, dP): instruction (c, t) contracts columns 16 c + 4 g + t, so a lane reads
//     its row in 16-byte pieces;
//   * products over the other sequence axis (P.V, dS.K, P^T.dO, dS^T.Q): instruction t of a 16-row tile contracts
//     rows 4 g + t, which is exactly where register t of the score accumulator lives, and the output column of
//     A-row i in pass n is NT i + n (NT = head_dim / 16), so a lane reads and writes NT consecutive elements.
#include <initializer_list>
#include <stdint.h>

#include "emi_device.h"

namespace emi {

typedef float f32q_t __attribute__((ext_vector_type(4)));

struct AttnShapeF32 {
  int seq, heads;
  int64_t sb, sh, ss;   // element strides of batch, head, sequence position
};

constexpr float kMasked = -1.0e30f;

__device__ __forceinline__ f32q_t mfma_f32(float a, float b, f32q_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// Rows row0 .. row0 + 15 (clamped to `last`) as an operand contracted over head_dim: f[c][t] of lane l is
// element (row0 + l % 16, 16 c + 4 (l / 16) + t).
template <int NT>
__device__ __forceinline__ void load_rows(const float* __restrict__ head, int64_t ss, int row0, int last, int lane,
                                          float (&f)[NT][4]) {
  int r = row0 + (lane & 15);
  r = r < last ? r : last;
  const float* p = head + (int64_t)r * ss + 4 * (lane >> 4);
#pragma unroll
  for (int c = 0; c < NT; c++) {
    const float4 x = *reinterpret_cast<const float4*>(p + 16 * c);
    f[c][0] = x.x; f[c][1] = x.y; f[c][2] = x.z; f[c][3] = x.w;
  }
}

// X . Y^T for two 16-row operands: register r of lane l is the dot product of X row 4 (l / 16) + r and Y row l % 16.
template <int NT>
__device__ __forceinline__ f32q_t rows_dot(const float (&x)[NT][4], const float (&y)[NT][4]) {
  f32q_t s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c = 0; c < NT; c++)
#pragma unroll
    for (int t = 0; t < 4; t++) s = mfma_f32(x[c][t], y[c][t], s);
  return s;
}

// acc += X[row0 .. row0 + 15]^T . W, where w[t] of lane l is W[row0 + 4 (l / 16) + t][l % 16] (the layout rows_dot
// leaves): acc[n][r] of lane l is output element (own row l % 16, column NT (4 (l / 16) + r) + n).
template <int NT>
__device__ __forceinline__ void add_cols(const float* __restrict__ head, int64_t ss, int row0, int last, int lane,
                                         const f32q_t w, f32q_t (&acc)[NT]) {
#pragma unroll
  for (int t = 0; t < 4; t++) {
    int r = row0 + 4 * (lane >> 4) + t;
    r = r < last ? r : last;                 // rows past the end carry weight 0
    const float* p = head + (int64_t)r * ss + NT * (lane & 15);
    float x[NT];
#pragma unroll
    for (int n = 0; n < NT; n++) x[n] = p[n];
#pragma unroll
    for (int n = 0; n < NT; n++) acc[n] = mfma_f32(x[n], w[t], acc[n]);
  }
}

// The two halves of add_cols, for callers that issue the loads well before the weights exist.
template <int NT>
__device__ __forceinline__ void load_cols(const float* __restrict__ head, int64_t ss, int row0, int last, int lane,
                                          float (&x)[4][NT]) {
#pragma unroll
  for (int t = 0; t < 4; t++) {
    int r = row0 + 4 * (lane >> 4) + t;
    r = r < last ? r : last;
    const float* p = head + (int64_t)r * ss + NT * (lane & 15);
#pragma unroll
    for (int n = 0; n < NT; n++) x[t][n] = p[n];
  }
}
template <int NT>
__device__ __forceinline__ void mma_cols(const float (&x)[4][NT], const f32q_t w, f32q_t (&acc)[NT]) {
#pragma unroll
  for (int t = 0; t < 4; t++)
#pragma unroll
    for (int n = 0; n < NT; n++) acc[n] = mfma_f32(x[t][n], w[t], acc[n]);
}

template <int NT>
__device__ __forceinline__ void store_cols(float* __restrict__ row, int lane, const f32q_t (&acc)[NT], float mul) {
#pragma unroll
  for (int r = 0; r < 4; r++) {
    float* p = row + NT * (4 * (lane >> 4) + r);
#pragma unroll
    for (int n = 0; n < NT; n++) p[n] = acc[n][r] * mul;
  }
}

__device__ __forceinline__ float groups_max(float x) {      // over the four lanes that share l % 16
  x = fmaxf(x, __shfl_xor(x, 16, 64));
  return fmaxf(x, __shfl_xor(x, 32, 64));
}
__device__ __forceinline__ float groups_sum(float x) {
  x += __shfl_xor(x, 16, 64);
  return x + __shfl_xor(x, 32, 64);
}

// Forward: o = softmax(scale q k^T) v, lse = log-sum-exp of the scaled scores.
template <int NT>
__global__ __launch_bounds__(64) void attn_fwd_f32_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                          const float* __restrict__ v, float* __restrict__ o,
                                                          float* __restrict__ lse, AttnShapeF32 sh, float scale, int causal) {
  const int lane = threadIdx.x, G = lane >> 4;
  const int q0 = (int)(gridDim.x - 1 - blockIdx.x) * 16;          // longest causal rows first
  const int bh = blockIdx.y;
  const int64_t base = (int64_t)(bh / sh.heads) * sh.sb + (int64_t)(bh % sh.heads) * sh.sh;
  const int last = sh.seq - 1;
  const int myq = q0 + (lane & 15);
  float qf[NT][4];
  load_rows<NT>(q + base, sh.ss, q0, last, lane, qf);
  const int nkeys = causal ? (q0 + 16 < sh.seq ? q0 + 16 : sh.seq) : sh.seq;
  float m = kMasked, lsum = 0.f;
  f32q_t acc[NT];
#pragma unroll
  for (int n = 0; n < NT; n++) acc[n] = f32q_t{0.f, 0.f, 0.f, 0.f};
  constexpr bool AHEAD = NT <= 4;      // head_dim <= 64: all K and V operands of a 64-key step fit in registers, so
                                       // their loads are issued together and the step waits for memory once
  for (int k0 = 0; k0 < nkeys; k0 += 64) {
    f32q_t s[4];
    float mx = kMasked;
    float kfa[AHEAD ? 4 : 1][NT][4], vxa[AHEAD ? 4 : 1][4][NT];
    if constexpr (AHEAD) {
#pragma unroll
      for (int kt = 0; kt < 4; kt++)
        if (k0 + 16 * kt < nkeys) load_rows<NT>(k + base, sh.ss, k0 + 16 * kt, last, lane, kfa[kt]);
#pragma unroll
      for (int kt = 0; kt < 4; kt++)
        if (k0 + 16 * kt < nkeys) load_cols<NT>(v + base, sh.ss, k0 + 16 * kt, last, lane, vxa[kt]);
    }
#pragma unroll
    for (int kt = 0; kt < 4; kt++) {
      const int kb = k0 + 16 * kt;
      if (kb < nkeys) {
        if constexpr (AHEAD) {
          s[kt] = rows_dot<NT>(kfa[kt], qf);
        } else {
          float kf[NT][4];
          load_rows<NT>(k + base, sh.ss, kb, last, lane, kf);
          s[kt] = rows_dot<NT>(kf, qf);
        }
      } else {
        s[kt] = f32q_t{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int key = kb + 4 * G + r;
        const bool valid = key < nkeys && (!causal || key <= myq);
        s[kt][r] = valid ? s[kt][r] * scale : kMasked;
        mx = fmaxf(mx, s[kt][r]);
      }
    }
    // key 0 is visible to every query, so the running maximum is finite from the first tile on
    const float m_new = fmaxf(m, groups_max(mx));
    const float alpha = expf(m - m_new);
    float psum = 0.f;
#pragma unroll
    for (int kt = 0; kt < 4; kt++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        s[kt][r] = expf(s[kt][r] - m_new);
        psum += s[kt][r];
      }
    lsum = lsum * alpha + psum;               // this lane's share of the row sum; the groups are added at the end
#pragma unroll
    for (int n = 0; n < NT; n++) acc[n] *= alpha;
#pragma unroll
    for (int kt = 0; kt < 4; kt++)
      if (k0 + 16 * kt < nkeys) {
        if constexpr (AHEAD) mma_cols<NT>(vxa[kt], s[kt], acc);
        else add_cols<NT>(v + base, sh.ss, k0 + 16 * kt, last, lane, s[kt], acc);
      }
    m = m_new;
  }
  lsum = groups_sum(lsum);
  if (myq < sh.seq) {
    store_cols<NT>(o + base + (int64_t)myq * sh.ss, lane, acc, 1.f / lsum);
    if (G == 0) lse[(int64_t)bh * sh.seq + myq] = m + logf(lsum);
  }
}

// dQ = scale dS K with dS = P (dP - delta), P = exp(scale q k^T - lse), dP = dO V^T.
template <int NT>
__global__ __launch_bounds__(64) void attn_bwd_dq_f32_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                             const float* __restrict__ v, const float* __restrict__ d_o,
                                                             const float* __restrict__ lse, const float* __restrict__ delta,
                                                             float* __restrict__ dq, AttnShapeF32 sh, float scale,
                                                             int causal) {
  const int lane = threadIdx.x, G = lane >> 4;
  const int q0 = (int)(gridDim.x - 1 - blockIdx.x) * 16;
  const int bh = blockIdx.y;
  const int64_t base = (int64_t)(bh / sh.heads) * sh.sb + (int64_t)(bh % sh.heads) * sh.sh;
  const int last = sh.seq - 1;
  const int myq = q0 + (lane & 15);
  const int qc = myq < last ? myq : last;
  float qf[NT][4], dof[NT][4];
  load_rows<NT>(q + base, sh.ss, q0, last, lane, qf);
  load_rows<NT>(d_o + base, sh.ss, q0, last, lane, dof);
  const float L = lse[(int64_t)bh * sh.seq + qc], dl = delta[(int64_t)bh * sh.seq + qc];
  const int nkeys = causal ? (q0 + 16 < sh.seq ? q0 + 16 : sh.seq) : sh.seq;
  f32q_t acc[NT];
#pragma unroll
  for (int n = 0; n < NT; n++) acc[n] = f32q_t{0.f, 0.f, 0.f, 0.f};
  // U key tiles per step, all their operands requested before the first product (one wait for memory per step)
  constexpr int U = NT <= 3 ? 4 : (NT <= 4 ? 2 : 1);      // (166 registers at NT = 4: three wavefronts per SIMD)
  for (int kb0 = 0; kb0 < nkeys; kb0 += 16 * U) {
    float kf[U][NT][4], vf[U][NT][4], kx[U][4][NT];
#pragma unroll
    for (int u = 0; u < U; u++)
      if (kb0 + 16 * u < nkeys) {
        load_rows<NT>(k + base, sh.ss, kb0 + 16 * u, last, lane, kf[u]);
        load_rows<NT>(v + base, sh.ss, kb0 + 16 * u, last, lane, vf[u]);
        load_cols<NT>(k + base, sh.ss, kb0 + 16 * u, last, lane, kx[u]);        // for dQ += dS . K
      }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int kb = kb0 + 16 * u;
      if (kb >= nkeys) break;
      f32q_t s = rows_dot<NT>(kf[u], qf);
      const f32q_t dp = rows_dot<NT>(vf[u], dof);
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int key = kb + 4 * G + r;
        const bool valid = key < nkeys && (!causal || key <= myq);
        const float p = valid ? expf(s[r] * scale - L) : 0.f;
        s[r] = p * (dp[r] - dl) * scale;
      }
      mma_cols<NT>(kx[u], s, acc);
    }
  }
  if (myq < sh.seq) store_cols<NT>(dq + base + (int64_t)myq * sh.ss, lane, acc, 1.f);
}

// dV = P^T dO, dK = scale dS^T Q: one wavefront per 16 keys, walking the queries that see them.
template <int NT>
__global__ __launch_bounds__(64) void attn_bwd_dkv_f32_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                              const float* __restrict__ v, const float* __restrict__ d_o,
                                                              const float* __restrict__ lse, const float* __restrict__ delta,
                                                              float* __restrict__ dk, float* __restrict__ dv,
                                                              AttnShapeF32 sh, float scale, int causal) {
  const int lane = threadIdx.x, G = lane >> 4;
  const int key0 = (int)blockIdx.x * 16;                           // the earliest keys see the most queries
  const int bh = blockIdx.y;
  const int64_t base = (int64_t)(bh / sh.heads) * sh.sb + (int64_t)(bh % sh.heads) * sh.sh;
  const int last = sh.seq - 1;
  const int mykey = key0 + (lane & 15);
  float kf[NT][4], vf[NT][4];
  load_rows<NT>(k + base, sh.ss, key0, last, lane, kf);
  load_rows<NT>(v + base, sh.ss, key0, last, lane, vf);
  const float* lrow = lse + (int64_t)bh * sh.seq;
  const float* drow = delta + (int64_t)bh * sh.seq;
  f32q_t acck[NT], accv[NT];
#pragma unroll
  for (int n = 0; n < NT; n++) acck[n] = accv[n] = f32q_t{0.f, 0.f, 0.f, 0.f};
  // U query tiles per step, operands (and the rows' lse / delta) requested together; two tiles only while the
  // registers allow three wavefronts per SIMD to stay resident
  constexpr int U = NT <= 3 ? 2 : 1;
  for (int qb0 = causal ? key0 : 0; qb0 < sh.seq; qb0 += 16 * U) {
    float qf[U][NT][4], dof[U][NT][4], qx[U][4][NT], dox[U][4][NT], lq[U][4], dq_[U][4];
#pragma unroll
    for (int u = 0; u < U; u++)
      if (qb0 + 16 * u < sh.seq) {
        load_rows<NT>(q + base, sh.ss, qb0 + 16 * u, last, lane, qf[u]);
        load_rows<NT>(d_o + base, sh.ss, qb0 + 16 * u, last, lane, dof[u]);
        load_cols<NT>(d_o + base, sh.ss, qb0 + 16 * u, last, lane, dox[u]);    // for dV += P^T . dO
        load_cols<NT>(q + base, sh.ss, qb0 + 16 * u, last, lane, qx[u]);       // for dK += dS^T . Q
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const int qi = qb0 + 16 * u + 4 * G + r;
          const int qc = qi < last ? qi : last;
          lq[u][r] = lrow[qc];
          dq_[u][r] = drow[qc];
        }
      }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int qb = qb0 + 16 * u;
      if (qb >= sh.seq) break;
      f32q_t s = rows_dot<NT>(qf[u], kf);               // register r: query qb + 4 G + r, key mykey
      f32q_t dp = rows_dot<NT>(dof[u], vf);
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int qi = qb + 4 * G + r;
        const bool valid = qi < sh.seq && (!causal || mykey <= qi);
        const float p = valid ? expf(s[r] * scale - lq[u][r]) : 0.f;
        s[r] = p;
        dp[r] = p * (dp[r] - dq_[u][r]) * scale;
      }
      mma_cols<NT>(dox[u], s, accv);
      mma_cols<NT>(qx[u], dp, acck);
    }
  }
  if (mykey < sh.seq) {
    store_cols<NT>(dk + base + (int64_t)mykey * sh.ss, lane, acck, 1.f);
    store_cols<NT>(dv + base + (int64_t)mykey * sh.ss, lane, accv, 1.f);
  }
}

static bool f32_mfma_ok(int64_t seq, int64_t d, int64_t sb, int64_t shh, int64_t ss, std::initializer_list<const void*> ptrs) {
  if (d % 16 != 0 || d > 128 || seq < 1) return false;
  if ((sb | shh | ss) & 3) return false;
  for (const void* p : ptrs)
    if (reinterpret_cast<uintptr_t>(p) & 15) return false;
  return true;
}

#define EMI_ATTN_F32_DISPATCH(NTV, CALL)      \
  switch (NTV) {                              \
    case 1: { constexpr int NT = 1; CALL; break; } \
    case 2: { constexpr int NT = 2; CALL; break; } \
    case 3: { constexpr int NT = 3; CALL; break; } \
    case 4: { constexpr int NT = 4; CALL; break; } \
    case 5: { constexpr int NT = 5; CALL; break; } \
    case 6: { constexpr int NT = 6; CALL; break; } \
    case 7: { constexpr int NT = 7; CALL; break; } \
    default: { constexpr int NT = 8; CALL; break; } \
  }

// Forward on the fp32 matrix-core path; -1 when the operands do not qualify (the caller then takes the
// one-wavefront-per-row kernel).
int launch_attn_fwd_f32_mfma(hipStream_t st, const void* q, const void* k, const void* v, void* o, float* lse, int64_t batch,
                             int64_t heads, int64_t seq, int64_t head_dim, int64_t sb, int64_t shh, int64_t ss, float scale,
                             int causal) {
  if (!f32_mfma_ok(seq, head_dim, sb, shh, ss, {q, k, v, o})) return -1;
  const AttnShapeF32 shp{(int)seq, (int)heads, sb, shh, ss};
  const dim3 grid((unsigned)((seq + 15) / 16), (unsigned)(batch * heads));
  EMI_ATTN_F32_DISPATCH((int)(head_dim / 16),
                        hipLaunchKernelGGL(attn_fwd_f32_kernel<NT>, grid, dim3(64), 0, st, (const float*)q, (const float*)k,
                                           (const float*)v, (float*)o, lse, shp, scale, causal));
  EMI_CHECK_LAUNCH("emi_attn_fwd(fp32 mfma)");
  return EMI_OK;
}

// dQ, dK, dV on the fp32 matrix-core path given delta = rowsum(dO * O); -1 when the operands do not qualify.
int launch_attn_bwd_f32_mfma(hipStream_t st, const void* q, const void* k, const void* v, const void* d_o, const float* lse,
                             const float* delta, void* dq, void* dk, void* dv, int64_t batch, int64_t heads, int64_t seq,
                             int64_t head_dim, int64_t sb, int64_t shh, int64_t ss, float scale, int causal) {
  if (!f32_mfma_ok(seq, head_dim, sb, shh, ss, {q, k, v, d_o, dq, dk, dv})) return -1;
  const AttnShapeF32 shp{(int)seq, (int)heads, sb, shh, ss};
  const dim3 grid((unsigned)((seq + 15) / 16), (unsigned)(batch * heads));
  EMI_ATTN_F32_DISPATCH((int)(head_dim / 16),
                        hipLaunchKernelGGL(attn_bwd_dkv_f32_kernel<NT>, grid, dim3(64), 0, st, (const float*)q, (const float*)k,
                                           (const float*)v, (const float*)d_o, lse, delta, (float*)dk, (float*)dv, shp, scale,
                                           causal));
  EMI_CHECK_LAUNCH("emi_attn_bwd(fp32 mfma dkv)");
  EMI_ATTN_F32_DISPATCH((int)(head_dim / 16),
                        hipLaunchKernelGGL(attn_bwd_dq_f32_kernel<NT>, grid, dim3(64), 0, st, (const float*)q, (const float*)k,
                                           (const float*)v, (const float*)d_o, lse, delta, (float*)dq, shp, scale, causal));
  EMI_CHECK_LAUNCH("emi_attn_bwd(fp32 mfma dq)");
  return EMI_OK;
}

}  // namespace emi
