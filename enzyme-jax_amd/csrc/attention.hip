// Causal softmax attention, forward and adjoint, for gfx950.
//
// Fast path (bf16, head_dim 64 or 128): flash-style, scores never leave the
// CU.  Everything is computed "transposed" so that one lane owns one query
// (forward, dQ) or one key (dK/dV) for its whole life:
//   S^T[key,query] = K . Q^T     MFMA A = K rows from LDS, B = Q in registers
//   O^T[d,query]   = V^T . P^T   MFMA A = V columns via the transposing LDS
//                                load, B = P straight from the accumulator
// so the softmax row statistics are per-lane scalars (one exchange with lane
// ^32 per tile) and rescaling O needs no cross-lane traffic.  K/V (or Q/dO)
// tiles stream HBM -> LDS with 16-byte direct-to-LDS loads, double buffered.
// The adjoint is atomics-free and deterministic: one kernel owns query blocks
// and produces dQ, another owns key blocks and produces dK and dV; both
// recompute P from q, k and the saved log-sum-exp.
//
// fp32 with head_dim a multiple of 16 (up to 128): attention_f32.hip, the same scheme on the fp32 matrix
// instruction.  Generic path (any other head_dim <= 256 or unaligned rows): one wavefront per query
// (or key) row, plain fp32 FMA, same maths.
#include <initializer_list>
#include <type_traits>
#include <utility>
#include <stdlib.h>

#include "emi_device.h"

namespace emi {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(8 * sizeof(float)))) float f32x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

#define EMI_LDS __attribute__((address_space(3)))

constexpr uint32_t kOobA = 0x80000000u;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kNegBig = -1.0e30f;

struct AttnShape {
  int seq, heads;
  int64_t sb, sh, ss;   // element strides of batch, head, sequence position
};

// Work assignment of the MFMA kernels.  Consecutive workgroup ids go to different XCDs
// (8 of them, each with its own L2), so a grid of (blocks per head) x (heads) that simply
// used blockIdx would hand every XCD the same few block positions of every head: with a
// causal mask that is a 2.4x imbalance between XCDs, and K/V of one head would be
// fetched into all eight L2s.  Instead every XCD gets a contiguous run of heads with all
// of their blocks, in the order given (longest first).
__device__ __forceinline__ void attn_block_coords(int* blk, int* bh) {
  const int nblk = gridDim.x, nbh = gridDim.y, total = nblk * nbh;
  const int lin = blockIdx.y * gridDim.x + blockIdx.x;
  const int per = total >> 3, rem = total & 7;
  const int xcd = lin & 7, idx = lin >> 3;
  const int v = xcd * per + (xcd < rem ? xcd : rem) + idx;
  // Heads are taken in groups of four and, inside a group, block positions go first
  // (the four longest blocks, then the four next longest, ...): list scheduling of
  // head-major order leaves the CUs of a XCD up to 10% apart at the end, this order
  // does not, and four heads of K/V still fit in the L2.
  constexpr int G = 4;
  const int g = v / (G * nblk), r = v - g * G * nblk;
  const int gh = nbh - g * G < G ? nbh - g * G : G;
  *blk = r / gh;
  *bh = g * G + (r - *blk * gh);
}

// ===========================================================================
// Generic path
// ===========================================================================

// Four consecutive elements as fp32 (8- or 16-byte load; the caller guarantees the alignment).
__device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
}
__device__ __forceinline__ void load4(const bf16* p, float (&v)[4]) {
  const uint2 a = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
  v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
}

// a . b and c . e over d elements (rows of two operand pairs that are always needed together); vec4: rows
// start on 4-element boundaries and d is a multiple of 4, so the loads are 4 elements wide.
template <typename T, bool TWO>
__device__ __forceinline__ void row_dots(const T* a, const T* b, const T* c, const T* e, int d, bool vec4, float* ab,
                                         float* ce) {
  float s0 = 0.f, s1 = 0.f;
  int i = 0;
  if (vec4) {
#pragma unroll 4
    for (; i + 4 <= d; i += 4) {
      float x[4], y[4];
      load4(a + i, x);
      load4(b + i, y);
      s0 += x[0] * y[0] + x[1] * y[1] + x[2] * y[2] + x[3] * y[3];
      if constexpr (TWO) {
        load4(c + i, x);
        load4(e + i, y);
        s1 += x[0] * y[0] + x[1] * y[1] + x[2] * y[2] + x[3] * y[3];
      }
    }
  }
  for (; i < d; i++) {
    s0 += to_f32(a[i]) * to_f32(b[i]);
    if constexpr (TWO) s1 += to_f32(c[i]) * to_f32(e[i]);
  }
  *ab = s0;
  if constexpr (TWO) *ce = s1;
}

// One wavefront per query.  Lanes split the keys of a 64-key chunk for the
// scores and split head_dim for the output (four rows of V in flight at a time).
template <typename T>
__global__ __launch_bounds__(256) void attn_fwd_generic_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                               const T* __restrict__ v, T* __restrict__ o,
                                                               float* __restrict__ lse, AttnShape sh, int d, float scale,
                                                               int causal, int vec4) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int qi = blockIdx.x * 4 + wave;
  const int bh = blockIdx.y;
  if (qi >= sh.seq) return;
  const int64_t base = (int64_t)(bh / sh.heads) * sh.sb + (int64_t)(bh % sh.heads) * sh.sh;
  const T* qr = q + base + (int64_t)qi * sh.ss;
  const int nkeys = causal ? qi + 1 : sh.seq;
  float m = kNegBig, l = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < nkeys; k0 += 64) {
    const int key = k0 + lane;
    float s = kNegBig;
    if (key < nkeys) {
      float dot;
      row_dots<T, false>(qr, k + base + (int64_t)key * sh.ss, qr, qr, d, vec4 != 0, &dot, nullptr);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float alpha = expf(m - m_new);
    const float p = key < nkeys ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int c = 0; c < 4; c++) acc[c] *= alpha;
    const int cnt = nkeys - k0 < 64 ? nkeys - k0 : 64;
    for (int j = 0; j < cnt; j += 4) {
      float pj[4];
      const T* vr[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {                      // rows past the last key: weight 0, row clamped
        pj[u] = __shfl(p, (j + u) & 63, 64);
        const int row = k0 + j + u < nkeys ? k0 + j + u : nkeys - 1;
        vr[u] = v + base + (int64_t)row * sh.ss;
      }
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const int i = lane + c * 64;
        if (i < d) {
          float x[4];
#pragma unroll
          for (int u = 0; u < 4; u++) x[u] = to_f32(vr[u][i]);
#pragma unroll
          for (int u = 0; u < 4; u++) acc[c] += pj[u] * x[u];
        }
      }
    }
    m = m_new;
  }
  T* orow = o + base + (int64_t)qi * sh.ss;
#pragma unroll
  for (int c = 0; c < 4; c++) {
    const int i = lane + c * 64;
    if (i < d) orow[i] = from_f32<T>(acc[c] / l);
  }
  if (lane == 0) lse[(int64_t)bh * sh.seq + qi] = m + logf(l);
}

// delta[b,h,s] = sum_i dO[b,h,s,i] * O[b,h,s,i]; one wavefront per row.
template <typename T>
__global__ __launch_bounds__(256) void attn_delta_kernel(const T* __restrict__ o, const T* __restrict__ d_o,
                                                         float* __restrict__ delta, AttnShape sh, int d) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int qi = blockIdx.x * 4 + wave;
  const int bh = blockIdx.y;
  if (qi >= sh.seq) return;
  const int64_t off = (int64_t)(bh / sh.heads) * sh.sb + (int64_t)(bh % sh.heads) * sh.sh + (int64_t)qi * sh.ss;
  float s = 0.f;
  for (int i = lane; i < d; i += 64) s += to_f32(o[off + i]) * to_f32(d_o[off + i]);
  s = wave_sum(s);
  if (lane == 0) delta[(int64_t)bh * sh.seq + qi] = s;
}

// dQ: one wavefront per query.
template <typename T>
__global__ __launch_bounds__(256) void attn_bwd_dq_generic_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                                  const T* __restrict__ v, const T* __restrict__ d_o,
                                                                  const float* __restrict__ lse,
                                                                  const float* __restrict__ delta, T* __restrict__ dq,
                                                                  AttnShape sh, int d, float scale, int causal, int vec4) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int qi = blockIdx.x * 4 + wave;
  const int bh = blockIdx.y;
  if (qi >= sh.seq) return;
  const int64_t base = (int64_t)(bh / sh.heads) * sh.sb + (int64_t)(bh % sh.heads) * sh.sh;
  const T* qr = q + base + (int64_t)qi * sh.ss;
  const T* dor = d_o + base + (int64_t)qi * sh.ss;
  const float L = lse[(int64_t)bh * sh.seq + qi], dl = delta[(int64_t)bh * sh.seq + qi];
  const int nkeys = causal ? qi + 1 : sh.seq;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < nkeys; k0 += 64) {
    const int key = k0 + lane;
    float ds = 0.f;
    if (key < nkeys) {
      float dot, dp;
      row_dots<T, true>(qr, k + base + (int64_t)key * sh.ss, dor, v + base + (int64_t)key * sh.ss, d, vec4 != 0, &dot, &dp);
      const float p = expf(dot * scale - L);
      ds = p * (dp - dl) * scale;
    }
    const int cnt = nkeys - k0 < 64 ? nkeys - k0 : 64;
    for (int j = 0; j < cnt; j += 4) {
      float dsj[4];
      const T* kr[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {                      // rows past the last key: weight 0, row clamped
        dsj[u] = __shfl(ds, (j + u) & 63, 64);
        const int row = k0 + j + u < nkeys ? k0 + j + u : nkeys - 1;
        kr[u] = k + base + (int64_t)row * sh.ss;
      }
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const int i = lane + c * 64;
        if (i < d) {
          float x[4];
#pragma unroll
          for (int u = 0; u < 4; u++) x[u] = to_f32(kr[u][i]);
#pragma unroll
          for (int u = 0; u < 4; u++) acc[c] += dsj[u] * x[u];
        }
      }
    }
  }
  T* out = dq + base + (int64_t)qi * sh.ss;
#pragma unroll
  for (int c = 0; c < 4; c++) {
    const int i = lane + c * 64;
    if (i < d) out[i] = from_f32<T>(acc[c]);
  }
}

// dK, dV: one wavefront per key.
template <typename T>
__global__ __launch_bounds__(256) void attn_bwd_dkv_generic_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                                   const T* __restrict__ v, const T* __restrict__ d_o,
                                                                   const float* __restrict__ lse,
                                                                   const float* __restrict__ delta, T* __restrict__ dk,
                                                                   T* __restrict__ dv, AttnShape sh, int d, float scale,
                                                                   int causal, int vec4) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ki = blockIdx.x * 4 + wave;
  const int bh = blockIdx.y;
  if (ki >= sh.seq) return;
  const int64_t base = (int64_t)(bh / sh.heads) * sh.sb + (int64_t)(bh % sh.heads) * sh.sh;
  const T* kr = k + base + (int64_t)ki * sh.ss;
  const T* vr = v + base + (int64_t)ki * sh.ss;
  const int qstart = causal ? ki : 0;
  float acck[4] = {0.f, 0.f, 0.f, 0.f}, accv[4] = {0.f, 0.f, 0.f, 0.f};
  for (int q0 = qstart; q0 < sh.seq; q0 += 64) {
    const int qi = q0 + lane;
    float p = 0.f, ds = 0.f;
    if (qi < sh.seq) {
      float dot, dp;
      row_dots<T, true>(q + base + (int64_t)qi * sh.ss, kr, d_o + base + (int64_t)qi * sh.ss, vr, d, vec4 != 0, &dot, &dp);
      p = expf(dot * scale - lse[(int64_t)bh * sh.seq + qi]);
      ds = p * (dp - delta[(int64_t)bh * sh.seq + qi]) * scale;
    }
    const int cnt = sh.seq - q0 < 64 ? sh.seq - q0 : 64;
    for (int j = 0; j < cnt; j += 2) {
      float pj[2], dsj[2];
      const T* qr[2];
      const T* dor[2];
#pragma unroll
      for (int u = 0; u < 2; u++) {                      // rows past the last query: weight 0, row clamped
        pj[u] = __shfl(p, (j + u) & 63, 64);
        dsj[u] = __shfl(ds, (j + u) & 63, 64);
        const int row = q0 + j + u < sh.seq ? q0 + j + u : sh.seq - 1;
        qr[u] = q + base + (int64_t)row * sh.ss;
        dor[u] = d_o + base + (int64_t)row * sh.ss;
      }
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const int i = lane + c * 64;
        if (i < d) {
          float x[2], y[2];
#pragma unroll
          for (int u = 0; u < 2; u++) x[u] = to_f32(dor[u][i]), y[u] = to_f32(qr[u][i]);
#pragma unroll
          for (int u = 0; u < 2; u++) accv[c] += pj[u] * x[u], acck[c] += dsj[u] * y[u];
        }
      }
    }
  }
#pragma unroll
  for (int c = 0; c < 4; c++) {
    const int i = lane + c * 64;
    if (i < d) {
      dk[base + (int64_t)ki * sh.ss + i] = from_f32<T>(acck[c]);
      dv[base + (int64_t)ki * sh.ss + i] = from_f32<T>(accv[c]);
    }
  }
}

// ===========================================================================
// bf16 MFMA path
// ===========================================================================

// LDS tile [rows][D] bf16.  16-byte chunk c of row r lives at chunk
// c ^ swz<D>(r), chosen so that 16 consecutive rows at one logical chunk
// (ds_read_b128 operand fetch) and 4 consecutive rows x 64 bytes (the
// transposing ds_read_b64_tr_b16 fetch) both spread over all banks.
template <int D> __device__ __forceinline__ int swz(int row);
template <> __device__ __forceinline__ int swz<128>(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }
template <> __device__ __forceinline__ int swz<64>(int row) { return (((row >> 1) & 1) << 2) | ((row >> 2) & 3); }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t attn_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

// Stream a [ROWS][D] tile (rows row0.. of one head) into LDS; rows >= seq read
// as zeros.  `rsrc` is based at the head's first element.
template <int D, int ROWS, int NW>
__device__ __forceinline__ void load_rows_tile(__amdgpu_buffer_rsrc_t rsrc, EMI_LDS uint8_t* lds, int wave, int lane,
                                               int row0, int seq, int64_t ss) {
  constexpr int CPR = D / 8;              // chunks per row
  constexpr int RPL = 64 / CPR;           // rows per wave-load
  constexpr int NLOAD = ROWS / RPL / NW;
  static_assert(NLOAD >= 1, "tile smaller than one pass of the block");
#pragma unroll
  for (int it = 0; it < NLOAD; it++) {
    const int r = (it * NW + wave) * RPL + lane / CPR;
    const int pc = lane % CPR;
    const int lc = pc ^ swz<D>(r);
    uint32_t voff = (uint32_t)((int64_t)(row0 + r) * ss + lc * 8) * 2u;
    if (row0 + r >= seq) voff = kOobA;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, lds + (it * NW + wave) * 1024, 16, voff, 0, 0, 0);
  }
}

// One of those loads on its own, for a kernel that spreads them between its MFMAs: lane_off is the per-lane part of
// the byte offset of load 0 at tile row 0, computed once per kernel; load `it` lies it * NW * (64 / (D / 8)) rows
// further (a multiple of 16 rows: the swizzle does not change), which together with the tile's first row is a
// wave-uniform term.  No bounds test: a row past the end of the sequence lies past the end of the buffer descriptor
// (which ends with the last row of the head) and reads as zero.
template <int D, int NW> __device__ __forceinline__ uint32_t tile_lane_offset(int wave, int lane, int64_t ss) {
  constexpr int CPR = D / 8, RPL = 64 / CPR;
  static_assert((NW * RPL) % 16 == 0, "swizzle period");
  const int r = wave * RPL + lane / CPR;
  const int lc = (lane % CPR) ^ swz<D>(r);
  return (uint32_t)((int64_t)r * ss + lc * 8) * 2u;
}
template <int D, int NW>
__device__ __forceinline__ uint32_t tile_piece_offset(uint32_t lane_off, int it, int row0, uint32_t row_bytes) {
  return lane_off + (uint32_t)(row0 + it * NW * (64 / (D / 8))) * row_bytes;
}
// load `it` of wavefront `wave` into its 1 KB piece of the LDS tile
template <int D, int NW>
__device__ __forceinline__ void load_tile_piece(__amdgpu_buffer_rsrc_t rsrc, EMI_LDS uint8_t* tile, int wave, uint32_t lane_off,
                                                int it, int row0, uint32_t row_bytes) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, tile + (it * NW + wave) * 1024, 16,
                                           tile_piece_offset<D, NW>(lane_off, it, row0, row_bytes), 0, 0, 0);
}

// Operand fragment "32 tile rows x 16 of D": lane l holds row row_base + (l & 31),
// D-index 16*step + 8*(l >> 5) + 0..7.
template <int D>
__device__ __forceinline__ bf16x8_t row_frag(const EMI_LDS uint8_t* tile, int row_base, int step, int lane) {
  const int row = row_base + (lane & 31);
  const int chunk = (step * 2 + (lane >> 5)) ^ swz<D>(row);
  return *reinterpret_cast<const EMI_LDS bf16x8_t*>(tile + row * (D * 2) + chunk * 16);
}

// Operand fragment "32 of D x 16 tile rows" (the tile transposed): lane l holds
// D-index col_base + (l & 31) and tile rows row_base + 4*(l>>5) + {0..3, 8..11},
// which is exactly the row set a lane owns in registers 8s..8s+7 of a 32x32
// accumulator (row_base = 16*s within the 32-row sub-tile).
template <int D>
__device__ __forceinline__ bf16x8_t col_frag(const EMI_LDS uint8_t* tile, int row_base, int col_base, int lane) {
  const int i = lane & 15;
  const int r0 = row_base + (lane >> 5) * 4 + (i >> 2);
  const int r1 = r0 + 8;
  const int col = col_base + ((lane >> 4) & 1) * 16 + (i & 3) * 4;
  const int chunk = col >> 3, within = (col & 7) * 2;
  const EMI_LDS uint8_t* p0 = tile + r0 * (D * 2) + ((chunk ^ swz<D>(r0)) * 16) + within;
  const EMI_LDS uint8_t* p1 = tile + r1 * (D * 2) + ((chunk ^ swz<D>(r1)) * 16) + within;
  bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((EMI_LDS bf16x4_t*)p0);
  bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((EMI_LDS bf16x4_t*)p1);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Eight consecutive accumulator registers -> one bf16x8 MFMA operand.
__device__ __forceinline__ bf16x8_t acc_to_frag(const f32x16_t& a, int s) {
  f32x8_t t;
#pragma unroll
  for (int e = 0; e < 8; e++) t[e] = a[8 * s + e];
  return __builtin_convertvector(t, bf16x8_t);
}

// Register-resident operand: 32 rows (one per lane & 31) x D, straight from HBM.
template <int D>
__device__ __forceinline__ void load_reg_rows(const uint16_t* head_base, int row, int seq, int64_t ss, int lane,
                                              bf16x8_t (&f)[D / 16]) {
#pragma unroll
  for (int t = 0; t < D / 16; t++) {
    if (row < seq) {
      f[t] = *reinterpret_cast<const bf16x8_t*>(head_base + (int64_t)row * ss + t * 16 + 8 * (lane >> 5));
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) f[t][e] = (__bf16)0.0f;
    }
  }
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Row index inside a 32x32 accumulator tile held by register r of this lane.
__device__ __forceinline__ int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

// ---------------------------------------------------------------------------
// Forward: block = 4 waves x 32 queries, KV tiles of 64 keys.
// ---------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256, 2) void attn_fwd_bf16_kernel(const uint16_t* __restrict__ q,
                                                            const uint16_t* __restrict__ k,
                                                            const uint16_t* __restrict__ v, uint16_t* __restrict__ o,
                                                            float* __restrict__ lse, AttnShape sh, uint32_t head_bytes,
                                                            float scale_log2e, int causal) {
  constexpr int BQ = 128, BKV = 64, NW = 4;
  constexpr int TILE = BKV * D * 2, STAGE = 2 * TILE;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[];
  EMI_LDS uint8_t* smem = (EMI_LDS uint8_t*)smem_raw;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int blk, bh;
  attn_block_coords(&blk, &bh);
  const int qblk = gridDim.x - 1 - blk;              // longest rows first
  const int64_t base = (int64_t)(bh / sh.heads) * sh.sb + (int64_t)(bh % sh.heads) * sh.sh;
  const int seq = sh.seq;
  const int q0 = qblk * BQ + wave * 32;
  const int qrow = q0 + (lane & 31);

  bf16x8_t qf[D / 16];
  load_reg_rows<D>(q + base, qrow, seq, sh.ss, lane, qf);

  const __amdgpu_buffer_rsrc_t rK = attn_rsrc(k + base, head_bytes);
  const __amdgpu_buffer_rsrc_t rV = attn_rsrc(v + base, head_bytes);
  const int kv_end = causal ? (qblk * BQ + BQ < seq ? qblk * BQ + BQ : seq) : seq;
  const int nkv = (kv_end + BKV - 1) / BKV;

  f32x16_t acc_o[D / 32];
#pragma unroll
  for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc_o[dt][r] = 0.f;
  float m = kNegBig, l = 0.f;

  load_rows_tile<D, BKV, NW>(rK, smem, wave, lane, 0, seq, sh.ss);
  load_rows_tile<D, BKV, NW>(rV, smem + TILE, wave, lane, 0, seq, sh.ss);
  __builtin_amdgcn_s_waitcnt(0x0f70);
  __syncthreads();

  for (int j = 0; j < nkv; j++) {
    if (j + 1 < nkv) {
      EMI_LDS uint8_t* nxt = smem + ((j + 1) & 1) * STAGE;
      load_rows_tile<D, BKV, NW>(rK, nxt, wave, lane, (j + 1) * BKV, seq, sh.ss);
      load_rows_tile<D, BKV, NW>(rV, nxt + TILE, wave, lane, (j + 1) * BKV, seq, sh.ss);
    }
    const EMI_LDS uint8_t* sK = smem + (j & 1) * STAGE;
    const EMI_LDS uint8_t* sV = sK + TILE;
    const int key0 = j * BKV;
    if (!(causal && key0 > q0 + 31)) {     // wave-uniform: this tile is not entirely in the future
      f32x16_t s[2];
#pragma unroll
      for (int T = 0; T < 2; T++) {
#pragma unroll
        for (int r = 0; r < 16; r++) s[T][r] = 0.f;
#pragma unroll
        for (int t = 0; t < D / 16; t++)
          s[T] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(row_frag<D>(sK, T * 32, t, lane), qf[t], s[T], 0, 0, 0);
      }
      const bool need_mask = (causal && key0 + BKV - 1 > q0) || key0 + BKV > seq;
      float mt = kNegBig;
#pragma unroll
      for (int T = 0; T < 2; T++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          if (need_mask) {
            const int key = key0 + T * 32 + acc_row(r, lane);
            if ((causal && key > qrow) || key >= seq) s[T][r] = kNegBig;
          }
          mt = fmaxf(mt, s[T][r]);
        }
      mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
      const float m_new = fmaxf(m, mt * scale_log2e);      // running max in the scaled log2 domain
      const float alpha = fast_exp2(m - m_new);
      float rs = 0.f;
#pragma unroll
      for (int T = 0; T < 2; T++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float p = fast_exp2(fmaf(s[T][r], scale_log2e, -m_new));
          s[T][r] = p;
          rs += p;
        }
      l = l * alpha + rs;
      m = m_new;
#pragma unroll
      for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc_o[dt][r] *= alpha;
#pragma unroll
      for (int T = 0; T < 2; T++)
#pragma unroll
        for (int sI = 0; sI < 2; sI++) {
          const bf16x8_t pf = acc_to_frag(s[T], sI);
#pragma unroll
          for (int dt = 0; dt < D / 32; dt++)
            acc_o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(col_frag<D>(sV, T * 32 + sI * 16, dt * 32, lane), pf,
                                                                acc_o[dt], 0, 0, 0);
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
  }

  // Epilogue.  A lane owns one query and, per register quad, four consecutive d: written
  // straight to HBM that is 8 bytes per lane to 32 different rows.  Instead each wavefront
  // stages its 32 x D tile through its slice of the (now idle) LDS and writes rows with
  // 16-byte, row-contiguous stores.  Chunk c of row r sits at chunk c ^ (r % CH), the two
  // 8-byte halves swapped when (r / CH) is odd: conflict free for both access shapes.
  // (the loop ended with all loads landed and a barrier: the LDS is idle)
  l += __shfl_xor(l, 32, 64);
  {
    constexpr int CH = D / 8, RB = D * 2;
    EMI_LDS uint8_t* wl = smem + wave * (32 * RB);
    const float inv = 1.0f / l;
    const int r = lane & 31, g = lane >> 5;
#pragma unroll
    for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
      for (int jj = 0; jj < 4; jj++) {
        u32x2_t w;
        w[0] = pack_bf16x2(acc_o[dt][4 * jj] * inv, acc_o[dt][4 * jj + 1] * inv);
        w[1] = pack_bf16x2(acc_o[dt][4 * jj + 2] * inv, acc_o[dt][4 * jj + 3] * inv);
        const int c = dt * 4 + jj;
        *reinterpret_cast<EMI_LDS u32x2_t*>(wl + r * RB + ((c ^ (r & (CH - 1))) << 4) + ((g ^ ((r / CH) & 1)) << 3)) = w;
      }
    if (qrow < seq && lane < 32) lse[(int64_t)bh * seq + qrow] = (m + __builtin_amdgcn_logf(l)) * kLn2;
#pragma unroll
    for (int it = 0; it < 32 * CH / 64; it++) {
      const int row = it * (64 / CH) + lane / CH, c = lane % CH;
      u32x4_t v4 = *reinterpret_cast<const EMI_LDS u32x4_t*>(wl + row * RB + ((c ^ (row & (CH - 1))) << 4));
      if ((row / CH) & 1) v4 = __builtin_shufflevector(v4, v4, 2, 3, 0, 1);
      if (q0 + row < seq) *reinterpret_cast<u32x4_t*>(o + base + (int64_t)(q0 + row) * sh.ss + c * 8) = v4;
    }
  }
}

// Transposing LDS read as inline assembly (the result is valid after an attn_tr_wait that covers it), and the wait:
// at most N LDS operations issued after the two reads may still be outstanding.
template <int OFF> __device__ __forceinline__ u32x2_t attn_tr_read(uint32_t addr) {
  static_assert(OFF >= 0 && OFF < 65536, "ds offset field");
  u32x2_t r;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
  return r;
}
template <int N> __device__ __forceinline__ void attn_tr_wait(u32x2_t& lo, u32x2_t& hi) {
  static_assert(N >= 0 && N < 16, "lgkmcnt field");
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(lo), "+v"(hi) : "n"(N));
}

template <typename F, int... Is>
__device__ __forceinline__ void attn_static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F> __device__ __forceinline__ void attn_static_for(F&& f) {
  attn_static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// ---------------------------------------------------------------------------
// Forward, ping-pong form: block = 8 waves x 32 queries in two groups of four, one
// wavefront of each group per SIMD.  A key/value tile step is two phases separated by
// s_barrier: a VALU phase (softmax of the scores in registers) and an MFMA phase (scores
// of the next tile, then P.V of this one).  The groups run one phase apart, so on every
// SIMD the softmax of one wavefront overlaps the matrix work of the other.
//   bundle b(j) = {K tile j+1, V tile j}: what MFMA phase j reads; three bundles in LDS.
//   MFMA phase j issues the loads of b(j+2) between its P.V MFMAs (the slot was last read
//   by the MFMA phases j-1 of both groups, which ended before this phase began) and ends
//   by waiting for its own part of b(j+1) before the barrier.
// The running maximum is only raised when some row's tile maximum exceeds it by more
// than 8 (in log2 units), so the rescaling of O runs on a few early tiles only; P then
// stays below 2^8 and the final O/l and log-sum-exp are exact for whatever m was used.
// ---------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(512) void attn_fwd_pp_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k,
                                                          const uint16_t* __restrict__ v, uint16_t* __restrict__ o,
                                                          float* __restrict__ lse, AttnShape sh, uint32_t head_bytes,
                                                          float scale_log2e, int causal) {
  constexpr int BQ = 256, BKV = 64, NW = 8;
  constexpr int TILE = BKV * D * 2, BUNDLE = 2 * TILE;
  constexpr int LPB = 2 * (BKV * D * 2 / 1024 / NW);       // loads per wave per bundle
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[];
  EMI_LDS uint8_t* smem = (EMI_LDS uint8_t*)smem_raw;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int blk, bh;
  attn_block_coords(&blk, &bh);
  const int qblk = gridDim.x - 1 - blk;              // longest rows first
  const int64_t base = (int64_t)(bh / sh.heads) * sh.sb + (int64_t)(bh % sh.heads) * sh.sh;
  const int seq = sh.seq;
  const int q0 = qblk * BQ + wave * 32;
  const int qrow = q0 + (lane & 31);

  bf16x8_t qf[D / 16];
  load_reg_rows<D>(q + base, qrow, seq, sh.ss, lane, qf);

  const __amdgpu_buffer_rsrc_t rK = attn_rsrc(k + base, head_bytes);
  const __amdgpu_buffer_rsrc_t rV = attn_rsrc(v + base, head_bytes);
  const int kv_end = causal ? (qblk * BQ + BQ < seq ? qblk * BQ + BQ : seq) : seq;
  const int nt = (kv_end + BKV - 1) / BKV;
  const int krow_l = lane & 31;                      // K row this lane feeds into the score MFMAs

  f32x16_t acc_o[D / 32];
#pragma unroll
  for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc_o[dt][r] = 0.f;
  float m = kNegBig, l = 0.f;
  f32x16_t s[2];
  bf16x8_t pf[2][2];

  auto phase_end = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  auto issue_bundle = [&](int jb, int slot) __attribute__((always_inline)) {
    EMI_LDS uint8_t* sK = smem + slot * TILE;
    EMI_LDS uint8_t* sV = smem + 3 * TILE + slot * TILE;
    load_rows_tile<D, BKV, NW>(rK, sK, wave, lane, (jb + 1) * BKV, seq, sh.ss);
    const int vrow0 = jb < 0 ? 0 : jb * BKV;
    load_rows_tile<D, BKV, NW>(rV, sV, wave, lane, vrow0, seq, sh.ss);
  };
  // MFMA phase: scores of tile j+1 (DO_S) and P.V of tile j (DO_PV) out of bundle SLOT.
  // The operand fragments go through a ring of DEPTH registers sets: the LDS read of
  // operation i + DEPTH is issued right after the MFMA of operation i, so the LDS latency
  // hides behind DEPTH MFMAs.
  // The V operand (V^T fragments of a row-major V tile) comes through transposing LDS reads, two 8-byte reads per
  // fragment with the lane mapping of col_frag.  They are written as inline assembly with their own lgkmcnt waits: the compiler
  // puts a wait for every outstanding direct-to-LDS load in front of a transposing read it knows of, which would
  // make every MFMA phase wait for the bundle issued one step earlier.  vadr[dt][h]: LDS address of this lane's 8
  // bytes for d-block dt, key rows h*8 + ..., key block 0, ring slot 0.
  uint32_t vadr[D / 32][2];
  {
    const int i16 = lane & 15;
#pragma unroll
    for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int r = (lane >> 5) * 4 + (i16 >> 2) + 8 * h;
        const int col = dt * 32 + ((lane >> 4) & 1) * 16 + (i16 & 3) * 4;
        vadr[dt][h] = (uint32_t)(uintptr_t)(smem + 3 * TILE) + (uint32_t)(r * (D * 2) + (((col >> 3) ^ swz<D>(r)) << 4) + (col & 7) * 2);
      }
  }
  // Load n (0 .. LPB-1; K loads first, then V loads) of bundle jb into ring slot slot2.
  const uint32_t lane_off = tile_lane_offset<D, NW>(wave, lane, sh.ss);
  const uint32_t row_bytes = (uint32_t)sh.ss * 2u;
  auto issue_one = [&](const int n, const int slot2, int jb) __attribute__((always_inline)) {
    constexpr int NL = LPB / 2;
    if (n < NL) load_tile_piece<D, NW>(rK, smem + slot2 * TILE, wave, lane_off, n, (jb + 1) * BKV, row_bytes);
    else load_tile_piece<D, NW>(rV, smem + 3 * TILE + slot2 * TILE, wave, lane_off, n - NL, jb * BKV, row_bytes);
  };
  // jb_issue: the bundle whose loads this phase issues (phases that compute both products only)
  auto mfma_phase = [&](auto do_s_c, auto do_pv_c, auto slot_c, int jb_issue) __attribute__((always_inline)) {
    constexpr bool DO_S = decltype(do_s_c)::value, DO_PV = decltype(do_pv_c)::value;
    constexpr int SLOT = decltype(slot_c)::value;
    constexpr int NS = DO_S ? 2 * (D / 16) : 0, NPV = DO_PV ? 4 * (D / 32) : 0, NOP = NS + NPV, DEPTH = 6;
    // K tiles of the three bundles first, then the V tiles: every fragment address is
    // one of a few per-lane bases plus an immediate offset below 64 KiB
    const EMI_LDS uint8_t* sK = smem + SLOT * TILE;
    bf16x8_t ring[DEPTH];
    u32x2_t tlo[DEPTH], thi[DEPTH];            // halves of V fragments in flight (asm path)
    auto fetch = [&](auto ic) __attribute__((always_inline)) {
      constexpr int i = decltype(ic)::value;
      if constexpr (i < NS) {
        constexpr int t = i >> 1, T = i & 1;
        const int row = T * 32 + krow_l;
        const int chunk = (t * 2 + (lane >> 5)) ^ swz<D>(row);
        ring[i % DEPTH] = *reinterpret_cast<const EMI_LDS bf16x8_t*>(sK + row * (D * 2) + chunk * 16);
      } else {
        constexpr int x = i - NS, dt = x % (D / 32), sI = (x / (D / 32)) & 1, T = x / (2 * (D / 32));
        constexpr int OFF = SLOT * TILE + (T * 32 + sI * 16) * (D * 2);
        tlo[i % DEPTH] = attn_tr_read<OFF>(vadr[dt][0]);
        thi[i % DEPTH] = attn_tr_read<OFF>(vadr[dt][1]);
      }
    };
    if constexpr (DO_S) {
#pragma unroll
      for (int T = 0; T < 2; T++)
#pragma unroll
        for (int r = 0; r < 16; r++) s[T][r] = 0.f;
    }
    attn_static_for<(DEPTH < NOP ? DEPTH : NOP)>([&](auto ic) __attribute__((always_inline)) { fetch(ic); });
    __builtin_amdgcn_sched_barrier(0);
    attn_static_for<NOP>([&](auto ic) __attribute__((always_inline)) {
      constexpr int i = decltype(ic)::value;
      if constexpr (i < NS) {
        s[i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[i % DEPTH], qf[i >> 1], s[i & 1], 0, 0, 0);
      } else {
        constexpr int x = i - NS, dt = x % (D / 32), sI = (x / (D / 32)) & 1, T = x / (2 * (D / 32));
        // the reads of the fragments behind this one (all of them V fragments) may still be in flight
        constexpr int AFTER = 2 * ((NOP - 1 - i) < (DEPTH - 1) ? (NOP - 1 - i) : (DEPTH - 1));
        attn_tr_wait<AFTER>(tlo[i % DEPTH], thi[i % DEPTH]);
        const u32x4_t w = {tlo[i % DEPTH][0], tlo[i % DEPTH][1], thi[i % DEPTH][0], thi[i % DEPTH][1]};
        ring[i % DEPTH] = __builtin_bit_cast(bf16x8_t, w);
        acc_o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[i % DEPTH], pf[T][sI], acc_o[dt], 0, 0, 0);
      }
      if constexpr (i + DEPTH < NOP) fetch(std::integral_constant<int, i + DEPTH>{});
      // The loads of the bundle two steps ahead go out one at a time between the P.V MFMAs (no K read, before
      // which the compiler would wait for them, follows).  Issued together at the end of the phase, the 16 loads
      // of a group queue up in the memory pipeline and hold every wavefront for 300-400 cycles with its matrix
      // core idle (4096 keys x 128: 629 -> 590 us).
      if constexpr (DO_S && DO_PV) {
        constexpr int GAP = NPV / LPB;
        if constexpr (i >= NS && (i - NS) % GAP == 0 && (i - NS) / GAP < LPB) issue_one((i - NS) / GAP, (SLOT + 2) % 3, jb_issue);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  auto softmax = [&](int j) __attribute__((always_inline)) {
    const int key0 = j * BKV;
    if ((causal && key0 + BKV - 1 > q0) || key0 + BKV > seq) {
      asm volatile("" ::: "memory");     // keeps this a branch: most tiles need no mask
#pragma unroll
      for (int T = 0; T < 2; T++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int mrow = acc_row(r, lane);
          const int key = key0 + T * 32 + mrow;
          if ((causal && key > qrow) || key >= seq) s[T][r] = kNegBig;
        }
    }
    float mt = s[0][0];
#pragma unroll
    for (int T = 0; T < 2; T++)
#pragma unroll
      for (int r = 0; r < 16; r++) mt = fmaxf(mt, s[T][r]);
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64)) * scale_log2e;
    if (__builtin_amdgcn_ballot_w64(mt > m + 8.0f) != 0) {      // wave-uniform, rare after the first tiles
      const float m_new = fmaxf(m, mt);
      const float alpha = fast_exp2(m - m_new);
      l *= alpha;
#pragma unroll
      for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc_o[dt][r] *= alpha;
      m = m_new;
    }
    float rs = 0.f;
#pragma unroll
    for (int T = 0; T < 2; T++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float p = fast_exp2(fmaf(s[T][r], scale_log2e, -m));
        s[T][r] = p;
        rs += p;
      }
      pf[T][0] = acc_to_frag(s[T], 0);
      pf[T][1] = acc_to_frag(s[T], 1);
    }
    l += rs;
  };
  // One tile step; bundle b(j) sits in slot (j + 1) % 3 = SLOT.  Every wavefront meets every barrier and issues its
  // share of every bundle, but a tile that lies wholly in the causal future of the wavefront's 32 queries (the
  // last tiles of the block's diagonal, for the wavefronts with the lower queries) costs it neither softmax nor
  // matrix work: nt_w is the number of tiles that hold a key this wavefront can see.
  const int nt_w = causal ? ((q0 + 31) / BKV + 1 < nt ? (q0 + 31) / BKV + 1 : nt) : nt;
  auto step = [&](auto slot_c, int j) __attribute__((always_inline)) {
    constexpr int SLOT = decltype(slot_c)::value;
    if (j < nt_w) softmax(j);                         // VALU phase
    phase_end();
    __builtin_amdgcn_s_setprio(1);                    // MFMA phase
    if (j < nt_w) mfma_phase(std::true_type{}, std::true_type{}, slot_c, j + 2);    // (its last scores are never used)
    else issue_bundle(j + 2, (SLOT + 2) % 3);
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_s_waitcnt(0x0f70 | (LPB & 15));  // vmcnt(LPB): own part of b(j+1) has landed
    phase_end();
  };

  issue_bundle(-1, 0);
  issue_bundle(0, 1);
  __builtin_amdgcn_s_waitcnt(0x0f70);                 // vmcnt(0)
  issue_bundle(1, 2);
  phase_end();
  if (wave >= 4) phase_end();                         // second group runs one phase behind
  __builtin_amdgcn_s_setprio(1);
  mfma_phase(std::true_type{}, std::false_type{}, std::integral_constant<int, 0>{}, 0);      // MFMA phase -1
  __builtin_amdgcn_s_setprio(0);
  phase_end();
  for (int j = 0; j < nt; j += 3) {
    step(std::integral_constant<int, 1>{}, j);
    if (j + 1 < nt) step(std::integral_constant<int, 2>{}, j + 1);
    if (j + 2 < nt) step(std::integral_constant<int, 0>{}, j + 2);
  }
  if (wave < 4) phase_end();
  __builtin_amdgcn_s_waitcnt(0x0f70);                 // loads past the last tile

  // Epilogue.  A lane owns one query and, per register quad, four consecutive d: written
  // straight to HBM that is 8 bytes per lane to 32 different rows.  Instead each wavefront
  // stages its 32 x D tile through its slice of the (now idle) LDS and writes rows with
  // 16-byte, row-contiguous stores.  Chunk c of row r sits at chunk c ^ (r % CH), the two
  // 8-byte halves swapped when (r / CH) is odd: conflict free for both access shapes.
  phase_end();                                        // every wavefront's loads have landed
  l += __shfl_xor(l, 32, 64);
  {
    constexpr int CH = D / 8, RB = D * 2;
    EMI_LDS uint8_t* wl = smem + wave * (32 * RB);
    const float inv = 1.0f / l;
    const int r = lane & 31, g = lane >> 5;
#pragma unroll
    for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
      for (int jj = 0; jj < 4; jj++) {
        u32x2_t w;
        w[0] = pack_bf16x2(acc_o[dt][4 * jj] * inv, acc_o[dt][4 * jj + 1] * inv);
        w[1] = pack_bf16x2(acc_o[dt][4 * jj + 2] * inv, acc_o[dt][4 * jj + 3] * inv);
        const int c = dt * 4 + jj;
        *reinterpret_cast<EMI_LDS u32x2_t*>(wl + r * RB + ((c ^ (r & (CH - 1))) << 4) + ((g ^ ((r / CH) & 1)) << 3)) = w;
      }
    if (qrow < seq && lane < 32) lse[(int64_t)bh * seq + qrow] = (m + __builtin_amdgcn_logf(l)) * kLn2;
#pragma unroll
    for (int it = 0; it < 32 * CH / 64; it++) {
      const int row = it * (64 / CH) + lane / CH, c = lane % CH;
      u32x4_t v4 = *reinterpret_cast<const EMI_LDS u32x4_t*>(wl + row * RB + ((c ^ (row & (CH - 1))) << 4));
      if ((row / CH) & 1) v4 = __builtin_shufflevector(v4, v4, 2, 3, 0, 1);
      if (q0 + row < seq) *reinterpret_cast<u32x4_t*>(o + base + (int64_t)(q0 + row) * sh.ss + c * 8) = v4;
    }
  }
}

// The adjoint of RoPE (test/llama.py:161-168) on four consecutive elements of a head's row (two rotation pairs): the
// cotangent of the rotated vector is turned back by the angle.  t points at the (cos, sin) entries of the two pairs.
__device__ __forceinline__ void unrope_quad(const float* t, float& x0, float& x1, float& x2, float& x3) {
  const float4 cs = *reinterpret_cast<const float4*>(t);
  const float y0 = cs.x * x0 + cs.y * x1, y1 = cs.x * x1 - cs.y * x0;
  const float y2 = cs.z * x2 + cs.w * x3, y3 = cs.z * x3 - cs.w * x2;
  x0 = y0, x1 = y1, x2 = y2, x3 = y3;
}

// ---------------------------------------------------------------------------
// dQ: block = 4 waves x 32 queries; K and V tiles of 64 keys through LDS.
//   S^T = K Q^T, dP^T = V dO^T, dS^T = P^T (dP^T - delta), dQ^T = K^T dS^T
// With `o` given the kernel also does the adjoint's pre-pass for its 128 queries: delta = rowsum(dO . O) from the dO
// fragments it holds anyway and the matching fragments of O (a lane and its partner 32 lanes on hold alternate groups
// of eight elements of a row), written as delta * delta_sign to delta_out and lse * log2(e) to lse2_out for the dK/dV kernel, which then has
// to run after this one.  Without `o`, delta comes in through `delta`.
// ---------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256, 2) void attn_bwd_dq_bf16_kernel(const uint16_t* __restrict__ q,
                                                               const uint16_t* __restrict__ k,
                                                               const uint16_t* __restrict__ v,
                                                               const uint16_t* __restrict__ d_o,
                                                               const float* __restrict__ lse,
                                                               const float* __restrict__ delta,
                                                               uint16_t* __restrict__ dq, AttnShape sh,
                                                               uint32_t head_bytes, float scale, int causal,
                                                               float delta_sign, const float* __restrict__ unrope,
                                                               const uint16_t* __restrict__ o, float* __restrict__ delta_out,
                                                               float* __restrict__ lse2_out) {
  constexpr int BQ = 128, BKV = 64, NW = 4;
  constexpr int TILE = BKV * D * 2, STAGE = 2 * TILE;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[];
  EMI_LDS uint8_t* smem = (EMI_LDS uint8_t*)smem_raw;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int blk, bh;
  attn_block_coords(&blk, &bh);
  const int qblk = gridDim.x - 1 - blk;
  const int64_t base = (int64_t)(bh / sh.heads) * sh.sb + (int64_t)(bh % sh.heads) * sh.sh;
  const int seq = sh.seq;
  const int q0 = qblk * BQ + wave * 32;
  const int qrow = q0 + (lane & 31);
  const float scale_log2e = scale * kLog2e;

  bf16x8_t qf[D / 16], dof[D / 16];
  load_reg_rows<D>(q + base, qrow, seq, sh.ss, lane, qf);
  load_reg_rows<D>(d_o + base, qrow, seq, sh.ss, lane, dof);
  const float L2 = qrow < seq ? lse[(int64_t)bh * seq + qrow] * kLog2e : 0.f;
  float dl;
  if (o != nullptr) {
    bf16x8_t of[D / 16];
    load_reg_rows<D>(o + base, qrow, seq, sh.ss, lane, of);
    // sums of eight products, then pairs of them 8, 4, 2 and 1 apart (the last pair is the partner lane's)
    float cs[D / 16];
#pragma unroll
    for (int t = 0; t < D / 16; t++) {
      const u32x4_t a = __builtin_bit_cast(u32x4_t, of[t]), b = __builtin_bit_cast(u32x4_t, dof[t]);
      float c = 0.f;
#pragma unroll
      for (int w = 0; w < 4; w++) {
        c += __uint_as_float(a[w] << 16) * __uint_as_float(b[w] << 16);
        c += __uint_as_float(a[w] & 0xffff0000u) * __uint_as_float(b[w] & 0xffff0000u);
      }
      cs[t] = c;
    }
#pragma unroll
    for (int m = D / 32; m >= 1; m >>= 1)
#pragma unroll
      for (int t = 0; t < m; t++) cs[t] += cs[t + m];
    dl = cs[0] + __shfl_xor(cs[0], 32, 64);
    if (qrow < seq && lane < 32) {
      delta_out[(int64_t)bh * seq + qrow] = dl * delta_sign;
      lse2_out[(int64_t)bh * seq + qrow] = L2;
    }
  } else {
    dl = qrow < seq ? delta[(int64_t)bh * seq + qrow] * delta_sign : 0.f;
  }

  const __amdgpu_buffer_rsrc_t rK = attn_rsrc(k + base, head_bytes);
  const __amdgpu_buffer_rsrc_t rV = attn_rsrc(v + base, head_bytes);
  const int kv_end = causal ? (qblk * BQ + BQ < seq ? qblk * BQ + BQ : seq) : seq;
  const int nkv = (kv_end + BKV - 1) / BKV;

  f32x16_t acc[D / 32];
#pragma unroll
  for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[dt][r] = 0.f;

  load_rows_tile<D, BKV, NW>(rK, smem, wave, lane, 0, seq, sh.ss);
  load_rows_tile<D, BKV, NW>(rV, smem + TILE, wave, lane, 0, seq, sh.ss);
  __builtin_amdgcn_s_waitcnt(0x0f70);
  __syncthreads();

  for (int j = 0; j < nkv; j++) {
    if (j + 1 < nkv) {
      EMI_LDS uint8_t* nxt = smem + ((j + 1) & 1) * STAGE;
      load_rows_tile<D, BKV, NW>(rK, nxt, wave, lane, (j + 1) * BKV, seq, sh.ss);
      load_rows_tile<D, BKV, NW>(rV, nxt + TILE, wave, lane, (j + 1) * BKV, seq, sh.ss);
    }
    const EMI_LDS uint8_t* sK = smem + (j & 1) * STAGE;
    const EMI_LDS uint8_t* sV = sK + TILE;
    const int key0 = j * BKV;
    if (!(causal && key0 > q0 + 31)) {
      const bool need_mask = (causal && key0 + BKV - 1 > q0) || key0 + BKV > seq;
#pragma unroll 1
      for (int T = 0; T < 2; T++) {
        f32x16_t s, dp;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.f, dp[r] = 0.f;
#pragma unroll
        for (int t = 0; t < D / 16; t++) {
          s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(row_frag<D>(sK, T * 32, t, lane), qf[t], s, 0, 0, 0);
          dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(row_frag<D>(sV, T * 32, t, lane), dof[t], dp, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float p = fast_exp2(s[r] * scale_log2e - L2);
          if (need_mask) {
            const int key = key0 + T * 32 + acc_row(r, lane);
            if ((causal && key > qrow) || key >= seq) p = 0.f;
          }
          s[r] = p * (dp[r] - dl);
        }
#pragma unroll
        for (int sI = 0; sI < 2; sI++) {
          const bf16x8_t dsf = acc_to_frag(s, sI);
#pragma unroll
          for (int dt = 0; dt < D / 32; dt++)
            acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(col_frag<D>(sK, T * 32 + sI * 16, dt * 32, lane), dsf,
                                                              acc[dt], 0, 0, 0);
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
  }
  if (qrow < seq) {
    uint16_t* out = dq + base + (int64_t)qrow * sh.ss;
    const float* trow = unrope ? unrope + (int64_t)qrow * D : nullptr;     // D/2 (cos, sin) pairs per position
#pragma unroll
    for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
      for (int jj = 0; jj < 4; jj++) {
        const int dcol = dt * 32 + 8 * jj + 4 * (lane >> 5);
        float x0 = acc[dt][4 * jj] * scale, x1 = acc[dt][4 * jj + 1] * scale, x2 = acc[dt][4 * jj + 2] * scale,
              x3 = acc[dt][4 * jj + 3] * scale;
        if (trow != nullptr) unrope_quad(trow + dcol, x0, x1, x2, x3);
        uint2 w;
        w.x = pack_bf16x2(x0, x1);
        w.y = pack_bf16x2(x2, x3);
        *reinterpret_cast<uint2*>(out + dcol) = w;
      }
  }
}

// ---------------------------------------------------------------------------
// dK, dV, software-pipelined form: block = 4 wavefronts x 32 keys, one wavefront per SIMD
// (K, V fragments and both accumulators stay in registers).  Work proceeds in halves of a
// 64-query tile (32 queries, index H):
//   A(H): S, dP   = rows of Q, dO against K, V                (16 MFMAs)
//   B(H): P = exp2(S*c - lse2), dS = P*(dP - delta)            (VALU)
//   C(H): dV^T += dO^T P, dK^T += Q^T dS  (columns of dO, Q)   (16 MFMAs)
// Iteration H runs A(H+1) interleaved with B(H), so the softmax arithmetic of one half
// issues in the shadow of the MFMAs of the next, then C(H).  Tiles sit in a ring of
// three LDS slots; once per tile the wavefronts meet at a barrier, after which the loads
// of tile t+3 may overwrite tile t: they go out one by one between the MFMAs of the first
// half of tile t+1.  The column fragments are fetched with
// ds_read_b64_tr_b16 through inline asm: the compiler orders every LDS read it knows of
// behind all outstanding direct-to-LDS loads, which would serialise loading and compute.
// ---------------------------------------------------------------------------
__device__ __forceinline__ u32x2_t lds_read_tr_asm(uint32_t addr) {
  u32x2_t r;
  asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(r) : "v"(addr));
  return r;
}
// s_waitcnt lgkmcnt(N) that the MFMA consuming `a`, `b` cannot be moved above.
template <int N> __device__ __forceinline__ void lgkm_wait_for(u32x2_t& a, u32x2_t& b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}

template <int D>
__global__ __launch_bounds__(256) void attn_bwd_dkv_sp_kernel(const uint16_t* __restrict__ q,
                                                              const uint16_t* __restrict__ k,
                                                              const uint16_t* __restrict__ v,
                                                              const uint16_t* __restrict__ d_o,
                                                              const float* __restrict__ lse2,
                                                              const float* __restrict__ delta, uint16_t* __restrict__ dk,
                                                              uint16_t* __restrict__ dv, AttnShape sh,
                                                              uint32_t head_bytes, float scale, int causal,
                                                              const float* __restrict__ unrope) {
  constexpr int BKEY = 128, BQT = 64, NW = 4, NSLOT = 3;
  constexpr int TILE = BQT * D * 2;
  constexpr int STATS = 2 * NSLOT * TILE;                 // lse2 and delta of each slot: 2 x 256 bytes
  constexpr int LPB = 2 * (TILE / 1024 / NW) + 1;         // loads per wavefront per tile
  static_assert(LPB < 16, "vmcnt immediate");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[];
  EMI_LDS uint8_t* smem = (EMI_LDS uint8_t*)smem_raw;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int kblk, bh;                                           // early key blocks see the most queries: first
  attn_block_coords(&kblk, &bh);
  const int64_t base = (int64_t)(bh / sh.heads) * sh.sb + (int64_t)(bh % sh.heads) * sh.sh;
  const int seq = sh.seq;
  const int k0 = kblk * BKEY + wave * 32;
  const int krow = k0 + (lane & 31);
  const float scale_log2e = scale * kLog2e;

  bf16x8_t kf[D / 16], vf[D / 16];
  load_reg_rows<D>(k + base, krow, seq, sh.ss, lane, kf);
  load_reg_rows<D>(v + base, krow, seq, sh.ss, lane, vf);

  const __amdgpu_buffer_rsrc_t rQ = attn_rsrc(q + base, head_bytes);
  const __amdgpu_buffer_rsrc_t rDO = attn_rsrc(d_o + base, head_bytes);
  const __amdgpu_buffer_rsrc_t rL = attn_rsrc(lse2 + (int64_t)bh * seq, (uint32_t)seq * 4u);
  const __amdgpu_buffer_rsrc_t rDl = attn_rsrc(delta + (int64_t)bh * seq, (uint32_t)seq * 4u);
  const int qt0 = causal ? (kblk * BKEY) / BQT : 0;       // first query tile that can see this key block
  const int nt = (seq + BQT - 1) / BQT - qt0;             // >= 1: the block holds at least one key < seq

  f32x16_t acc_k[D / 32], acc_v[D / 32];
#pragma unroll
  for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc_k[dt][r] = 0.f, acc_v[dt][r] = 0.f;
  bf16x8_t pf[2], dsf[2];

  // tile ti (query tile qt0 + ti) -> slot; rows >= seq read as zeros
  auto issue_stats = [&](int row0, int slot) __attribute__((always_inline)) {
    // one 256-byte load of lse2 (even wavefronts) or delta (odd ones); the copies are identical
    const uint32_t voff = row0 + lane < seq ? (uint32_t)(row0 + lane) * 4u : kOobA;
    __builtin_amdgcn_raw_ptr_buffer_load_lds((wave & 1) ? rDl : rL, smem + STATS + slot * 512 + (wave & 1) * 256, 4, voff, 0, 0,
                                             0);
  };
  auto issue_tile = [&](int ti, int slot) __attribute__((always_inline)) {
    const int row0 = (qt0 + ti) * BQT;
    load_rows_tile<D, BQT, NW>(rQ, smem + slot * TILE, wave, lane, row0, seq, sh.ss);
    load_rows_tile<D, BQT, NW>(rDO, smem + NSLOT * TILE + slot * TILE, wave, lane, row0, seq, sh.ss);
    issue_stats(row0, slot);
  };
  // The same loads one at a time (n = 0 .. LPB-1: Q rows, dO rows, statistics), for the steady state, where they
  // go out between MFMAs: issued together after the barrier, the 36 loads of a block queue up in the memory
  // pipeline and every wavefront, alone on its SIMD, waits for its last one with the matrix core idle.
  const uint32_t lane_off = tile_lane_offset<D, NW>(wave, lane, sh.ss);
  const uint32_t row_bytes = (uint32_t)sh.ss * 2u;
  auto issue_part = [&](const int n, int ti, int slot) __attribute__((always_inline)) {
    constexpr int NLQ = (LPB - 1) / 2;
    const int row0 = (qt0 + ti) * BQT;
    if (n < NLQ) load_tile_piece<D, NW>(rQ, smem + slot * TILE, wave, lane_off, n, row0, row_bytes);
    else if (n < 2 * NLQ) load_tile_piece<D, NW>(rDO, smem + NSLOT * TILE + slot * TILE, wave, lane_off, n - NLQ, row0, row_bytes);
    else issue_stats(row0, slot);
  };
  constexpr int LA = (LPB + 1) / 2, LC = LPB - LA;        // loads issued inside stage A/B and inside stage C
  // A(H+1) with B(H), interleaved by hand: after each of the 16 MFMAs of A (S and dP - delta
  // of half (slot_n, Tn) into sn, dpn; the dP accumulator starts from the -delta of its rows,
  // read from LDS, which saves a subtraction per score) comes the softmax arithmetic of one
  // score of half (ti, slot_p, Tp) held in sp, dpp.  The scheduler is fenced after every
  // step: left alone it issues all MFMAs first and the VALU work after them.
  auto stage_ab = [&](auto masked_c, auto do_b_c, auto issue_c, int slot_n, int Tn, f32x16_t& sn, f32x16_t& dpn, int ti,
                      int slot_p, int Tp, f32x16_t& sp, f32x16_t& dpp, int ti_issue, int slot_issue)
                      __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_c)::value, DO_B = decltype(do_b_c)::value, ISSUE = decltype(issue_c)::value;
    const EMI_LDS uint8_t* sQ = smem + slot_n * TILE;
    const EMI_LDS uint8_t* sDO = smem + NSLOT * TILE + slot_n * TILE;
    const EMI_LDS float* sNd = (const EMI_LDS float*)(smem + STATS + slot_n * 512) + 64 + Tn * 32 + 4 * (lane >> 5);
    const EMI_LDS float* sL = (const EMI_LDS float*)(smem + STATS + slot_p * 512) + Tp * 32 + 4 * (lane >> 5);
    const int qbase = (qt0 + ti) * BQT + Tp * 32;
    constexpr int NOP = 2 * (D / 16), DEPTH = 4;
    static_assert(NOP == 16 || NOP == 8, "one score per MFMA (or two)");
    constexpr int EPM = 16 / NOP;                    // scores handled per MFMA
    auto fetch = [&](int i) __attribute__((always_inline)) -> bf16x8_t {
      return row_frag<D>((i & 1) ? sDO : sQ, Tn * 32, i >> 1, lane);
    };
    f32x4_t L4[4];
#pragma unroll
    for (int rq = 0; rq < 4; rq++) {
      const f32x4_t nd = *reinterpret_cast<const EMI_LDS f32x4_t*>(sNd + 8 * rq);
      if constexpr (DO_B) L4[rq] = *reinterpret_cast<const EMI_LDS f32x4_t*>(sL + 8 * rq);
#pragma unroll
      for (int e = 0; e < 4; e++) dpn[4 * rq + e] = nd[e];
    }
    const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    bf16x8_t ring[DEPTH];
#pragma unroll
    for (int i = 0; i < DEPTH; i++) ring[i] = fetch(i);
    f32x16_t ds;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < NOP; i++) {
      if (i & 1) dpn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[i % DEPTH], vf[i >> 1], dpn, 0, 0, 0);
      else sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[i % DEPTH], kf[i >> 1], i == 0 ? zero16 : sn, 0, 0, 0);
      if (i + DEPTH < NOP) ring[i % DEPTH] = fetch(i + DEPTH);
      if constexpr (ISSUE) {
        constexpr int SP = NOP / LA;
        if (i % SP == 1 && i / SP < LA) issue_part(i / SP, ti_issue, slot_issue);
      }
      if constexpr (DO_B) {
#pragma unroll
        for (int u = 0; u < EPM; u++) {
          const int r = i * EPM + u;
          float p = fast_exp2(fmaf(sp[r], scale_log2e, -L4[r >> 2][r & 3]));
          if (MASKED && causal && krow > qbase + acc_row(r, lane)) p = 0.f;
          sp[r] = p;
          ds[r] = p * dpp[r];
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (DO_B) {
      pf[0] = acc_to_frag(sp, 0);
      pf[1] = acc_to_frag(sp, 1);
      dsf[0] = acc_to_frag(ds, 0);
      dsf[1] = acc_to_frag(ds, 1);
    }
  };
  // C: dV, dK contributions of half (slot, T).  16 column fragments, two asm reads each,
  // ring of 4 fragments: after the reads of fragment i+4 are issued, fragments i..i+4 (10
  // reads) are outstanding and lgkmcnt(8) means fragment i has arrived.
  auto stage_c = [&](auto issue_c, int slot, int T, int ti_issue, int slot_issue) __attribute__((always_inline)) {
    constexpr bool ISSUE = decltype(issue_c)::value;
    const uint32_t aQ = (uint32_t)(uintptr_t)(smem + slot * TILE);
    const uint32_t aDO = (uint32_t)(uintptr_t)(smem + NSLOT * TILE + slot * TILE);
    // per-lane address of the first read of col_frag<D>(tile, row_base, col_base): see col_frag
    const int li = lane & 15;
    const int r0l = (lane >> 5) * 4 + (li >> 2);
    const int coll = ((lane >> 4) & 1) * 16 + (li & 3) * 4;
    auto addr = [&](uint32_t tile, int row, int col) __attribute__((always_inline)) {
      return tile + (uint32_t)(row * (D * 2) + (((col >> 3) ^ swz<D>(row)) * 16) + (col & 7) * 2);
    };
    constexpr int NF = 4 * (D / 32), DEPTH = 4;
    u32x2_t lo[DEPTH], hi[DEPTH];
    auto fetch = [&](int i, int slot_i) __attribute__((always_inline)) {
      const int which = i & 1, dt = (i >> 1) % (D / 32), sI = i / (2 * (D / 32));
      const int row = T * 32 + sI * 16 + r0l, col = dt * 32 + coll;
      lo[slot_i] = lds_read_tr_asm(addr(which ? aQ : aDO, row, col));
      hi[slot_i] = lds_read_tr_asm(addr(which ? aQ : aDO, row + 8, col));
    };
    asm volatile("s_waitcnt lgkmcnt(0)");
#pragma unroll
    for (int i = 0; i < DEPTH; i++) fetch(i, i);
#pragma unroll
    for (int i = 0; i < NF; i++) {
      const int which = i & 1, dt = (i >> 1) % (D / 32), sI = i / (2 * (D / 32));
      const int rem = NF - 1 - i < DEPTH - 1 ? NF - 1 - i : DEPTH - 1;     // fragments still in flight behind i
      if (rem == 3) lgkm_wait_for<6>(lo[i % DEPTH], hi[i % DEPTH]);
      else if (rem == 2) lgkm_wait_for<4>(lo[i % DEPTH], hi[i % DEPTH]);
      else if (rem == 1) lgkm_wait_for<2>(lo[i % DEPTH], hi[i % DEPTH]);
      else lgkm_wait_for<0>(lo[i % DEPTH], hi[i % DEPTH]);
      u32x4_t w = {lo[i % DEPTH][0], lo[i % DEPTH][1], hi[i % DEPTH][0], hi[i % DEPTH][1]};
      const bf16x8_t af = __builtin_bit_cast(bf16x8_t, w);
      if (which) acc_k[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, dsf[sI], acc_k[dt], 0, 0, 0);
      else acc_v[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, pf[sI], acc_v[dt], 0, 0, 0);
      if (i + DEPTH < NF) fetch(i + DEPTH, i % DEPTH);
      if constexpr (ISSUE) {
        constexpr int SP = NF / LC;
        if (i % SP == 1 && i / SP < LC) issue_part(LA + i / SP, ti_issue, slot_issue);
      }
    }
  };

  issue_tile(0, 0);
  issue_tile(1, 1);
  __builtin_amdgcn_s_waitcnt(0x0f70);                 // vmcnt(0)
  __syncthreads();

  f32x16_t sA, dpA, sB, dpB;                          // scores of even / odd halves
  stage_ab(std::false_type{}, std::false_type{}, std::false_type{}, 0, 0, sA, dpA, 0, 0, 0, sB, dpB, 0, 0);
  int slot = 0;                                       // slot of tile ti
  auto tile_step = [&](auto masked_c, int ti) __attribute__((always_inline)) {
    const int nslot = slot == NSLOT - 1 ? 0 : slot + 1;
    const int pslot = slot == 0 ? NSLOT - 1 : slot - 1;   // slot of tile ti-1 = slot of tile ti+2
    // iteration 2*ti: A(half 1 of this tile) with B(half 0), then C(half 0).  The loads of tile ti+2 go out
    // between the MFMAs of this iteration: every wavefront has passed the barrier that ended tile ti-1, whose
    // slot they fill, and they have the second iteration to land.
    stage_ab(masked_c, std::true_type{}, std::true_type{}, slot, 1, sB, dpB, ti, slot, 0, sA, dpA, ti + 2, pslot);
    stage_c(std::true_type{}, slot, 0, ti + 2, pslot);
    // iteration 2*ti+1: A(half 0 of the next tile) with B(half 1), then C(half 1)
    stage_ab(masked_c, std::true_type{}, std::false_type{}, nslot, 0, sA, dpA, ti, slot, 1, sB, dpB, 0, 0);
    stage_c(std::false_type{}, slot, 1, 0, 0);
    // Tile ti is finished.  Own part of tile ti+2 must have landed; after the barrier every wavefront is done
    // with tile ti and sees tile ti+2.
    __builtin_amdgcn_s_waitcnt(0x0f70);               // vmcnt(0)
    __builtin_amdgcn_s_barrier();
    slot = nslot;
  };
  // Only the first two query tiles of a key block can hold queries that precede its keys.
  int ti = 0;
  for (; ti < nt && ti < 2; ti++) tile_step(std::true_type{}, ti);
  for (; ti < nt; ti++) tile_step(std::false_type{}, ti);
  __builtin_amdgcn_s_waitcnt(0x0f70);                 // loads past the last tile
  __syncthreads();

  // Output through LDS for row-contiguous 16-byte stores (layout as in the forward kernel):
  // dK (scaled), then dV, of this wavefront's 32 keys.
  {
    constexpr int CH = D / 8, RB = D * 2;
    EMI_LDS uint8_t* wl = smem + wave * (32 * RB);
    const int r = lane & 31, g = lane >> 5;
    const float* trow = (unrope != nullptr && krow < seq) ? unrope + (int64_t)krow * D : nullptr;   // dK only
#pragma unroll
    for (int which = 0; which < 2; which++) {
      const float mul = which ? 1.0f : scale;
#pragma unroll
      for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
          const f32x16_t& a = which ? acc_v[dt] : acc_k[dt];
          float x0 = a[4 * jj] * mul, x1 = a[4 * jj + 1] * mul, x2 = a[4 * jj + 2] * mul, x3 = a[4 * jj + 3] * mul;
          if (which == 0 && trow != nullptr) unrope_quad(trow + dt * 32 + 8 * jj + 4 * g, x0, x1, x2, x3);
          u32x2_t w;
          w[0] = pack_bf16x2(x0, x1);
          w[1] = pack_bf16x2(x2, x3);
          const int c = dt * 4 + jj;
          *reinterpret_cast<EMI_LDS u32x2_t*>(wl + r * RB + ((c ^ (r & (CH - 1))) << 4) + ((g ^ ((r / CH) & 1)) << 3)) = w;
        }
      uint16_t* out = which ? dv : dk;
#pragma unroll
      for (int it = 0; it < 32 * CH / 64; it++) {
        const int row = it * (64 / CH) + lane / CH, c = lane % CH;
        u32x4_t v4 = *reinterpret_cast<const EMI_LDS u32x4_t*>(wl + row * RB + ((c ^ (row & (CH - 1))) << 4));
        if ((row / CH) & 1) v4 = __builtin_shufflevector(v4, v4, 2, 3, 0, 1);
        if (k0 + row < seq) *reinterpret_cast<u32x4_t*>(out + base + (int64_t)(k0 + row) * sh.ss + c * 8) = v4;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Forward mode (tangent) of attention on the matrix cores; same transposed formulation as
// the forward kernel (lane = query).  Per 64-key tile and 32-key half:
//   S^T = K Q^T,  tS^T = K tQ^T + tK Q^T,  p = exp2(S c - lse2),  w = p tS scale
//   A_w^T += V^T w^T,  A_o^T += V^T p^T,  A_t^T += tV^T p^T,  mu += sum_keys w
// and finally  to = A_w - mu A_o + A_t  (tP = P (tS - rowsum(P tS)), to = tP V + P tV).
// Block = 4 wavefronts x 32 queries, one wavefront per SIMD (three output accumulators);
// K, V, tK, tV tiles double-buffered in LDS.  A null tangent is zero and its products are
// skipped (block-uniform branches).
// ---------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void attn_jvp_bf16_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k,
                                                            const uint16_t* __restrict__ v, const float* __restrict__ lse,
                                                            const uint16_t* __restrict__ tq, const uint16_t* __restrict__ tk,
                                                            const uint16_t* __restrict__ tv, uint16_t* __restrict__ to,
                                                            AttnShape sh, uint32_t head_bytes, float scale, int causal) {
  constexpr int BQ = 128, BKV = 64, NW = 4;
  constexpr int TILE = BKV * D * 2, STAGE = 4 * TILE;       // K, V, tK, tV
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[];
  EMI_LDS uint8_t* smem = (EMI_LDS uint8_t*)smem_raw;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int blk, bh;
  attn_block_coords(&blk, &bh);
  const int qblk = gridDim.x - 1 - blk;              // longest rows first
  const int64_t base = (int64_t)(bh / sh.heads) * sh.sb + (int64_t)(bh % sh.heads) * sh.sh;
  const int seq = sh.seq;
  const int q0 = qblk * BQ + wave * 32;
  const int qrow = q0 + (lane & 31);
  const float scale_log2e = scale * kLog2e;
  const bool has_tq = tq != nullptr, has_tk = tk != nullptr, has_tv = tv != nullptr;

  bf16x8_t qf[D / 16], tqf[D / 16];
  load_reg_rows<D>(q + base, qrow, seq, sh.ss, lane, qf);
  if (has_tq) load_reg_rows<D>(tq + base, qrow, seq, sh.ss, lane, tqf);
  const float L2 = qrow < seq ? lse[(int64_t)bh * seq + qrow] * kLog2e : 0.f;

  const __amdgpu_buffer_rsrc_t rK = attn_rsrc(k + base, head_bytes);
  const __amdgpu_buffer_rsrc_t rV = attn_rsrc(v + base, head_bytes);
  const __amdgpu_buffer_rsrc_t rTK = attn_rsrc(has_tk ? tk + base : k + base, head_bytes);
  const __amdgpu_buffer_rsrc_t rTV = attn_rsrc(has_tv ? tv + base : v + base, head_bytes);
  const int kv_end = causal ? (qblk * BQ + BQ < seq ? qblk * BQ + BQ : seq) : seq;
  const int nkv = (kv_end + BKV - 1) / BKV;

  f32x16_t acc_w[D / 32], acc_o[D / 32], acc_t[D / 32];
#pragma unroll
  for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc_w[dt][r] = 0.f, acc_o[dt][r] = 0.f, acc_t[dt][r] = 0.f;
  float mu = 0.f;

  auto issue = [&](int j, EMI_LDS uint8_t* dst) __attribute__((always_inline)) {
    load_rows_tile<D, BKV, NW>(rK, dst, wave, lane, j * BKV, seq, sh.ss);
    load_rows_tile<D, BKV, NW>(rV, dst + TILE, wave, lane, j * BKV, seq, sh.ss);
    if (has_tk) load_rows_tile<D, BKV, NW>(rTK, dst + 2 * TILE, wave, lane, j * BKV, seq, sh.ss);
    if (has_tv) load_rows_tile<D, BKV, NW>(rTV, dst + 3 * TILE, wave, lane, j * BKV, seq, sh.ss);
  };
  issue(0, smem);
  __builtin_amdgcn_s_waitcnt(0x0f70);
  __syncthreads();

  for (int j = 0; j < nkv; j++) {
    if (j + 1 < nkv) issue(j + 1, smem + ((j + 1) & 1) * STAGE);
    const EMI_LDS uint8_t* sK = smem + (j & 1) * STAGE;
    const EMI_LDS uint8_t* sV = sK + TILE;
    const EMI_LDS uint8_t* sTK = sK + 2 * TILE;
    const EMI_LDS uint8_t* sTV = sK + 3 * TILE;
    const int key0 = j * BKV;
    if (!(causal && key0 > q0 + 31)) {     // wave-uniform: this tile is not entirely in the future
      const bool need_mask = (causal && key0 + BKV - 1 > q0) || key0 + BKV > seq;
#pragma unroll 1
      for (int T = 0; T < 2; T++) {
        f32x16_t s, ts;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.f, ts[r] = 0.f;
#pragma unroll
        for (int t = 0; t < D / 16; t++) {
          const bf16x8_t kf = row_frag<D>(sK, T * 32, t, lane);
          s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[t], s, 0, 0, 0);
          if (has_tq) ts = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, tqf[t], ts, 0, 0, 0);
        }
        if (has_tk) {
#pragma unroll
          for (int t = 0; t < D / 16; t++)
            ts = __builtin_amdgcn_mfma_f32_32x32x16_bf16(row_frag<D>(sTK, T * 32, t, lane), qf[t], ts, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float p = fast_exp2(fmaf(s[r], scale_log2e, -L2));
          if (need_mask) {
            const int key = key0 + T * 32 + acc_row(r, lane);
            if ((causal && key > qrow) || key >= seq) p = 0.f;
          }
          const float w = p * ts[r] * scale;
          mu += w;
          s[r] = p;
          ts[r] = w;
        }
#pragma unroll
        for (int sI = 0; sI < 2; sI++) {
          const bf16x8_t pf = acc_to_frag(s, sI), wf = acc_to_frag(ts, sI);
#pragma unroll
          for (int dt = 0; dt < D / 32; dt++) {
            const bf16x8_t vt = col_frag<D>(sV, T * 32 + sI * 16, dt * 32, lane);
            acc_o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vt, pf, acc_o[dt], 0, 0, 0);
            if (has_tq || has_tk) acc_w[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vt, wf, acc_w[dt], 0, 0, 0);
          }
          if (has_tv) {
#pragma unroll
            for (int dt = 0; dt < D / 32; dt++)
              acc_t[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(col_frag<D>(sTV, T * 32 + sI * 16, dt * 32, lane), pf,
                                                                  acc_t[dt], 0, 0, 0);
          }
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
  }

  // a lane pair (l, l ^ 32) holds the two halves of a query's keys
  mu += __shfl_xor(mu, 32, 64);
  {
    constexpr int CH = D / 8, RB = D * 2;
    EMI_LDS uint8_t* wl = smem + wave * (32 * RB);
    const int r = lane & 31, g = lane >> 5;
#pragma unroll
    for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
      for (int jj = 0; jj < 4; jj++) {
        float o4[4];
#pragma unroll
        for (int e = 0; e < 4; e++) o4[e] = acc_w[dt][4 * jj + e] - mu * acc_o[dt][4 * jj + e] + acc_t[dt][4 * jj + e];
        u32x2_t w;
        w[0] = pack_bf16x2(o4[0], o4[1]);
        w[1] = pack_bf16x2(o4[2], o4[3]);
        const int c = dt * 4 + jj;
        *reinterpret_cast<EMI_LDS u32x2_t*>(wl + r * RB + ((c ^ (r & (CH - 1))) << 4) + ((g ^ ((r / CH) & 1)) << 3)) = w;
      }
#pragma unroll
    for (int it = 0; it < 32 * CH / 64; it++) {
      const int row = it * (64 / CH) + lane / CH, c = lane % CH;
      u32x4_t v4 = *reinterpret_cast<const EMI_LDS u32x4_t*>(wl + row * RB + ((c ^ (row & (CH - 1))) << 4));
      if ((row / CH) & 1) v4 = __builtin_shufflevector(v4, v4, 2, 3, 0, 1);
      if (q0 + row < seq) *reinterpret_cast<u32x4_t*>(to + base + (int64_t)(q0 + row) * sh.ss + c * 8) = v4;
    }
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

struct AttnArgs {
  int64_t batch, heads, seq, d, sb, sh, ss;
};

static int check_common(const char* name, const AttnArgs& a, int dtype) {
  EMI_REQUIRE(a.batch >= 0 && a.heads > 0 && a.seq > 0 && a.d > 0, "%s: bad shape [%lld,%lld,%lld,%lld]", name,
              (long long)a.batch, (long long)a.heads, (long long)a.seq, (long long)a.d);
  EMI_REQUIRE(dtype == EMI_F32 || dtype == EMI_BF16, "%s: unsupported dtype code %d (want 11=f32 or 16=bf16)", name, dtype);
  EMI_REQUIRE(a.d <= 256, "%s: head_dim %lld > 256 is not supported", name, (long long)a.d);
  EMI_REQUIRE(a.ss >= a.d && a.sh > 0 && a.sb > 0, "%s: bad strides (b=%lld h=%lld s=%lld)", name, (long long)a.sb,
              (long long)a.sh, (long long)a.ss);
  EMI_REQUIRE(a.seq <= 0x7fffffff / 4 && a.batch * a.heads <= 65535, "%s: seq or batch*heads too large", name);
  return EMI_OK;
}

// The MFMA path needs 16-byte chunks and 32-bit byte offsets inside one head.
static bool mfma_ok(const AttnArgs& a, int dtype, std::initializer_list<const void*> ptrs) {
  if (dtype != EMI_BF16 || (a.d != 64 && a.d != 128)) return false;
  if ((a.sb % 8) || (a.sh % 8) || (a.ss % 8)) return false;
  if ((a.seq - 1) * a.ss + a.d >= (int64_t)0x3fffff00) return false;
  if ((a.seq + 256) * a.ss >= (int64_t)0x7fffff00) return false;    // tiles addressed past the last row: 32-bit byte offsets
  for (const void* p : ptrs)
    if (!aligned16(p)) return false;
  return true;
}

template <typename K> static int reserve_lds(K kern, int bytes, const char* name) {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return emi_fail(EMI_INTERNAL, "%s: cannot reserve %d bytes of LDS: %s", name, bytes, hipGetErrorString(e));
  return EMI_OK;
}

// Tangent of attention on the MFMA path; -1 when the operands do not qualify (the caller
// then takes the one-wavefront-per-row kernel).
int launch_attn_jvp_mfma(hipStream_t st, const void* q, const void* k, const void* v, const float* lse, const void* tq,
                         const void* tk, const void* tv, void* to, int64_t batch, int64_t heads, int64_t seq, int64_t head_dim,
                         int64_t sb, int64_t shh, int64_t ss, float scale, int causal, int dtype) {
  const AttnArgs a{batch, heads, seq, head_dim, sb, shh, ss};
  if (!mfma_ok(a, dtype, {q, k, v, to, tq ? tq : q, tk ? tk : k, tv ? tv : v}) || seq < 128 || batch * heads > 65535) return -1;
  const AttnShape shp{(int)seq, (int)heads, sb, shh, ss};
  const uint32_t head_bytes = (uint32_t)(((seq - 1) * ss + head_dim) * 2);
  const dim3 grid((unsigned)((seq + 127) / 128), (unsigned)(batch * heads));
#define EMI_ATTN_JVP(DD)                                                                                                 \
  do {                                                                                                                   \
    constexpr int smem = 2 * 4 * 64 * DD * 2;                                                                            \
    if (int rc = reserve_lds(attn_jvp_bf16_kernel<DD>, smem, "emi_attn_jvp")) return rc;                                 \
    hipLaunchKernelGGL(attn_jvp_bf16_kernel<DD>, grid, dim3(256), smem, st, (const uint16_t*)q, (const uint16_t*)k,      \
                       (const uint16_t*)v, lse, (const uint16_t*)tq, (const uint16_t*)tk, (const uint16_t*)tv,           \
                       (uint16_t*)to, shp, head_bytes, scale, causal);                                                   \
  } while (0)
  if (head_dim == 128) EMI_ATTN_JVP(128);
  else EMI_ATTN_JVP(64);
#undef EMI_ATTN_JVP
  EMI_CHECK_LAUNCH("emi_attn_jvp");
  return EMI_OK;
}

// attention_f32.hip: the fp32 matrix-core kernels (head_dim a multiple of 16, 16-byte aligned rows); -1 = not applicable
int launch_attn_fwd_f32_mfma(hipStream_t st, const void* q, const void* k, const void* v, void* o, float* lse, int64_t batch,
                             int64_t heads, int64_t seq, int64_t head_dim, int64_t sb, int64_t shh, int64_t ss, float scale,
                             int causal);
int launch_attn_bwd_f32_mfma(hipStream_t st, const void* q, const void* k, const void* v, const void* d_o, const float* lse,
                             const float* delta, void* dq, void* dk, void* dv, int64_t batch, int64_t heads, int64_t seq,
                             int64_t head_dim, int64_t sb, int64_t shh, int64_t ss, float scale, int causal);

}  // namespace emi

using namespace emi;


// The generic kernels read four elements per load when every row starts on a 4-element boundary (8 bytes of bf16,
// 16 of fp32) and head_dim is a multiple of 4.
static inline int rows_vec4(int dtype, int64_t head_dim, int64_t sb, int64_t sh, int64_t ss, std::initializer_list<const void*> ptrs) {
  const uintptr_t mask = dtype == EMI_BF16 ? 7 : 15;
  if ((head_dim | sb | sh | ss) & 3) return 0;
  for (const void* p : ptrs)
    if (reinterpret_cast<uintptr_t>(p) & mask) return 0;
  return 1;
}

extern "C" size_t emi_attn_fwd_workspace_bytes(int64_t batch, int64_t heads, int64_t seq, int64_t head_dim) {
  (void)batch; (void)heads; (void)seq; (void)head_dim;
  return 0;          // the forward kernels need no scratch (V is transposed by the LDS reads)
}

extern "C" int emi_attn_fwd_ws(emi_stream_t stream, const void* q, const void* k, const void* v, void* o, float* lse,
                               void* workspace, size_t workspace_bytes, int64_t batch, int64_t heads, int64_t seq,
                               int64_t head_dim, int64_t stride_b, int64_t stride_h, int64_t stride_s, float scale,
                               int causal, int dtype) {
  const AttnArgs a{batch, heads, seq, head_dim, stride_b, stride_h, stride_s};
  if (int rc = check_common("emi_attn_fwd", a, dtype)) return rc;
  if (batch == 0) return EMI_OK;
  EMI_REQUIRE(q && k && v && o && lse, "emi_attn_fwd: null buffer");
  (void)workspace; (void)workspace_bytes;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const AttnShape shp{(int)seq, (int)heads, stride_b, stride_h, stride_s};
  const unsigned bh = (unsigned)(batch * heads);
  if (mfma_ok(a, dtype, {q, k, v, o})) {
    const uint32_t head_bytes = (uint32_t)(((seq - 1) * stride_s + head_dim) * 2);
    const float sl2 = scale * kLog2e;
    // 256-query blocks; at 512 keys and fewer the 128-query kernel below is faster (25 vs 31 us at 16 x 12 x 512 x 64)
    if (seq > 512) {
      const dim3 gridp((unsigned)((seq + 255) / 256), bh);
#define EMI_ATTN_FWD_PP(DD)                                                                                          \
  do {                                                                                                               \
    constexpr int smem = 3 * 2 * 64 * DD * 2;                                                                        \
    if (int rc = reserve_lds(attn_fwd_pp_kernel<DD>, smem, "emi_attn_fwd")) return rc;                               \
    hipLaunchKernelGGL(attn_fwd_pp_kernel<DD>, gridp, dim3(512), smem, st, (const uint16_t*)q, (const uint16_t*)k,   \
                       (const uint16_t*)v, (uint16_t*)o, lse, shp, head_bytes, sl2, causal);                         \
  } while (0)
      if (head_dim == 128) EMI_ATTN_FWD_PP(128);
      else EMI_ATTN_FWD_PP(64);
#undef EMI_ATTN_FWD_PP
      EMI_CHECK_LAUNCH("emi_attn_fwd");
      return EMI_OK;
    }
    const dim3 grid((unsigned)((seq + 127) / 128), bh);
    if (head_dim == 128) {
      constexpr int smem = 2 * 2 * 64 * 128 * 2;
      if (int rc = reserve_lds(attn_fwd_bf16_kernel<128>, smem, "emi_attn_fwd")) return rc;
      hipLaunchKernelGGL(attn_fwd_bf16_kernel<128>, grid, dim3(256), smem, st, (const uint16_t*)q, (const uint16_t*)k,
                         (const uint16_t*)v, (uint16_t*)o, lse, shp, head_bytes, sl2, causal);
    } else {
      constexpr int smem = 2 * 2 * 64 * 64 * 2;
      if (int rc = reserve_lds(attn_fwd_bf16_kernel<64>, smem, "emi_attn_fwd")) return rc;
      hipLaunchKernelGGL(attn_fwd_bf16_kernel<64>, grid, dim3(256), smem, st, (const uint16_t*)q, (const uint16_t*)k,
                         (const uint16_t*)v, (uint16_t*)o, lse, shp, head_bytes, sl2, causal);
    }
    EMI_CHECK_LAUNCH("emi_attn_fwd");
    return EMI_OK;
  }
  if (dtype == EMI_F32) {
    const int rc = launch_attn_fwd_f32_mfma(st, q, k, v, o, lse, batch, heads, seq, head_dim, stride_b, stride_h, stride_s,
                                            scale, causal);
    if (rc >= 0) return rc;
  }
  const dim3 grid((unsigned)((seq + 3) / 4), bh);
  const int vec4 = rows_vec4(dtype, head_dim, shp.sb, shp.sh, shp.ss, {q, k});
  if (dtype == EMI_BF16)
    hipLaunchKernelGGL(attn_fwd_generic_kernel<bf16>, grid, dim3(256), 0, st, (const bf16*)q, (const bf16*)k,
                       (const bf16*)v, (bf16*)o, lse, shp, (int)head_dim, scale, causal, vec4);
  else
    hipLaunchKernelGGL(attn_fwd_generic_kernel<float>, grid, dim3(256), 0, st, (const float*)q, (const float*)k,
                       (const float*)v, (float*)o, lse, shp, (int)head_dim, scale, causal, vec4);
  EMI_CHECK_LAUNCH("emi_attn_fwd(generic)");
  return EMI_OK;
}

extern "C" int emi_attn_fwd(emi_stream_t stream, const void* q, const void* k, const void* v, void* o, float* lse,
                            int64_t batch, int64_t heads, int64_t seq, int64_t head_dim, int64_t stride_b,
                            int64_t stride_h, int64_t stride_s, float scale, int causal, int dtype) {
  return emi_attn_fwd_ws(stream, q, k, v, o, lse, nullptr, 0, batch, heads, seq, head_dim, stride_b, stride_h, stride_s,
                         scale, causal, dtype);
}

extern "C" size_t emi_attn_bwd_workspace_bytes(int64_t batch, int64_t heads, int64_t seq, int64_t head_dim) {
  (void)head_dim;
  if (batch <= 0 || heads <= 0 || seq <= 0) return 0;
  return 2 * (size_t)batch * (size_t)heads * (size_t)seq * sizeof(float);   // delta = rowsum(dO * O), lse * log2(e)
}

extern "C" int emi_rope(emi_stream_t stream, const void* x, const float* table, void* y, int64_t batch, int64_t seq,
                        int64_t heads, int64_t head_dim, int inverse, int dtype);

// unrope: null, or the RoPE angle table [seq, head_dim/2] of (cos, sin): dq and dk are then the cotangents of the
// vectors before their rotation (the MFMA kernels turn them back as they store them; otherwise a pass over each).
static int attn_bwd_impl(emi_stream_t stream, const void* q, const void* k, const void* v, const void* o, const float* lse,
                         const void* d_o, void* dq, void* dk, void* dv, void* workspace, size_t workspace_bytes, int64_t batch,
                         int64_t heads, int64_t seq, int64_t head_dim, int64_t stride_b, int64_t stride_h, int64_t stride_s,
                         float scale, int causal, int dtype, const float* unrope) {
  const AttnArgs a{batch, heads, seq, head_dim, stride_b, stride_h, stride_s};
  if (int rc = check_common("emi_attn_bwd", a, dtype)) return rc;
  if (batch == 0) return EMI_OK;
  EMI_REQUIRE(q && k && v && o && lse && d_o && dq && dk && dv, "emi_attn_bwd: null buffer");
  if (unrope != nullptr) {
    EMI_REQUIRE((reinterpret_cast<uintptr_t>(unrope) & 15) == 0, "emi_attn_bwd_rope: the angle table must be 16-byte aligned");
    if (!mfma_ok(a, dtype, {q, k, v, o, d_o, dq, dk, dv})) {
      EMI_REQUIRE(stride_h == head_dim && stride_s == heads * head_dim && stride_b == seq * stride_s,
                  "emi_attn_bwd_rope: this shape needs contiguous [batch, seq, heads, head_dim] operands");
      int rc = attn_bwd_impl(stream, q, k, v, o, lse, d_o, dq, dk, dv, workspace, workspace_bytes, batch, heads, seq, head_dim,
                             stride_b, stride_h, stride_s, scale, causal, dtype, nullptr);
      if (rc == EMI_OK) rc = emi_rope(stream, dq, unrope, dq, batch, seq, heads, head_dim, 1, dtype);
      if (rc == EMI_OK) rc = emi_rope(stream, dk, unrope, dk, batch, seq, heads, head_dim, 1, dtype);
      return rc;
    }
  }
  const size_t need = emi_attn_bwd_workspace_bytes(batch, heads, seq, head_dim);
  EMI_REQUIRE(workspace != nullptr && workspace_bytes >= need, "emi_attn_bwd: workspace of %zu bytes needed, got %zu", need,
              workspace_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const AttnShape shp{(int)seq, (int)heads, stride_b, stride_h, stride_s};
  const unsigned bh = (unsigned)(batch * heads);
  float* delta = static_cast<float*>(workspace);
  float* lse2 = delta + (size_t)batch * heads * seq;
  const dim3 grid4((unsigned)((seq + 3) / 4), bh);
  const bool fast = mfma_ok(a, dtype, {q, k, v, o, d_o, dq, dk, dv});
  const float delta_sign = -1.0f;          // the MFMA kernels accumulate dP onto -delta
  if (fast) {
    // the dQ kernel computes delta and lse * log2(e) for its own queries and leaves them for the dK/dV kernel
  } else if (dtype == EMI_BF16)
    hipLaunchKernelGGL(attn_delta_kernel<bf16>, grid4, dim3(256), 0, st, (const bf16*)o, (const bf16*)d_o, delta, shp,
                       (int)head_dim);
  else
    hipLaunchKernelGGL(attn_delta_kernel<float>, grid4, dim3(256), 0, st, (const float*)o, (const float*)d_o, delta, shp,
                       (int)head_dim);
  EMI_CHECK_LAUNCH("emi_attn_bwd(delta)");
  if (fast) {
    const uint32_t head_bytes = (uint32_t)(((seq - 1) * stride_s + head_dim) * 2);
    const dim3 grid((unsigned)((seq + 127) / 128), bh);
#define EMI_ATTN_BWD_LAUNCH(DD)                                                                                          \
  do {                                                                                                                   \
    constexpr int smem_q = 2 * 2 * 64 * DD * 2;                                                                          \
    constexpr int smem_sp = 6 * 64 * DD * 2 + 3 * 512;                                                                   \
    if (int rc = reserve_lds(attn_bwd_dq_bf16_kernel<DD>, smem_q, "emi_attn_bwd")) return rc;                            \
    hipLaunchKernelGGL(attn_bwd_dq_bf16_kernel<DD>, grid, dim3(256), smem_q, st, (const uint16_t*)q, (const uint16_t*)k, \
                       (const uint16_t*)v, (const uint16_t*)d_o, lse, (const float*)nullptr, (uint16_t*)dq, shp,         \
                       head_bytes, scale, causal, delta_sign, unrope, (const uint16_t*)o, delta, lse2);                  \
    EMI_CHECK_LAUNCH("emi_attn_bwd(dq)");                                                                                \
    if (int rc = reserve_lds(attn_bwd_dkv_sp_kernel<DD>, smem_sp, "emi_attn_bwd")) return rc;                            \
    hipLaunchKernelGGL(attn_bwd_dkv_sp_kernel<DD>, grid, dim3(256), smem_sp, st, (const uint16_t*)q,                     \
                       (const uint16_t*)k, (const uint16_t*)v, (const uint16_t*)d_o, lse2, delta, (uint16_t*)dk,         \
                       (uint16_t*)dv, shp, head_bytes, scale, causal, unrope);                                           \
  } while (0)
    if (head_dim == 128) EMI_ATTN_BWD_LAUNCH(128);
    else EMI_ATTN_BWD_LAUNCH(64);
#undef EMI_ATTN_BWD_LAUNCH
    EMI_CHECK_LAUNCH("emi_attn_bwd(dkv)");
    return EMI_OK;
  }
  if (dtype == EMI_F32) {
    const int rc = launch_attn_bwd_f32_mfma(st, q, k, v, d_o, lse, delta, dq, dk, dv, batch, heads, seq, head_dim, stride_b,
                                            stride_h, stride_s, scale, causal);
    if (rc >= 0) return rc;
  }
  const int vec4 = rows_vec4(dtype, head_dim, shp.sb, shp.sh, shp.ss, {q, k, v, d_o});
  if (dtype == EMI_BF16) {
    hipLaunchKernelGGL(attn_bwd_dq_generic_kernel<bf16>, grid4, dim3(256), 0, st, (const bf16*)q, (const bf16*)k,
                       (const bf16*)v, (const bf16*)d_o, lse, delta, (bf16*)dq, shp, (int)head_dim, scale, causal, vec4);
    hipLaunchKernelGGL(attn_bwd_dkv_generic_kernel<bf16>, grid4, dim3(256), 0, st, (const bf16*)q, (const bf16*)k,
                       (const bf16*)v, (const bf16*)d_o, lse, delta, (bf16*)dk, (bf16*)dv, shp, (int)head_dim, scale,
                       causal, vec4);
  } else {
    hipLaunchKernelGGL(attn_bwd_dq_generic_kernel<float>, grid4, dim3(256), 0, st, (const float*)q, (const float*)k,
                       (const float*)v, (const float*)d_o, lse, delta, (float*)dq, shp, (int)head_dim, scale, causal, vec4);
    hipLaunchKernelGGL(attn_bwd_dkv_generic_kernel<float>, grid4, dim3(256), 0, st, (const float*)q, (const float*)k,
                       (const float*)v, (const float*)d_o, lse, delta, (float*)dk, (float*)dv, shp, (int)head_dim, scale,
                       causal, vec4);
  }
  EMI_CHECK_LAUNCH("emi_attn_bwd(generic)");
  return EMI_OK;
}

extern "C" int emi_attn_bwd(emi_stream_t stream, const void* q, const void* k, const void* v, const void* o,
                            const float* lse, const void* d_o, void* dq, void* dk, void* dv, void* workspace,
                            size_t workspace_bytes, int64_t batch, int64_t heads, int64_t seq, int64_t head_dim,
                            int64_t stride_b, int64_t stride_h, int64_t stride_s, float scale, int causal, int dtype) {
  return attn_bwd_impl(stream, q, k, v, o, lse, d_o, dq, dk, dv, workspace, workspace_bytes, batch, heads, seq, head_dim,
                       stride_b, stride_h, stride_s, scale, causal, dtype, nullptr);
}

extern "C" int emi_attn_bwd_rope(emi_stream_t stream, const void* q, const void* k, const void* v, const void* o,
                                 const float* lse, const void* d_o, void* dq, void* dk, void* dv, const float* rope_table,
                                 void* workspace, size_t workspace_bytes, int64_t batch, int64_t heads, int64_t seq,
                                 int64_t head_dim, int64_t stride_b, int64_t stride_h, int64_t stride_s, float scale,
                                 int causal, int dtype) {
  EMI_REQUIRE(rope_table != nullptr || batch == 0, "emi_attn_bwd_rope: null angle table");
  return attn_bwd_impl(stream, q, k, v, o, lse, d_o, dq, dk, dv, workspace, workspace_bytes, batch, heads, seq, head_dim,
                       stride_b, stride_h, stride_s, scale, causal, dtype, rope_table);
}
