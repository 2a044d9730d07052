// GEMM for the llama projections, FFN and their adjoints on gfx950 MFMA.
//
//   C[M,N] = op(A) . op(B) [+ R]      fp32 accumulate, one rounding at the end
//
// Fast path (bf16): v_mfma_f32_32x32x16_bf16, block tile BM x BN x 64, operands
// streamed HBM -> LDS with 16-byte direct-to-LDS buffer loads (no VGPR
// staging; out-of-range chunks read as zero), two LDS stages, XOR-swizzled so
// both the k-contiguous reads (ds_read_b128) and the k-major reads
// (ds_read_b64_tr_b16, the transposing LDS load) are bank-conflict free.
// One kernel template covers the three operand layouts of the path:
//   NT  Y  = X . W^T    (A k-contiguous, B k-contiguous)   forward
//   NN  dX = dY . W     (A k-contiguous, B k-major)        input adjoint
//   TN  dW = dY^T . X   (A k-major,      B k-major)        weight adjoint
// Generic path (fp32, or bf16 with shapes/alignments the fast path does not
// take): v_mfma_f32_32x32x2_f32 with predicated scalar loads.
#include <stdlib.h>
#include <type_traits>
#include <utility>

#include "emi_device.h"

namespace emi {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

#define EMI_LDS __attribute__((address_space(3)))

constexpr uint32_t kOob = 0x80000000u;   // beyond any buffer's num_records: loads return 0

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

// XCD-aware tile order: consecutive workgroup ids land on different XCDs
// (8 of them, each with its own L2), so give every XCD a contiguous run of
// tiles, and walk tiles in groups of GROUP_M tile-rows so that the A and B
// panels a XCD touches stay in its L2.
// Several products of one shape in one launch of the 128x128 kernel (emi_gemm_grouped).  count == 0: the plain
// single product.  sum == 0: independent results C[i] = op(A[i]) . op(B[i]) [+ R[i]], the grid holds count times the
// tiles; sum == 1: every product is accumulated into the tile of C[0] (+ R[0]), pair after pair.
constexpr int kMaxGroup = 48;      // products per launch (the argument block stays under 2 KB)
struct GemmGroup {
  const uint16_t* A[kMaxGroup];
  const uint16_t* B[kMaxGroup];
  const uint16_t* R[kMaxGroup];
  uint16_t* C[kMaxGroup];
  int count, sum;
};
struct NoGroup {};       // placeholder argument of the kernels' ungrouped instantiations

__device__ __forceinline__ int xcd_contiguous_id() {
  const int nb = gridDim.x, bid = blockIdx.x;
  const int per = nb >> 3, rem = nb & 7;
  const int xcd = bid & 7, idx = bid >> 3;
  return xcd * per + (xcd < rem ? xcd : rem) + idx;
}

template <int GROUP_M = 8>
__device__ __forceinline__ void tile_coords(int pid, int tiles_m, int tiles_n, int* tm, int* tn) {
  const int group_size = GROUP_M * tiles_n;
  const int group = pid / group_size;
  const int first_m = group * GROUP_M;
  const int gm = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int in_group = pid - group * group_size;
  *tm = first_m + in_group % gm;
  *tn = in_group / gm;
}

// --- LDS tile layouts -------------------------------------------------------
// The LDS serves 256 bytes (64 banks) per clock: 16 lanes of a ds_read_b128.
// k-contiguous operand tile: [rows][BK] bf16.  Rows are 2*BK bytes, so 256/(2*BK)
// rows share one 256-byte bank line; 16-byte chunk c of row r is stored at chunk
// c ^ swz_kc(r), which spreads 16 consecutive rows at one logical chunk (one
// MFMA operand fetch) over all 16 slots of the line.
// k-major operand tile: [BK][COLS] bf16 (COLS*2-byte rows, a multiple of 256):
// chunk c of row k is stored at chunk c ^ (4 * (k & 3)), which does the same for
// the 4 rows x 64 bytes that 32 lanes of a transposing ds_read_b64_tr_b16 touch.

template <int BK> __device__ __forceinline__ int swz_kc(int row) {
  static_assert(BK == 64 || BK == 32, "BK");
  return BK == 64 ? ((row >> 1) & 7) : ((row >> 2) & 3);
}

// One 1 KiB wave-load (number `it` of this wave) of a k-contiguous tile.
template <int BK, int NW>
__device__ __forceinline__ void load_one_kcontig(__amdgpu_buffer_rsrc_t rsrc, EMI_LDS uint8_t* lds, int wave, int lane,
                                                 uint32_t row0_off_bytes, int ld, int k0, int K, int it) {
  constexpr int CPR = BK / 8;                 // 16-byte chunks per row
  constexpr int RPW = 64 / CPR;               // rows per 1 KiB wave-load
  const int r_in = lane / CPR, pc = lane % CPR;
  const int r = (it * NW + wave) * RPW + r_in;
  const int lc = pc ^ swz_kc<BK>(r);
  const int k = k0 + lc * 8;
  uint32_t voff = row0_off_bytes + (uint32_t)(r * ld + k) * 2u;
  if (k >= K) voff = kOob;
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, lds + (it * NW + wave) * 1024, 16, voff, 0, 0, 0);
}

template <int ROWS, int BK, int NW>
__device__ __forceinline__ void load_tile_kcontig(__amdgpu_buffer_rsrc_t rsrc, EMI_LDS uint8_t* lds, int wave, int lane,
                                                  uint32_t row0_off_bytes, int ld, int k0, int K) {
  constexpr int NLOAD = ROWS * BK * 2 / 1024 / NW;
  static_assert(NLOAD >= 1, "tile smaller than one pass of the block");
#pragma unroll
  for (int it = 0; it < NLOAD; it++) load_one_kcontig<BK, NW>(rsrc, lds, wave, lane, row0_off_bytes, ld, k0, K, it);
}

template <int COLS, int NW>
__device__ __forceinline__ void load_one_kmajor(__amdgpu_buffer_rsrc_t rsrc, EMI_LDS uint8_t* lds, int wave, int lane,
                                                int col0, int ncols, int ld, int k0, int K, int it) {
  constexpr int CPR = COLS / 8;               // 16-byte chunks per k-row
  static_assert(CPR >= 16, "k-major tile too narrow");
  const int slot = (it * NW + wave) * 64 + lane;
  const int k = slot / CPR, pc = slot % CPR;
  const int lc = pc ^ (4 * (k & 3));
  const int col = col0 + lc * 8;
  uint32_t voff = (uint32_t)((k0 + k) * ld + col) * 2u;
  if (k0 + k >= K || col >= ncols) voff = kOob;
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, lds + (it * NW + wave) * 1024, 16, voff, 0, 0, 0);
}

template <int COLS, int BK, int NW>
__device__ __forceinline__ void load_tile_kmajor(__amdgpu_buffer_rsrc_t rsrc, EMI_LDS uint8_t* lds, int wave, int lane,
                                                 int col0, int ncols, int ld, int k0, int K) {
  constexpr int NLOAD = BK * COLS * 2 / 1024 / NW;
  static_assert(NLOAD >= 1, "tile smaller than one pass of the block");
#pragma unroll
  for (int it = 0; it < NLOAD; it++) load_one_kmajor<COLS, NW>(rsrc, lds, wave, lane, col0, ncols, ld, k0, K, it);
}

// MFMA operand fragment (32 rows x 16 k) for k-step kk of the tile.
// Lane l holds row (l & 31), k = 8*(l >> 5) + 0..7 of the step.
template <int BK>
__device__ __forceinline__ bf16x8_t frag_kcontig(const EMI_LDS uint8_t* tile, int row_base, int kk, int lane) {
  const int row = row_base + (lane & 31);
  const int chunk = (kk * 2 + (lane >> 5)) ^ swz_kc<BK>(row);
  return *reinterpret_cast<const EMI_LDS bf16x8_t*>(tile + row * (BK * 2) + chunk * 16);
}

// Same fragment out of a k-major tile with two transposing loads.  Within a
// 16-lane group, lane i supplies the address of k-row (i >> 2), columns
// 4*(i & 3).. +3, and receives column (i), k-rows 0..3.
template <int COLS>
__device__ __forceinline__ bf16x8_t frag_kmajor(const EMI_LDS uint8_t* tile, int col_base, int kk, int lane) {
  const int i = lane & 15;
  const int kq = i >> 2;                                        // k & 3 of the row this lane addresses
  const int col = col_base + ((lane >> 4) & 1) * 16 + (i & 3) * 4;
  const int krow = kk * 16 + (lane >> 5) * 8 + kq;
  const int chunk = (col >> 3) ^ (4 * kq);
  const EMI_LDS uint8_t* p = tile + krow * (COLS * 2) + chunk * 16 + (col & 7) * 2;
  bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((EMI_LDS bf16x4_t*)p);
  bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((EMI_LDS bf16x4_t*)(p + 4 * COLS * 2));
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// s_waitcnt vmcnt(N) with the other counters left alone.
template <int N> __device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0f70);
}

// Epilogue shared by the bf16 kernels.  With swapped MFMA operands register r of
// lane l holds C[row = l%32][col = 8*(r/4) + 4*(l/32) + r%4] of its 32x32 tile:
// four consecutive columns per register quad.  Each wave stages its WR x WC
// sub-tile (rows rbase.., columns cbase..) through its own slice of the now idle
// LDS as bf16 and writes it out with 16-byte, row-contiguous stores; the residual
// comes in the same way (16-byte loads -> LDS -> accumulator layout) and is added
// in fp32 before the single rounding.  Slice layout: rows of 2*WC bytes, chunk c
// of row r at chunk c ^ e_swz(r), the two 8-byte halves of a chunk swapped when
// (r>>4)&1, which makes the 8-byte column-quad accesses of 32 lanes (32 rows)
// conflict free.
template <int WR, int WC, int TM, int TN>
__device__ __forceinline__ void epilogue_bf16(f32x16_t (&acc)[TM][TN], EMI_LDS uint8_t* smem, int wave, int lane,
                                              int rbase, int cbase, const uint16_t* R, uint16_t* C, int M, int N,
                                              int ldr, int ldc, int vec_ok) {
  static_assert(WC == 64 || WC == 128, "epilogue supports 64- or 128-column wave tiles");
  static_assert(WR == TM * 32 && WC == TN * 32, "wave tile");
  constexpr int RSB = WC * 2, CH = WC / 8, RPP = 64 / CH;     // row bytes, chunks per row, rows per 64-lane pass
  EMI_LDS uint8_t* wl = smem + wave * (WR * RSB);
  const int lrow = lane & 31, lhalf = lane >> 5;
  auto e_swz = [](int row) { return WC == 64 ? ((row >> 1) & 7) : (row & 15); };
  auto quad_slot = [&](int row, int chunk) {
    return row * RSB + ((chunk ^ e_swz(row)) << 4) + ((lhalf ^ ((row >> 4) & 1)) << 3);
  };
  if (R != nullptr) {
#pragma unroll
    for (int it = 0; it < WR / RPP; it++) {
      const int row = it * RPP + lane / CH, c = lane % CH;
      const int grow = rbase + row, gcol = cbase + c * 8;
      u32x4_t v = {0u, 0u, 0u, 0u};
      if (grow < M && gcol < N) {
        const uint16_t* src = R + (int64_t)grow * ldr + gcol;
        if (vec_ok && gcol + 8 <= N) {
          v = *reinterpret_cast<const u32x4_t*>(src);
        } else {
#pragma unroll
          for (int e = 0; e < 8; e++)
            if (gcol + e < N) v[e >> 1] |= (uint32_t)src[e] << ((e & 1) * 16);
        }
      }
      if ((row >> 4) & 1) v = __builtin_shufflevector(v, v, 2, 3, 0, 1);
      *reinterpret_cast<EMI_LDS u32x4_t*>(wl + row * RSB + ((c ^ e_swz(row)) << 4)) = v;
    }
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const u32x2_t w = *reinterpret_cast<const EMI_LDS u32x2_t*>(wl + quad_slot(i * 32 + lrow, j * 4 + q));
          acc[i][j][4 * q + 0] += __uint_as_float(w[0] << 16);
          acc[i][j][4 * q + 1] += __uint_as_float(w[0] & 0xffff0000u);
          acc[i][j][4 * q + 2] += __uint_as_float(w[1] << 16);
          acc[i][j][4 * q + 3] += __uint_as_float(w[1] & 0xffff0000u);
        }
  }
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        u32x2_t w;
        w[0] = pack_bf16x2(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1]);
        w[1] = pack_bf16x2(acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
        *reinterpret_cast<EMI_LDS u32x2_t*>(wl + quad_slot(i * 32 + lrow, j * 4 + q)) = w;
      }
#pragma unroll
  for (int it = 0; it < WR / RPP; it++) {
    const int row = it * RPP + lane / CH, c = lane % CH;
    const int grow = rbase + row, gcol = cbase + c * 8;
    u32x4_t v = *reinterpret_cast<const EMI_LDS u32x4_t*>(wl + row * RSB + ((c ^ e_swz(row)) << 4));
    if ((row >> 4) & 1) v = __builtin_shufflevector(v, v, 2, 3, 0, 1);
    if (grow < M && gcol < N) {
      uint16_t* dst = C + (int64_t)grow * ldc + gcol;
      if (vec_ok && gcol + 8 <= N) {
        *reinterpret_cast<u32x4_t*>(dst) = v;
      } else {
#pragma unroll
        for (int e = 0; e < 8; e++)
          if (gcol + e < N) dst[e] = (uint16_t)(v[e >> 1] >> ((e & 1) * 16));
      }
    }
  }
}

// Software pipeline, NSTAGE == 2: tile t+1 streams into the other LDS stage while
// tile t is multiplied; one barrier per tile.
// NSTAGE == 4: tiles t+2 and t+3 are in flight while tile t is multiplied and
// tile t+1 has already landed, so the operand fragments of the first k-step of
// tile t+1 are fetched before the barrier and the MFMA stream never waits on LDS.
// Loads past the end of K are still issued (they read as zeros) so that the
// number of outstanding loads is a compile-time constant.
template <int BM, int BN, int BK, int NSTAGE, int WM, int WN, bool A_KMAJOR, bool B_KMAJOR>
__global__ __launch_bounds__(WM* WN * 64) void gemm_bf16_kernel(const uint16_t* __restrict__ A,
                                                                 const uint16_t* __restrict__ B, const uint16_t* R,
                                                                 uint16_t* C, int M, int N, int K, int lda, int ldb,
                                                                 int ldr, int ldc, uint32_t a_bytes, uint32_t b_bytes,
                                                                 int vec_ok, float* __restrict__ part, int k_per_split,
                                                                 GemmGroup grp) {
  constexpr int NW = WM * WN;
  constexpr int KS = BK / 16;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2, STAGE = A_BYTES + B_BYTES;
  constexpr int LPT = (A_BYTES + B_BYTES) / 1024 / NW;      // direct-to-LDS loads per wave per tile
  static_assert(NSTAGE == 2 || NSTAGE == 4, "NSTAGE");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[];
  EMI_LDS uint8_t* smem = (EMI_LDS uint8_t*)smem_raw;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;

  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  int tile_m, tile_n;
  // split-K: the grid is one run of tiles x splits blocks, split-major, so that the blocks of one XCD work on
  // the same slab of K and that slab of A and B is fetched into one L2 rather than into all eight
  // (a group of independent products: split-major, then product, then tile)
  const int pid = xcd_contiguous_id();
  const int tiles = tiles_m * tiles_n;
  const int nprod = (grp.count > 0 && !grp.sum) ? grp.count : 1;
  const int split = part ? pid / (tiles * nprod) : 0;
  const int in_split = pid - split * tiles * nprod;
  const int prod = in_split / tiles;
  tile_coords(in_split - prod * tiles, tiles_m, tiles_n, &tile_m, &tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  if (grp.count > 0 && !grp.sum) {
    A = grp.A[prod];
    B = grp.B[prod];
    R = grp.R[prod];
    C = grp.C[prod];
    if (part) part += (int64_t)prod * (gridDim.x / (tiles * nprod)) * M * N;
  }
  const int npairs = (grp.count > 0 && grp.sum) ? grp.count : 1;

  __amdgpu_buffer_rsrc_t rA = make_rsrc(A, a_bytes);
  __amdgpu_buffer_rsrc_t rB = make_rsrc(B, b_bytes);

  auto issue_loads = [&](int stage, int k0) {
    EMI_LDS uint8_t* sA = smem + stage * STAGE;
    EMI_LDS uint8_t* sB = sA + A_BYTES;
    if constexpr (A_KMAJOR)
      load_tile_kmajor<BM, BK, NW>(rA, sA, wave, lane, m0, M, lda, k0, K);
    else
      load_tile_kcontig<BM, BK, NW>(rA, sA, wave, lane, (uint32_t)m0 * (uint32_t)lda * 2u, lda, k0, K);
    if constexpr (B_KMAJOR)
      load_tile_kmajor<BN, BK, NW>(rB, sB, wave, lane, n0, N, ldb, k0, K);
    else
      load_tile_kcontig<BN, BK, NW>(rB, sB, wave, lane, (uint32_t)n0 * (uint32_t)ldb * 2u, ldb, k0, K);
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  auto load_frags = [&](int stage, int kk, bf16x8_t (&a)[TM], bf16x8_t (&b)[TN]) {
    const EMI_LDS uint8_t* sA = smem + stage * STAGE;
    const EMI_LDS uint8_t* sB = sA + A_BYTES;
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const int base = wm * (BM / WM) + i * 32;
      if constexpr (A_KMAJOR) a[i] = frag_kmajor<BM>(sA, base, kk, lane);
      else a[i] = frag_kcontig<BK>(sA, base, kk, lane);
    }
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int base = wn * (BN / WN) + j * 32;
      if constexpr (B_KMAJOR) b[j] = frag_kmajor<BN>(sB, base, kk, lane);
      else b[j] = frag_kcontig<BK>(sB, base, kk, lane);
    }
  };
  // The MFMA operands are passed swapped (B fragment first): see the epilogue.
  auto mfma_step = [&](const bf16x8_t (&a)[TM], const bf16x8_t (&b)[TN]) {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[j], a[i], acc[i][j], 0, 0, 0);
  };

  // split-K (part != nullptr): split z owns k in [z * k_per_split, ...) and leaves an fp32 partial
  // tile in part[z][M][N]; gemm_splitk_reduce_kernel adds the partials (and R) in fixed order
  const int k_lo = split * k_per_split;
  if (part) K = k_lo + k_per_split < K ? k_lo + k_per_split : K;
  const int nk = (K - k_lo + BK - 1) / BK;
  // Operand fragments are double buffered: the LDS reads of the next k-step are
  // issued before the MFMAs of the current one so their latency hides behind them.
  bf16x8_t fa[2][TM], fb[2][TN];
  if constexpr (NSTAGE == 2) {
    for (int pair = 0; pair < npairs; pair++) {        // one pass unless several products are summed into this tile
      if (npairs > 1) {
        rA = make_rsrc(grp.A[pair], a_bytes);
        rB = make_rsrc(grp.B[pair], b_bytes);
      }
      issue_loads(0, k_lo);
      wait_vmcnt<0>();
      __syncthreads();
      for (int t = 0; t < nk; t++) {
        if (t + 1 < nk) issue_loads((t + 1) & 1, k_lo + (t + 1) * BK);
        load_frags(t & 1, 0, fa[0], fb[0]);
#pragma unroll
        for (int kk = 0; kk < KS; kk++) {
          if (kk + 1 < KS) load_frags(t & 1, kk + 1, fa[(kk + 1) & 1], fb[(kk + 1) & 1]);
          __builtin_amdgcn_sched_barrier(0);
          mfma_step(fa[kk & 1], fb[kk & 1]);
          __builtin_amdgcn_sched_barrier(0);
        }
        wait_vmcnt<0>();     // next stage has landed
        __syncthreads();     // and everyone is done reading this one
      }
    }
  } else {
    static_assert(KS % 2 == 0, "fragment double buffering assumes an even number of k-steps per tile");
    issue_loads(0, k_lo);
    issue_loads(1, k_lo + BK);
    issue_loads(2, k_lo + 2 * BK);
    wait_vmcnt<LPT>();     // tiles 0 and 1 have landed
    __syncthreads();
    load_frags(0, 0, fa[0], fb[0]);
    for (int t = 0; t < nk; t++) {
      issue_loads((t + 3) & 3, k_lo + (t + 3) * BK);
#pragma unroll
      for (int kk = 0; kk < KS; kk++) {
        if (kk + 1 < KS) load_frags(t & 3, kk + 1, fa[(kk + 1) & 1], fb[(kk + 1) & 1]);
        else load_frags((t + 1) & 3, 0, fa[0], fb[0]);
        __builtin_amdgcn_sched_barrier(0);
        mfma_step(fa[kk & 1], fb[kk & 1]);
        __builtin_amdgcn_sched_barrier(0);
      }
      wait_vmcnt<LPT>();   // everything but the newest tile (t+3) has landed: tiles <= t+2
      __syncthreads();     // visible to all; tile t's stage may be refilled next iteration
    }
    wait_vmcnt<0>();       // drain the zero-filled loads past the end of K before LDS is reused
    __syncthreads();
  }

  constexpr int WR = BM / WM, WC = BN / WN;
  static_assert(NW * WR * WC * 2 <= NSTAGE * STAGE, "epilogue staging does not fit in the LDS allocation");
  if (part != nullptr) {
    // accumulator layout (swapped operands): register 4q+e of lane l holds row l%32, column 8q + 4(l/32) + e
    float* pz = part + (int64_t)split * M * N;
    const bool vec4 = (N & 3) == 0;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const int row = m0 + wm * WR + i * 32 + (lane & 31);
          const int col = n0 + wn * WC + j * 32 + q * 8 + (lane >> 5) * 4;
          if (row < M && col < N) {
            float* dst = pz + (int64_t)row * N + col;
            if (vec4 && col + 4 <= N) {
              *reinterpret_cast<float4*>(dst) = make_float4(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
            } else {
#pragma unroll
              for (int e = 0; e < 4; e++)
                if (col + e < N) dst[e] = acc[i][j][4 * q + e];
            }
          }
        }
    return;
  }
  epilogue_bf16<WR, WC, TM, TN>(acc, smem, wave, lane, m0 + wm * WR, n0 + wn * WC, R, C, M, N, ldr, ldc, vec_ok);
}

// Epilogue for accumulators of v_mfma_f32_16x16x32_bf16 with swapped operands:
// register r of lane l holds C[row = l%16][col = 4*(l/16) + r] of its 16x16 tile.
// The wave tile is (16*TM) x 64; rows of 128 bytes in the wave's LDS slice, 16-byte
// chunk c of row r at chunk c ^ ((r >> 1) & 7): conflict free both for the 8-byte
// column-quad accesses of the accumulator layout and for the 16-byte row accesses
// of the global loads and stores.  CSPLIT: the wave tile's columns 32..63 lie CSPLIT
// columns further right in C (two 32-column strips instead of one 64-column strip).
// ROPE: the rows are token vectors of heads of `rope_hd` elements and the result is stored rotated (test/llama.py:161-168):
// a lane's four consecutive columns are two rotation pairs, whose (cos, sin) entries are 16 bytes of the fp32 table
// [rope_seq, rope_hd/2]; row r sits at position r % rope_seq.  Whole wave tiles only (the launcher checks).
template <int TM, int TN, int CSPLIT = 0, bool ROPE = false, bool FULL = false>
__device__ __forceinline__ void epilogue_bf16_t16(f32x4_t (&acc)[TM][TN], EMI_LDS uint8_t* smem, int wave, int lane,
                                                  int rbase, int cbase, const uint16_t* R, uint16_t* C, int M, int N,
                                                  int ldr, int ldc, int vec_ok, const float* rope = nullptr,
                                                  int rope_seq = 1, int rope_hd = 4) {
  static_assert(TN == 4, "64-column wave tile");
  static_assert(!ROPE || CSPLIT == 0, "rotation pairs are adjacent columns");
  constexpr int WR = TM * 16, RSB = 128;
  EMI_LDS uint8_t* wl = smem + wave * (WR * RSB);
  const int lrow = lane & 15, lq = lane >> 4;
  auto quad_slot = [&](int row, int j) {      // 8-byte slot of columns 16*j + 4*lq .. +3
    const int chunk = 2 * j + (lq >> 1);
    return row * RSB + ((chunk ^ ((row >> 1) & 7)) << 4) + ((lq & 1) << 3);
  };
  // Whole wave tile inside C and 16-byte accesses allowed (wave-uniform): straight-line
  // code, the residual comes in with direct-to-LDS loads that are all in flight at once.
  if (ROPE || FULL || (vec_ok && rbase + WR <= M && cbase + CSPLIT + 64 <= N)) {
    // Wave-load it covers rows 8*it .. 8*it+7: lane l moves physical chunk (l & 7) of row 8*it + (l >> 3),
    // whose swizzle term ((row >> 1) & 7) only depends on the parity of it.
    const int prow = lane >> 3, pc = lane & 7;
    const uint32_t ldsE = prow * RSB + ((pc ^ (prow >> 1)) << 4), ldsO = prow * RSB + ((pc ^ ((prow >> 1) + 4)) << 4);
    if (R != nullptr) {
      const uint8_t* rb = reinterpret_cast<const uint8_t*>(R + (int64_t)rbase * ldr + cbase);   // wave-uniform
      const int cE = pc ^ (prow >> 1), cO = pc ^ ((prow >> 1) + 4);                            // logical chunks
      const uint32_t gE = (uint32_t)prow * (uint32_t)ldr * 2u + (cE << 4) + (cE >= 4 ? CSPLIT * 2 : 0);
      const uint32_t gO = (uint32_t)prow * (uint32_t)ldr * 2u + (cO << 4) + (cO >= 4 ? CSPLIT * 2 : 0);
#pragma unroll
      for (int it = 0; it < WR / 8; it++) {
        const uint8_t* src = rb + (int64_t)it * 16 * ldr + ((it & 1) ? gO : gE);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (EMI_LDS void*)(wl + it * 1024), 16, 0, 0);
      }
      wait_vmcnt<0>();
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
          const u32x2_t w = *reinterpret_cast<const EMI_LDS u32x2_t*>(wl + quad_slot(i * 16 + lrow, j));
          acc[i][j][0] += __uint_as_float(w[0] << 16);
          acc[i][j][1] += __uint_as_float(w[0] & 0xffff0000u);
          acc[i][j][2] += __uint_as_float(w[1] << 16);
          acc[i][j][3] += __uint_as_float(w[1] & 0xffff0000u);
        }
    }
    if constexpr (ROPE) {
      const int hcol = (cbase + 4 * lq) % rope_hd;
      auto rotate = [&](int i, int j, const float4& t) {
        const float x0 = acc[i][j][0], x1 = acc[i][j][1], x2 = acc[i][j][2], x3 = acc[i][j][3];
        acc[i][j][0] = t.x * x0 - t.y * x1;
        acc[i][j][1] = t.y * x0 + t.x * x1;
        acc[i][j][2] = t.z * x2 - t.w * x3;
        acc[i][j][3] = t.w * x2 + t.z * x3;
      };
      const int p0 = rbase % rope_seq;                        // wave-uniform
      if (p0 + WR <= rope_seq) {
        // The wave tile's rows are consecutive positions of one sequence.  The table costs 4 bytes per element, twice
        // what the result does: only the entries of rows p and p + 16 are read, and the angle is advanced from one
        // 16-row block to the next by their difference (a rotation by 16 positions' worth of angle, the same for
        // every block; seven fp32 steps).
        const float* trow = rope + (int64_t)(p0 + lrow) * rope_hd;
        float4 cs[TN], dl[TN];
#pragma unroll
        for (int j = 0; j < TN; j++) {
          const int hc = (hcol + 16 * j) % rope_hd;
          cs[j] = *reinterpret_cast<const float4*>(trow + hc);
          const float4 nx = *reinterpret_cast<const float4*>(trow + 16 * rope_hd + hc);
          dl[j].x = nx.x * cs[j].x + nx.y * cs[j].y;
          dl[j].y = nx.y * cs[j].x - nx.x * cs[j].y;
          dl[j].z = nx.z * cs[j].z + nx.w * cs[j].w;
          dl[j].w = nx.w * cs[j].z - nx.z * cs[j].w;
        }
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < TN; j++) {
            rotate(i, j, cs[j]);
            if (i + 1 < TM) {
              const float4 c = cs[j];
              cs[j].x = c.x * dl[j].x - c.y * dl[j].y;
              cs[j].y = c.y * dl[j].x + c.x * dl[j].y;
              cs[j].z = c.z * dl[j].z - c.w * dl[j].w;
              cs[j].w = c.w * dl[j].z + c.z * dl[j].w;
            }
          }
      } else {
#pragma unroll
        for (int i = 0; i < TM; i++) {
          const float* trow = rope + (int64_t)((rbase + i * 16 + lrow) % rope_seq) * rope_hd;
#pragma unroll
          for (int j = 0; j < TN; j++) rotate(i, j, *reinterpret_cast<const float4*>(trow + (hcol + 16 * j) % rope_hd));
          __builtin_amdgcn_sched_barrier(0);      // one block's table entries in registers at a time
        }
      }
    }
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++) {
        u32x2_t w;
        w[0] = pack_bf16x2(acc[i][j][0], acc[i][j][1]);
        w[1] = pack_bf16x2(acc[i][j][2], acc[i][j][3]);
        *reinterpret_cast<EMI_LDS u32x2_t*>(wl + quad_slot(i * 16 + lrow, j)) = w;
      }
    uint8_t* cb = reinterpret_cast<uint8_t*>(C + (int64_t)rbase * ldc + cbase);                  // wave-uniform
    const uint32_t gC = (uint32_t)prow * (uint32_t)ldc * 2u + (pc << 4) + (pc >= 4 ? CSPLIT * 2 : 0);
#pragma unroll
    for (int it = 0; it < WR / 8; it++) {
      const u32x4_t v = *reinterpret_cast<const EMI_LDS u32x4_t*>(wl + it * 1024 + ((it & 1) ? ldsO : ldsE));
      *reinterpret_cast<u32x4_t*>(cb + (int64_t)it * 16 * ldc + gC) = v;
    }
    return;
  }
  if (R != nullptr) {
#pragma unroll
    for (int it = 0; it < WR / 8; it++) {
      const int row = it * 8 + (lane >> 3), c = lane & 7;
      const int grow = rbase + row, gcol = cbase + c * 8 + (c >= 4 ? CSPLIT : 0);
      u32x4_t v = {0u, 0u, 0u, 0u};
      if (grow < M && gcol < N) {
        const uint16_t* src = R + (int64_t)grow * ldr + gcol;
        if (vec_ok && gcol + 8 <= N) {
          v = *reinterpret_cast<const u32x4_t*>(src);
        } else {
#pragma unroll
          for (int e = 0; e < 8; e++)
            if (gcol + e < N) v[e >> 1] |= (uint32_t)src[e] << ((e & 1) * 16);
        }
      }
      *reinterpret_cast<EMI_LDS u32x4_t*>(wl + row * RSB + ((c ^ ((row >> 1) & 7)) << 4)) = v;
    }
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const u32x2_t w = *reinterpret_cast<const EMI_LDS u32x2_t*>(wl + quad_slot(i * 16 + lrow, j));
        acc[i][j][0] += __uint_as_float(w[0] << 16);
        acc[i][j][1] += __uint_as_float(w[0] & 0xffff0000u);
        acc[i][j][2] += __uint_as_float(w[1] << 16);
        acc[i][j][3] += __uint_as_float(w[1] & 0xffff0000u);
      }
  }
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      u32x2_t w;
      w[0] = pack_bf16x2(acc[i][j][0], acc[i][j][1]);
      w[1] = pack_bf16x2(acc[i][j][2], acc[i][j][3]);
      *reinterpret_cast<EMI_LDS u32x2_t*>(wl + quad_slot(i * 16 + lrow, j)) = w;
    }
#pragma unroll
  for (int it = 0; it < WR / 8; it++) {
    const int row = it * 8 + (lane >> 3), c = lane & 7;
    const int grow = rbase + row, gcol = cbase + c * 8 + (c >= 4 ? CSPLIT : 0);
    const u32x4_t v = *reinterpret_cast<const EMI_LDS u32x4_t*>(wl + row * RSB + ((c ^ ((row >> 1) & 7)) << 4));
    if (grow < M && gcol < N) {
      uint16_t* dst = C + (int64_t)grow * ldc + gcol;
      if (vec_ok && gcol + 8 <= N) {
        *reinterpret_cast<u32x4_t*>(dst) = v;
      } else {
#pragma unroll
        for (int e = 0; e < 8; e++)
          if (gcol + e < N) dst[e] = (uint16_t)(v[e >> 1] >> ((e & 1) * 16));
      }
    }
  }
}

// Epilogues of the ping-pong kernel that apply the SwiGLU of the FFN (test/llama.py:224-231) to the tile instead of
// leaving it to a pass of its own over [tokens, hidden]:
//   MODE 1 (forward, the accumulators hold b = x . W3^T): P0 = a = x . W1^T is read, Q0 = b and Q1 = g = a sigmoid(a) b
//          are written (the elementwise pass would read a and b again and write g);
//   MODE 2 (adjoint, the accumulators hold dg = dy . W2): P0 = a and P1 = b are read, Q0 = da and Q1 = db are written;
//          dg itself never reaches memory (the elementwise pass would read a, b and a stored dg).
// The products are rounded to bf16 before the elementwise arithmetic, as they are when they go through memory.
// Whole 128 x 64 wave tiles inside the matrices and 16-byte accesses only (the launcher checks).  All four matrices
// are [M, N] with leading dimension ld.  Tiles travel through the wavefront's 16 KiB LDS slice as in
// epilogue_bf16_t16: direct-to-LDS loads / 16-byte row stores on the memory side, 8-byte quads on the accumulator side.
template <int MODE>
__device__ __forceinline__ void epilogue_swiglu_t16(f32x4_t (&acc)[8][4], EMI_LDS uint8_t* smem, int wave, int lane, int rbase,
                                                    int cbase, const uint16_t* P0, const uint16_t* P1, uint16_t* Q0,
                                                    uint16_t* Q1, int ld) {
  constexpr int RSB = 128;
  EMI_LDS uint8_t* wl = smem + wave * (128 * RSB);
  const int lrow = lane & 15, lq = lane >> 4;
  auto quad_slot = [&](int row, int j) {      // 8-byte slot of columns 16*j + 4*lq .. +3 of LDS row `row`
    const int chunk = 2 * j + (lq >> 1);
    return row * RSB + ((chunk ^ ((row >> 1) & 7)) << 4) + ((lq & 1) << 3);
  };
  // wave-load / row-store number it covers LDS rows 8*it .. 8*it+7: lane l moves physical chunk (l & 7) of row
  // 8*it + (l >> 3), i.e. logical chunk (l & 7) ^ swizzle(row), whose swizzle only depends on the parity of it
  const int prow = lane >> 3, pc = lane & 7;
  const uint32_t gE = (uint32_t)prow * (uint32_t)ld * 2u + ((pc ^ (prow >> 1)) << 4);
  const uint32_t gO = (uint32_t)prow * (uint32_t)ld * 2u + ((pc ^ ((prow >> 1) + 4)) << 4);
  const uint32_t gC = (uint32_t)prow * (uint32_t)ld * 2u + (pc << 4);
  const uint32_t ldsE = prow * RSB + ((pc ^ (prow >> 1)) << 4), ldsO = prow * RSB + ((pc ^ ((prow >> 1) + 4)) << 4);
  // tile rows t0 .. t0+8*n-1 of `src` into LDS rows l0 ..
  auto load_rows = [&](const uint16_t* src, int t0, int l0, int n) __attribute__((always_inline)) {
    const uint8_t* sb = reinterpret_cast<const uint8_t*>(src + (int64_t)(rbase + t0) * ld + cbase);       // wave-uniform
#pragma unroll
    for (int it = 0; it < 8; it++) {
      if (it < n) {
        const uint8_t* p = sb + (int64_t)it * 16 * ld + (((l0 >> 3) + it) & 1 ? gO : gE);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)p,
                                         (EMI_LDS void*)(wl + (l0 + 8 * it) * RSB), 16, 0, 0);
      }
    }
  };
  // LDS rows l0 .. l0+8*n-1 to tile rows t0 .. of `dst`
  auto store_rows = [&](uint16_t* dst, int t0, int l0, int n) __attribute__((always_inline)) {
    uint8_t* db = reinterpret_cast<uint8_t*>(dst + (int64_t)(rbase + t0) * ld + cbase);                    // wave-uniform
#pragma unroll
    for (int it = 0; it < 16; it++) {
      if (it < n) {
        const u32x4_t v = *reinterpret_cast<const EMI_LDS u32x4_t*>(wl + (l0 + 8 * it) * RSB + ((((l0 >> 3) + it) & 1) ? ldsO : ldsE));
        *reinterpret_cast<u32x4_t*>(db + (int64_t)it * 16 * ld + gC) = v;
      }
    }
  };
  auto unpack = [](const u32x2_t w, float (&f)[4]) {
    f[0] = __uint_as_float(w[0] << 16);
    f[1] = __uint_as_float(w[0] & 0xffff0000u);
    f[2] = __uint_as_float(w[1] << 16);
    f[3] = __uint_as_float(w[1] & 0xffff0000u);
  };
  if constexpr (MODE == 1) {
    load_rows(P0, 0, 0, 8);
    load_rows(P0, 64, 64, 8);
    wait_vmcnt<0>();
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        EMI_LDS u32x2_t* slot = reinterpret_cast<EMI_LDS u32x2_t*>(wl + quad_slot(i * 16 + lrow, j));
        float a[4], b[4];
        unpack(*slot, a);
        u32x2_t bq;
        bq[0] = pack_bf16x2(acc[i][j][0], acc[i][j][1]);
        bq[1] = pack_bf16x2(acc[i][j][2], acc[i][j][3]);
        unpack(bq, b);
        *slot = bq;                               // b takes a's place in the slice; g stays in the registers
#pragma unroll
        for (int e = 0; e < 4; e++) acc[i][j][e] = emi_swiglu(a[e], b[e]);
      }
    store_rows(Q0, 0, 0, 16);
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        u32x2_t w;
        w[0] = pack_bf16x2(acc[i][j][0], acc[i][j][1]);
        w[1] = pack_bf16x2(acc[i][j][2], acc[i][j][3]);
        *reinterpret_cast<EMI_LDS u32x2_t*>(wl + quad_slot(i * 16 + lrow, j)) = w;
      }
    store_rows(Q1, 0, 0, 16);
  } else {
    // two passes over 64 tile rows: a in LDS rows 0..63, b in LDS rows 64..127
#pragma unroll
    for (int p = 0; p < 2; p++) {
      if (p) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // the first pass has read its rows out of the slice
      load_rows(P0, 64 * p, 0, 8);
      load_rows(P1, 64 * p, 64, 8);
      wait_vmcnt<0>();
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          EMI_LDS u32x2_t* sa = reinterpret_cast<EMI_LDS u32x2_t*>(wl + quad_slot(i * 16 + lrow, j));
          EMI_LDS u32x2_t* sb = reinterpret_cast<EMI_LDS u32x2_t*>(wl + quad_slot(64 + i * 16 + lrow, j));
          float a[4], b[4], g[4], da[4], db[4];
          unpack(*sa, a);
          unpack(*sb, b);
          u32x2_t gq;
          gq[0] = pack_bf16x2(acc[4 * p + i][j][0], acc[4 * p + i][j][1]);
          gq[1] = pack_bf16x2(acc[4 * p + i][j][2], acc[4 * p + i][j][3]);
          unpack(gq, g);
#pragma unroll
          for (int e = 0; e < 4; e++) emi_swiglu_adjoint(a[e], b[e], g[e], &da[e], &db[e]);
          u32x2_t wa, wb;
          wa[0] = pack_bf16x2(da[0], da[1]);
          wa[1] = pack_bf16x2(da[2], da[3]);
          wb[0] = pack_bf16x2(db[0], db[1]);
          wb[1] = pack_bf16x2(db[2], db[3]);
          *sa = wa;
          *sb = wb;
        }
      store_rows(Q0, 64 * p, 0, 8);
      store_rows(Q1, 64 * p, 64, 8);
    }
  }
}

// ---------------------------------------------------------------------------
// Ping-pong kernel for two k-contiguous operands (the NT layout): 256x256x64 block
// tile, 8 wavefronts = two groups of four, one wavefront of each group per SIMD.
// A tile step is cut into four slots separated by s_barrier; a wavefront
// alternates memory slots (LDS -> register fragment reads, HBM -> LDS loads) and
// compute slots (16 MFMAs), and the two groups run one slot apart, so on every SIMD
// one wavefront always feeds the matrix core while the other one moves data.
//
// Each operand tile is held as two 128-row regions per LDS stage.  A wavefront's
// 128x64 output tile is four 64x32 quadrants; a region is read into registers once
// per tile step (for the whole BK) and is therefore free to be refilled two tile
// steps ahead as soon as both groups have read it:
//   region A_h : block rows  wm*128 + h*64 + [0,64)   for wm = 0,1
//   region B_j : block cols  wn*64  + j*32 + [0,32)   for wn = 0..3
//   slot  Ma: read B_0, B_1, A_0; refill B_1, A_1 of the other stage (tile t+1)
//         Ca: quadrants (0,0), (0,1)
//         Mb: read A_1; refill A_0, B_0 (tile t+2)         Cb: quadrants (1,0), (1,1)
// A region written by loads issued in local slot L was last read in local slot
// <= L-2 by both groups; a wavefront waits for its own loads (vmcnt) two local
// slots before the first read of that region by either group.
// ---------------------------------------------------------------------------
// Transposing LDS read through inline asm with an immediate offset: the compiler
// orders every LDS read it knows of behind all outstanding direct-to-LDS loads,
// which would serialise loading and compute.  The result is valid after the next
// lds_tr_fence() over it.
template <int OFF> __device__ __forceinline__ u32x2_t lds_tr_read(uint32_t addr) {
  static_assert(OFF >= 0 && OFF < 65536, "ds offset field");
  u32x2_t r;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
  return r;
}
// Waits for all LDS reads of this wavefront; the values passed in cannot be used
// (or copied) by the compiler before the wait.
__device__ __forceinline__ void lds_tr_fence(u32x2_t (&t)[4][2][2]) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(t[0][0][0]), "+v"(t[0][0][1]), "+v"(t[0][1][0]), "+v"(t[0][1][1]), "+v"(t[1][0][0]), "+v"(t[1][0][1]),
                 "+v"(t[1][1][0]), "+v"(t[1][1][1]));
  asm volatile(""
               : "+v"(t[2][0][0]), "+v"(t[2][0][1]), "+v"(t[2][1][0]), "+v"(t[2][1][1]), "+v"(t[3][0][0]), "+v"(t[3][0][1]),
                 "+v"(t[3][1][0]), "+v"(t[3][1][1]));
}
template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F> __device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// AKM / BKM: the operand is stored k-major (A as [K][M], B as [K][N]) instead of
// k-contiguous (A as [M][K], B as [N][K]).  A k-major region holds [64 k][128 c]
// (256-byte rows), chunk ch of k-row k at ch ^ 4(k&3) ^ 2((k>>3)&1).  For A, c runs over
// the same block rows as the 128 rows of a k-contiguous region (two runs of 64; one run of
// 128 measured slower).  For B, region B_j is the contiguous block columns 128j + [0,128)
// and a wavefront owns the two 32-column strips 128j + 32*wn + [0,32) of C, so that every
// k-row of a region is one 256-byte run in memory.  A k-major region is
// read with two transposing loads per fragment: the 32 lanes that are served
// together address k-rows {0..3} and {8..11} (+4 for the second load), 32 bytes
// each, which the swizzle spreads over all 64 banks.
// GROUPED: the grid holds the tiles of grp.count independent products of one shape, product-major (GemmGroup with
// sum == 0); otherwise the last argument is an empty placeholder.
// EPI: 0 = the result [+ R]; 1 / 2 = the SwiGLU epilogues (epilogue_swiglu_t16; R is P0, C is Q0, plus P1 and Q1);
// 3 = the result [+ R] with RoPE applied to it (epilogue_bf16_t16<..., ROPE>); 4 = as 0 for matrices of whole tiles and
// 16-byte accesses (the launcher checks): without the code for ragged tiles the kernel needs no scratch memory;
// 5 = split-K: the grid holds tiles x splits blocks, split-major; split z owns k in [z * k_per_split, ...) and leaves its
// fp32 tile in part[z][M][N] for gemm_splitk_reduce_kernel (k-contiguous operands only).
struct NoEpi {};
struct SplitEpi {
  float* part;
  int k_per_split;
};
struct SwigluEpi {
  const uint16_t* P1;
  uint16_t* Q1;
};
struct RopeEpi {
  const float* table;      // [seq, head_dim / 2] of (cos, sin)
  int seq, head_dim;
};
template <int EPI> struct EpiArg { using type = NoEpi; };
template <> struct EpiArg<1> { using type = SwigluEpi; };
template <> struct EpiArg<2> { using type = SwigluEpi; };
template <> struct EpiArg<3> { using type = RopeEpi; };
template <> struct EpiArg<5> { using type = SplitEpi; };
template <bool AKM, bool BKM, bool GROUPED = false, int EPI = 0>
__global__ __launch_bounds__(512) void gemm_bf16_pingpong_kernel(const uint16_t* __restrict__ A,
                                                                  const uint16_t* __restrict__ B, const uint16_t* R,
                                                                  uint16_t* C, int M, int N, int K, int lda, int ldb,
                                                                  int ldr, int ldc, uint32_t a_bytes, uint32_t b_bytes,
                                                                  int vec_ok,
                                                                  std::conditional_t<GROUPED, GemmGroup, NoGroup> grp,
                                                                  typename EpiArg<EPI>::type epi = {}) {
  constexpr int BM = 256, BN = 256, BK = 64;
  constexpr int REGION = 128 * BK * 2;                          // 16 KiB
  // LDS map: A_h of stage s at (2s + h) regions, B_j of stage s at 64 KiB + (2s + j) regions, so that
  // every offset from a lane's A (or B) base address fits the 16-bit offset field of an LDS read.
  constexpr int B_BASE = 4 * REGION;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[];
  EMI_LDS uint8_t* smem = (EMI_LDS uint8_t*)smem_raw;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave >> 2, wn = wave & 3;

  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  int tile_m, tile_n;
  [[maybe_unused]] int split = 0;
  if constexpr (GROUPED) {
    const int pid = xcd_contiguous_id(), tiles = tiles_m * tiles_n;
    const int prod = pid / tiles;
    tile_coords(pid - prod * tiles, tiles_m, tiles_n, &tile_m, &tile_n);
    A = grp.A[prod];
    B = grp.B[prod];
    R = grp.R[prod];
    C = grp.C[prod];
  } else if constexpr (EPI == 5) {
    static_assert(!AKM && !BKM, "split-K serves the k-contiguous layout");
    const int pid = xcd_contiguous_id(), tiles = tiles_m * tiles_n;
    split = pid / tiles;
    tile_coords(pid - split * tiles, tiles_m, tiles_n, &tile_m, &tile_n);
    const int k_lo = split * epi.k_per_split;                      // < K: the launcher sizes the grid
    A += k_lo;
    B += k_lo;
    a_bytes -= (uint32_t)k_lo * 2u;
    b_bytes -= (uint32_t)k_lo * 2u;
    K = K - k_lo < epi.k_per_split ? K - k_lo : epi.k_per_split;
  } else {
    // With a long contraction and k-contiguous operands, groups of 4 tile-rows measured 3 % faster than 8
    // ([16384, 11008] x [4096, 11008]^T: 975 vs 1005 us): an XCD then re-reads the (cache-resident) weight panels
    // more often and the activation panels, which come from HBM, less often.
    if (!AKM && !BKM && K >= 8192) tile_coords<4>(xcd_contiguous_id(), tiles_m, tiles_n, &tile_m, &tile_n);
    else tile_coords(xcd_contiguous_id(), tiles_m, tiles_n, &tile_m, &tile_n);
  }
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const __amdgpu_buffer_rsrc_t rA = make_rsrc(A, a_bytes);
  const __amdgpu_buffer_rsrc_t rB = make_rsrc(B, b_bytes);

  // HBM -> LDS: a region is 16 wave-loads of 1 KiB; wavefront w issues loads w and w+8 of
  // every region.  k-contiguous: a wave-load is 8 rows x 128 bytes, lane l fills physical
  // chunk (l & 7) of region row 8q + (l >> 3).  k-major: 4 k-rows x 256 bytes, lane l fills
  // physical chunk (l & 15) of k-row 4q + (l >> 4).  Either way the lane fetches the logical
  // chunk that the swizzle maps to its slot.  lk: the k index (within the tile) of the chunk.
  uint32_t voffA[2][2], voffB[2][2];
  int lkA[2], lkB[2];
  const int lck = ((lane & 7) ^ (((lane >> 4) + 4 * (wave & 1)) & 7)) * 8;     // k-contiguous: k offset of the chunk
#pragma unroll
  for (int it = 0; it < 2; it++) {
    const int q = it * 8 + wave;
    const int rho = q * 8 + (lane >> 3);                                       // k-contiguous: region row
    const int km = q * 4 + (lane >> 4);                                        // k-major: k-row
    const int cm = ((lane & 15) ^ (4 * (km & 3)) ^ (2 * ((km >> 3) & 1))) * 8; // k-major: first of 8 columns
    lkA[it] = AKM ? km : lck;
    lkB[it] = BKM ? km : lck;
#pragma unroll
    for (int h = 0; h < 2; h++) {
      if constexpr (AKM) {
        const int grow = m0 + (cm >> 6) * 128 + h * 64 + (cm & 63);
        voffA[h][it] = grow < M ? ((uint32_t)km * (uint32_t)lda + (uint32_t)grow) * 2u : kOob;
      } else {
        const int grow = m0 + (rho >> 6) * 128 + h * 64 + (rho & 63);
        voffA[h][it] = grow < M ? ((uint32_t)grow * (uint32_t)lda + (uint32_t)lck) * 2u : kOob;
      }
      if constexpr (BKM) {
        const int gcol = n0 + h * 128 + cm;
        voffB[h][it] = gcol < N ? ((uint32_t)km * (uint32_t)ldb + (uint32_t)gcol) * 2u : kOob;
      } else {
        const int gcol = n0 + (rho >> 5) * 64 + h * 32 + (rho & 31);
        voffB[h][it] = gcol < N ? ((uint32_t)gcol * (uint32_t)ldb + (uint32_t)lck) * 2u : kOob;
      }
    }
  }
  const uint32_t kbytesA = AKM ? (uint32_t)lda * 2u : 2u, kbytesB = BKM ? (uint32_t)ldb * 2u : 2u;   // bytes per step in k
  auto refillA = [&](int h, int lds_off, int it, int k0) __attribute__((always_inline)) {
    const uint32_t v = (k0 + lkA[it] < K) ? voffA[h][it] + (uint32_t)k0 * kbytesA : kOob;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rA, smem + lds_off + (it * 8 + wave) * 1024, 16, v, 0, 0, 0);
  };
  auto refillB = [&](int j, int lds_off, int it, int k0) __attribute__((always_inline)) {
    const uint32_t v = (k0 + lkB[it] < K) ? voffB[j][it] + (uint32_t)k0 * kbytesB : kOob;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rB, smem + lds_off + (it * 8 + wave) * 1024, 16, v, 0, 0, 0);
  };

  // LDS -> registers.  Fragment of v_mfma_f32_16x16x32_bf16 (16 rows x 32 k): lane l holds
  // row (l & 15), k = 8*(l >> 4) .. +7 of k-step ks.
  // k-contiguous: one 16-byte read of logical chunk 4*ks + (l >> 4).
  const int l15 = lane & 15, sw = l15 >> 1, kq4 = lane >> 4;
  const int a_lane = (wm * 64 + l15) * (BK * 2);
  const int b_lane = B_BASE + (wn * 32 + l15) * (BK * 2);
  auto frag = [&](int base, int ks) __attribute__((always_inline)) {
    return *reinterpret_cast<const EMI_LDS bf16x8_t*>(smem + base + (((ks * 4 + kq4) ^ sw) << 4));
  };
  // k-major: two transposing reads; within 16 lanes, lane i addresses k-row (i >> 2), columns
  // 4*(i & 3).. +3 and receives column i, k-rows 0..3.  tadrA[blk] / tadrB[blk]: LDS address of
  // this lane's 8 bytes for 16-row block blk, k-step 0, first read, region 0.
  uint32_t tadrA[4], tadrB[2];
  {
    const int kq = l15 >> 2, g = lane >> 4, x = (l15 & 3) >> 1;
    const int t = x ^ (4 * kq) ^ (2 * (g & 1));
    const uint32_t lane_part = (uint32_t)(uintptr_t)smem + (uint32_t)((8 * g + kq) * 256 + (l15 & 1) * 8);
#pragma unroll
    for (int blk = 0; blk < 4; blk++) tadrA[blk] = lane_part + (uint32_t)(((wm * 8 + blk * 2) ^ t) << 4);
#pragma unroll
    for (int blk = 0; blk < 2; blk++) tadrB[blk] = lane_part + (uint32_t)B_BASE + (uint32_t)(((wn * 4 + blk * 2) ^ t) << 4);
  }

  // acc[i][j]: 16x16 tile at wave rows 16*i, wave columns 16*j (i = 4*h + row block)
  f32x4_t acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int r = 0; r < 4; r++) acc[i][j][r] = 0.f;

  bf16x8_t fa[4][2], fb[4][2];               // [16-row block][k-step]; fb: 0,1 = B_0, 2,3 = B_1
  u32x2_t ta[4][2][2], tb[4][2][2];          // halves of k-major fragments in flight
  auto join = [&](const u32x2_t (&t)[2]) __attribute__((always_inline)) {
    const u32x4_t w = {t[0][0], t[0][1], t[1][0], t[1][1]};
    return __builtin_bit_cast(bf16x8_t, w);
  };
  auto slot_end = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  // Compute slot: the 64 x 64 half of the wave tile that uses row half h (32 MFMAs).
  // The operands are passed swapped so that a lane owns 4 consecutive C columns.
  auto half_rows = [&](int h) __attribute__((always_inline)) {
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
      for (int j = 0; j < 4; j++)
#pragma unroll
        for (int i = 0; i < 4; i++)
          acc[h * 4 + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[j][ks], fa[i][ks], acc[h * 4 + i][j], 0, 0, 0);
    __builtin_amdgcn_s_setprio(0);
    slot_end();
  };
  // Read 16-row block blk (0..3) of region A_h / block blk (0..1) of region B_j of stage S, k-step ks.
  auto readA = [&](auto S, auto h, auto blk, auto ks) __attribute__((always_inline)) {
    constexpr int off = (2 * decltype(S)::value + decltype(h)::value) * REGION;
    constexpr int b = decltype(blk)::value, k = decltype(ks)::value;
    if constexpr (AKM) {
      ta[b][k][0] = lds_tr_read<off + k * 32 * 256>(tadrA[b]);
      ta[b][k][1] = lds_tr_read<off + k * 32 * 256 + 4 * 256>(tadrA[b]);
    } else {
      fa[b][k] = frag(off + a_lane + b * 16 * BK * 2, k);
    }
  };
  auto readB = [&](auto S, auto j, auto blk, auto ks) __attribute__((always_inline)) {
    constexpr int off = (2 * decltype(S)::value + decltype(j)::value) * REGION;
    constexpr int b = decltype(blk)::value, k = decltype(ks)::value, f = 2 * decltype(j)::value + b;
    if constexpr (BKM) {
      tb[f][k][0] = lds_tr_read<off + k * 32 * 256>(tadrB[b]);
      tb[f][k][1] = lds_tr_read<off + k * 32 * 256 + 4 * 256>(tadrB[b]);
    } else {
      fb[f][k] = frag(off + b_lane + b * 16 * BK * 2, k);
    }
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  auto tile_step = [&](auto S, int t) __attribute__((always_inline)) {
    constexpr int s = decltype(S)::value, o = s ^ 1;
    constexpr int offA0 = (2 * s) * REGION, offB0 = B_BASE + (2 * s) * REGION;                     // this stage
    constexpr int offA1o = (2 * o + 1) * REGION, offB1o = B_BASE + (2 * o + 1) * REGION;           // other stage
    // Ma: read B_0, A_0, B_1 of this stage; refill B_1, A_1 of the other stage (tile t+1).
    // Loads and reads alternate so that the texture path and the LDS work in parallel.
    static_for<4>([&](auto qc) __attribute__((always_inline)) {
      constexpr int q = decltype(qc)::value;
      if constexpr (q < 2) refillB(1, offB1o, q, (t + 1) * BK);
      else refillA(1, offA1o, q - 2, (t + 1) * BK);
      using KS = std::integral_constant<int, (q >> 1)>;
      using BL = std::integral_constant<int, (q & 1)>;
      using BA0 = std::integral_constant<int, 2 * (q & 1)>;
      using BA1 = std::integral_constant<int, 2 * (q & 1) + 1>;
      readB(S, I0{}, BL{}, KS{});
      readA(S, I0{}, BA0{}, KS{});
      readA(S, I0{}, BA1{}, KS{});
      readB(S, I1{}, BL{}, KS{});
    });
    if constexpr (AKM) lds_tr_fence(ta);
    if constexpr (BKM) lds_tr_fence(tb);
    if constexpr (AKM) {
#pragma unroll
      for (int b = 0; b < 4; b++)
#pragma unroll
        for (int k = 0; k < 2; k++) fa[b][k] = join(ta[b][k]);
    }
    if constexpr (BKM) {
#pragma unroll
      for (int b = 0; b < 4; b++)
#pragma unroll
        for (int k = 0; k < 2; k++) fb[b][k] = join(tb[b][k]);
    }
    wait_vmcnt<8>();                        // own part of A_1 of this tile has landed
    slot_end();
    half_rows(0);                           // Ca
    // Mb: read A_1; refill A_0, B_0 of this stage (tile t+2)
    static_for<4>([&](auto qc) __attribute__((always_inline)) {
      constexpr int q = decltype(qc)::value;
      if constexpr (q < 2) refillA(0, offA0, q, (t + 2) * BK);
      else refillB(0, offB0, q - 2, (t + 2) * BK);
      using KS = std::integral_constant<int, (q >> 1)>;
      using BA0 = std::integral_constant<int, 2 * (q & 1)>;
      using BA1 = std::integral_constant<int, 2 * (q & 1) + 1>;
      readA(S, I1{}, BA0{}, KS{});
      readA(S, I1{}, BA1{}, KS{});
    });
    if constexpr (AKM) {
      lds_tr_fence(ta);
#pragma unroll
      for (int b = 0; b < 4; b++)
#pragma unroll
        for (int k = 0; k < 2; k++) fa[b][k] = join(ta[b][k]);
    }
    wait_vmcnt<6>();                        // own part of A_0, B_0 and of B_1 of the next tile
    slot_end();
    half_rows(1);                           // Cb
  };

  // Prologue: tile 0 into stage 0; A_0, B_0 of tile 1 into stage 1 (its A_1, B_1 are
  // issued by the first memory slot).
#pragma unroll
  for (int it = 0; it < 2; it++) {
    refillA(0, 0, it, 0);
    refillB(0, B_BASE, it, 0);
    refillB(1, B_BASE + REGION, it, 0);
    refillA(1, REGION, it, 0);
    refillA(0, 2 * REGION, it, BK);
    refillB(0, B_BASE + 2 * REGION, it, BK);
  }
  wait_vmcnt<0>();
  slot_end();
  if (wm == 1) slot_end();                  // second group runs one slot behind the first

  const int nk = (K + BK - 1) / BK;
  int t = 0;
  for (; t + 1 < nk; t += 2) {
    tile_step(I0{}, t);
    tile_step(I1{}, t + 1);
  }
  if (t < nk) tile_step(I0{}, t);

  if (wm == 0) slot_end();
  wait_vmcnt<0>();                          // zero-filled loads past the end of K
  slot_end();

  if constexpr (EPI == 5) {
    // accumulator layout (swapped operands): register r of lane l holds row l % 16, column 4 * (l / 16) + r of its 16x16
    // tile.  Each wavefront stages 32 rows x 64 columns of fp32 at a time through its own slice of the idle LDS (rows 16
    // bytes further apart than their 256) and writes them as whole 256-byte rows, four per store instruction.
    constexpr int RS = 64 * 4 + 16;
    EMI_LDS uint8_t* wl = smem + wave * (32 * RS);
    float* pz = epi.part + (int64_t)split * M * N;
    const bool vec4 = (N & 3) == 0;
    const int lr = lane & 15, lg = lane >> 4;
#pragma unroll
    for (int p = 0; p < 4; p++) {
#pragma unroll
      for (int ii = 0; ii < 2; ii++)
#pragma unroll
        for (int j = 0; j < 4; j++)
          *reinterpret_cast<EMI_LDS f32x4_t*>(wl + (16 * ii + lr) * RS + (16 * j + 4 * lg) * 4) = acc[2 * p + ii][j];
#pragma unroll
      for (int it = 0; it < 8; it++) {
        const int row = it * 4 + lg, c = lr * 4;
        const f32x4_t v = *reinterpret_cast<const EMI_LDS f32x4_t*>(wl + row * RS + c * 4);
        const int grow = m0 + wm * 128 + 32 * p + row, gcol = n0 + wn * 64 + c;
        if (grow < M && gcol < N) {
          float* dst = pz + (int64_t)grow * N + gcol;
          if (vec4) {
            *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
          } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
              if (gcol + e < N) dst[e] = v[e];
          }
        }
      }
    }
  } else if constexpr (EPI == 3) {
    static_assert(!AKM && !BKM && !GROUPED, "the RoPE epilogue belongs to the k-contiguous single product");
    epilogue_bf16_t16<8, 4, 0, true>(acc, smem, wave, lane, m0 + wm * 128, n0 + wn * 64, R, C, M, N, ldr, ldc, vec_ok, epi.table,
                                     epi.seq, epi.head_dim);
  } else if constexpr (EPI == 4) {
    epilogue_bf16_t16<8, 4, (BKM ? 96 : 0), false, true>(acc, smem, wave, lane, m0 + wm * 128, n0 + wn * (BKM ? 32 : 64), R, C, M, N,
                                                         ldr, ldc, vec_ok);
  } else if constexpr (EPI != 0) {
    static_assert(!AKM && !BKM && !GROUPED, "the SwiGLU epilogues belong to the k-contiguous single product");
    epilogue_swiglu_t16<EPI>(acc, smem, wave, lane, m0 + wm * 128, n0 + wn * 64, R, epi.P1, C, epi.Q1, ldc);
  } else {
    epilogue_bf16_t16<8, 4, (BKM ? 96 : 0)>(acc, smem, wave, lane, m0 + wm * 128, n0 + wn * (BKM ? 32 : 64), R, C, M, N, ldr,
                                            ldc, vec_ok);
  }
}

// ---------------------------------------------------------------------------
// Generic path: any dtype/shape/alignment, fp32 MFMA (v_mfma_f32_32x32x2_f32).
// 256 threads, LDS tiles stored k-major as fp32.  These problems are small, so a block's time is
// the number of K-steps times the latency of one step: the steps are deep (64 for the 64x64 tile,
// 32 for 128x128) and the next step's elements are loaded into registers while the matrix cores
// work on the current one.
// ---------------------------------------------------------------------------
// WT: 32x32 MFMA tiles per wavefront and dimension: 2 -> 128x128 block tiles, 1 -> 64x64 (small problems: more
// blocks, shorter iterations).
template <typename T, int WT>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const T* __restrict__ A, const T* __restrict__ B, const T* R,
                                                           T* C, int M, int N, int K, int64_t lda, int64_t ldb,
                                                           int64_t ldr, int64_t ldc, int trans_a, int trans_b,
                                                           float* __restrict__ part, int k_per_split) {
  constexpr int BM = 64 * WT, BN = 64 * WT, BK = 128 / (WT * WT > 1 ? 4 : 2), PAD = 1;
  constexpr int NA = BM * BK / 256, NB = BN * BK / 256;      // elements per thread and step
  __shared__ float sA[BK][BM + PAD];
  __shared__ float sB[BK][BN + PAD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  f32x16_t acc[WT][WT];
#pragma unroll
  for (int i = 0; i < WT; i++)
#pragma unroll
    for (int j = 0; j < WT; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // split-K (part != nullptr): block z owns k in [z * k_per_split, ...) and writes an fp32 partial
  // tile to part[z][M][N]; a second kernel adds the partials (and R) in fixed order
  const int k_lo = part ? blockIdx.z * k_per_split : 0;
  const int k_hi = part ? (k_lo + k_per_split < K ? k_lo + k_per_split : K) : K;
  K = k_hi;
  // element `it` of this thread in a tile: (m, k) for A, (n, k) for B; the fast index follows memory
  auto a_mk = [&](int it, int& m, int& k) {
    if (trans_a) { m = tid & (BM - 1); k = tid / BM + it * (256 / BM); }     // A is [K,M]: m contiguous
    else { k = tid & (BK - 1); m = tid / BK + it * (256 / BK); }             // A is [M,K]: k contiguous
  };
  auto b_nk = [&](int it, int& n, int& k) {
    if (trans_b) { k = tid & (BK - 1); n = tid / BK + it * (256 / BK); }     // B is [N,K]
    else { n = tid & (BN - 1); k = tid / BN + it * (256 / BN); }             // B is [K,N]
  };
  float ra[NA], rb[NB];
  auto load_step = [&](int k0) {
#pragma unroll
    for (int it = 0; it < NA; it++) {
      int m, k;
      a_mk(it, m, k);
      ra[it] = (m0 + m < M && k0 + k < K)
                   ? to_f32(trans_a ? A[(int64_t)(k0 + k) * lda + m0 + m] : A[(int64_t)(m0 + m) * lda + k0 + k]) : 0.f;
    }
#pragma unroll
    for (int it = 0; it < NB; it++) {
      int n, k;
      b_nk(it, n, k);
      rb[it] = (n0 + n < N && k0 + k < K)
                   ? to_f32(trans_b ? B[(int64_t)(n0 + n) * ldb + k0 + k] : B[(int64_t)(k0 + k) * ldb + n0 + n]) : 0.f;
    }
  };
  if (k_lo < K) load_step(k_lo);
  for (int k0 = k_lo; k0 < K; k0 += BK) {
#pragma unroll
    for (int it = 0; it < NA; it++) {
      int m, k;
      a_mk(it, m, k);
      sA[k][m] = ra[it];
    }
#pragma unroll
    for (int it = 0; it < NB; it++) {
      int n, k;
      b_nk(it, n, k);
      sB[k][n] = rb[it];
    }
    __syncthreads();
    if (k0 + BK < K) load_step(k0 + BK);           // in flight while this step is multiplied
#pragma unroll
    for (int kk = 0; kk < BK; kk += 2) {
      const int k = kk + (lane >> 5);
      float a[WT], b[WT];
#pragma unroll
      for (int i = 0; i < WT; i++) a[i] = sA[k][wm * 32 * WT + i * 32 + (lane & 31)];
#pragma unroll
      for (int j = 0; j < WT; j++) b[j] = sB[k][wn * 32 * WT + j * 32 + (lane & 31)];
#pragma unroll
      for (int i = 0; i < WT; i++)
#pragma unroll
        for (int j = 0; j < WT; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }
  const int col_l = lane & 31, row_l = (lane >> 5) * 4;
#pragma unroll
  for (int i = 0; i < WT; i++)
#pragma unroll
    for (int j = 0; j < WT; j++) {
      const int col = n0 + wn * 32 * WT + j * 32 + col_l;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int row = m0 + wm * 32 * WT + i * 32 + (r >> 2) * 8 + row_l + (r & 3);
        if (row < M && col < N) {
          float v = acc[i][j][r];
          if (part != nullptr) {
            part[((int64_t)blockIdx.z * M + row) * N + col] = v;
          } else {
            if (R != nullptr) v += to_f32(R[(int64_t)row * ldr + col]);
            C[(int64_t)row * ldc + col] = from_f32<T>(v);
          }
        }
      }
    }
}

// ---------------------------------------------------------------------------
// fp32 products on aligned operands.  The 15M-parameter model's projections are 256 x 288 x 288: few tiles, and a
// block's time is its serial chain of K-steps, so the work is cut fine: a block owns a 32x32 tile of C and its four wavefronts each take a quarter
// of K, reading their operand fragments straight from global memory in the v_mfma_f32_32x32x2_f32 layout (lane l
// supplies A[l % 32][l / 32] and B[l / 32][l % 32]).  The contraction index of an instruction is the lane half
// g = l / 32; instruction t of an 8-wide chunk contracts k = k0 + 4 g + t, so a k-contiguous operand is read in
// 16-byte pieces and a k-major one in 128-byte rows.  The four partial tiles are added in wavefront order through
// LDS (fixed order: run-to-run identical bits).
// ---------------------------------------------------------------------------
// GROUPED: blockIdx.z picks one of grp.count independent products of one shape (GemmGroup with sum == 0, its pointers
// read as float).
// NW wavefronts share K; U 8-wide chunks are in flight per step.  ONCE: a wavefront's share of K is at most U chunks
// (K <= 96 NW), so everything is requested up front and the block waits for memory once: a short contraction is a
// chain of load latencies otherwise (256 x 288 x 288: 10 us in three steps).
template <bool A_KMAJOR, bool B_KMAJOR, bool GROUPED = false, int NW = 4, int U = 4, bool ONCE = false>
__global__ __launch_bounds__(NW * 64) void gemm_f32_small_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                                 const float* R, float* C, int M, int N, int K, int64_t lda,
                                                                 int64_t ldb, int64_t ldr, int64_t ldc,
                                                                 std::conditional_t<GROUPED, GemmGroup, NoGroup> grp,
                                                                 float* __restrict__ part = nullptr, int kps = 0) {
  __shared__ float red[NW - 1][16][64];
  if constexpr (GROUPED) {
    A = reinterpret_cast<const float*>(grp.A[blockIdx.z]);
    B = reinterpret_cast<const float*>(grp.B[blockIdx.z]);
    R = reinterpret_cast<const float*>(grp.R[blockIdx.z]);
    C = reinterpret_cast<float*>(grp.C[blockIdx.z]);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i = lane & 31, g = lane >> 5;
  const int m0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
  const int mi = m0 + i < M ? m0 + i : M - 1, ni = n0 + i < N ? n0 + i : N - 1;      // clamped: those results are not stored
  // split-K (part != nullptr, not GROUPED): plane blockIdx.z takes kps (a multiple of 8 NW) of K and leaves its
  // 32 x 32 partial in part[z][M][N] for gemm_splitk_reduce_kernel
  const int kb = part != nullptr ? (int)blockIdx.z * kps : 0;
  const int kend = part != nullptr && kb + kps < K ? kb + kps : K;
  const int kper = ((kend - kb + 8 * NW - 1) / (8 * NW)) * 8;    // this wavefront's share of K, rounded up to whole chunks
  const int ks = kb + wave * kper, ke = ks + kper < kend ? ks + kper : kend;
  const float* pa = A_KMAJOR ? A + mi : A + (int64_t)mi * lda;
  const float* pb = B_KMAJOR ? B + ni : B + (int64_t)ni * ldb;
  // elements k0 + 4 g + t, t = 0..3, of this lane's row (column) of an operand; zero past the wavefront's share of K
  auto frag = [&](const float* p, int64_t ld, bool kmajor, int k0, float (&f)[4]) {
    const int k = k0 + 4 * g;
    if (!kmajor) {
      if (k + 4 <= ke) {
        const float4 x = *reinterpret_cast<const float4*>(p + k);
        f[0] = x.x; f[1] = x.y; f[2] = x.z; f[3] = x.w;
      } else {
#pragma unroll
        for (int t = 0; t < 4; t++) f[t] = k + t < ke ? p[k + t] : 0.f;
      }
    } else {
#pragma unroll
      for (int t = 0; t < 4; t++) f[t] = k + t < ke ? p[(int64_t)(k + t) * ld] : 0.f;
    }
  };
  f32x16_t acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
  float a[U][4], b[U][4];
  auto load = [&](int k0, float (&fa)[U][4], float (&fb)[U][4]) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      frag(pa, lda, A_KMAJOR, k0 + 8 * u, fa[u]);
      frag(pb, ldb, B_KMAJOR, k0 + 8 * u, fb[u]);
    }
  };
  if (ks < ke) load(ks, a, b);
  if constexpr (ONCE) {
    if (ks < ke) {
#pragma unroll
      for (int u = 0; u < U; u++)
#pragma unroll
        for (int t = 0; t < 4; t++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][t], b[u][t], acc, 0, 0, 0);
    }
  } else {
    float an[U][4], bn[U][4];
    for (int k0 = ks; k0 < ke; k0 += 8 * U) {
      const bool more = k0 + 8 * U < ke;
      if (more) load(k0 + 8 * U, an, bn);            // in flight while this step is multiplied
#pragma unroll
      for (int u = 0; u < U; u++)
#pragma unroll
        for (int t = 0; t < 4; t++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][t], b[u][t], acc, 0, 0, 0);
      if (more) {
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
          for (int t = 0; t < 4; t++) { a[u][t] = an[u][t]; b[u][t] = bn[u][t]; }
      }
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int r = 0; r < 16; r++) red[wave - 1][r][lane] = acc[r];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int w = 0; w < NW - 1; w++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] += red[w][r][lane];
  // register r of lane l: row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32
  const int col = n0 + i;
#pragma unroll
  for (int r = 0; r < 16; r++) {
    const int row = m0 + (r >> 2) * 8 + g * 4 + (r & 3);
    if (row < M && col < N) {
      float v = acc[r];
      if (part != nullptr) {
        part[((int64_t)blockIdx.z * M + row) * N + col] = v;
      } else {
        if (R != nullptr) v += R[(int64_t)row * ldr + col];
        C[(int64_t)row * ldc + col] = v;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// fp32 products that fill the chip with 128 x 128 tiles (the logits and their adjoints: 256 x 32000 x 288 and its
// two transposes): the same matrix instruction fed from LDS.  The K-split kernel above has every 32 x 32 tile read
// its own 64 operand rows from the L2 (8 flop per byte), which bounds it at 35-55 TFLOP/s.  Here a block of four
// wavefronts (2 x 2, 64 x 64 each = four 32 x 32 accumulators) stages 128 x 32 pieces of both operands per step:
// a k-contiguous operand as [row][32 + 4] (a lane reads its 4 consecutive k as one 16-byte piece), a k-major one as
// [k][128] (four 4-byte reads, lanes along the rows).  Global loads of step s+1 are in flight while step s is
// multiplied (held in registers, written to LDS between two barriers).  part / kps as in the kernel above (planes of K).
// Needs 16-byte aligned bases and leading dimensions that are multiples of 4.
// ---------------------------------------------------------------------------
template <bool A_KMAJOR, bool B_KMAJOR>
__global__ __launch_bounds__(256) void gemm_f32_tiled_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                             const float* R, float* C, int M, int N, int K, int64_t lda,
                                                             int64_t ldb, int64_t ldr, int64_t ldc, float* __restrict__ part,
                                                             int kps) {
  constexpr int BT = 128, BK = 32, KC_LD = BK + 4;
  constexpr int A_FLOATS = A_KMAJOR ? BK * BT : BT * KC_LD, B_FLOATS = B_KMAJOR ? BK * BT : BT * KC_LD;
  __shared__ __attribute__((aligned(16))) float sA[A_FLOATS];
  __shared__ __attribute__((aligned(16))) float sB[B_FLOATS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int i = lane & 31, g = lane >> 5;
  const int m0 = blockIdx.y * BT, n0 = blockIdx.x * BT;
  const int kb = part != nullptr ? (int)blockIdx.z * kps : 0;
  const int kend = part != nullptr && kb + kps < K ? kb + kps : K;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;

  // global -> registers: four 16-byte pieces of each operand per thread and step; zero outside the operand
  auto gload = [&](const float* X, int64_t ld, bool kmajor, int row0, int rows, int k0, float4 (&v)[4]) {
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const int idx = tid + 256 * q;
      float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
      if (!kmajor) {
        const int row = row0 + (idx >> 3), k = k0 + (idx & 7) * 4;
        if (row < rows) {
          const float* p = X + (int64_t)row * ld + k;
          if (k + 4 <= kend) x = *reinterpret_cast<const float4*>(p);
          else {
            if (k < kend) x.x = p[0];
            if (k + 1 < kend) x.y = p[1];
            if (k + 2 < kend) x.z = p[2];
          }
        }
      } else {
        const int k = k0 + (idx >> 5), row = row0 + (idx & 31) * 4;
        if (k < kend) {
          const float* p = X + (int64_t)k * ld + row;
          if (row + 4 <= rows) x = *reinterpret_cast<const float4*>(p);
          else {
            if (row < rows) x.x = p[0];
            if (row + 1 < rows) x.y = p[1];
            if (row + 2 < rows) x.z = p[2];
          }
        }
      }
      v[q] = x;
    }
  };
  auto sstore = [&](float* sX, bool kmajor, const float4 (&v)[4]) {
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const int idx = tid + 256 * q;
      if (!kmajor) *reinterpret_cast<float4*>(sX + (idx >> 3) * KC_LD + (idx & 7) * 4) = v[q];
      else *reinterpret_cast<float4*>(sX + (idx >> 5) * BT + (idx & 31) * 4) = v[q];
    }
  };
  // the four k of chunk j (8 wide) that this lane contracts, for tile row r of an operand
  auto frag = [&](const float* sX, bool kmajor, int r, int j, float (&f)[4]) {
    if (!kmajor) {
      const float4 x = *reinterpret_cast<const float4*>(sX + r * KC_LD + 8 * j + 4 * g);
      f[0] = x.x; f[1] = x.y; f[2] = x.z; f[3] = x.w;
    } else {
#pragma unroll
      for (int t = 0; t < 4; t++) f[t] = sX[(8 * j + 4 * g + t) * BT + r];
    }
  };

  f32x16_t acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;

  float4 va[4], vb[4];
  gload(A, lda, A_KMAJOR, m0, M, kb, va);
  gload(B, ldb, B_KMAJOR, n0, N, kb, vb);
  for (int k0 = kb; k0 < kend; k0 += BK) {
    sstore(sA, A_KMAJOR, va);
    sstore(sB, B_KMAJOR, vb);
    __syncthreads();
    if (k0 + BK < kend) {                                // in flight while this step is multiplied
      gload(A, lda, A_KMAJOR, m0, M, k0 + BK, va);
      gload(B, ldb, B_KMAJOR, n0, N, k0 + BK, vb);
    }
#pragma unroll
    for (int j = 0; j < BK / 8; j++) {
      float fa[2][4], fb[2][4];
#pragma unroll
      for (int a = 0; a < 2; a++) frag(sA, A_KMAJOR, wm + a * 32 + i, j, fa[a]);
#pragma unroll
      for (int b = 0; b < 2; b++) frag(sB, B_KMAJOR, wn + b * 32 + i, j, fb[b]);
#pragma unroll
      for (int t = 0; t < 4; t++)
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
          for (int b = 0; b < 2; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[a][t], fb[b][t], acc[a][b], 0, 0, 0);
    }
    __syncthreads();                                     // every wavefront is done with this step's tiles
  }
  // register r of lane l: row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32 of its 32 x 32 tile
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int b = 0; b < 2; b++) {
      const int col = n0 + wn + b * 32 + i;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int row = m0 + wm + a * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
        if (row < M && col < N) {
          float v = acc[a][b][r];
          if (part != nullptr) {
            part[((int64_t)blockIdx.z * M + row) * N + col] = v;
          } else {
            if (R != nullptr) v += R[(int64_t)row * ldr + col];
            C[(int64_t)row * ldc + col] = v;
          }
        }
      }
    }
}

// VEC: a thread owns four consecutive columns of a row (N, ldr and ldc multiples of 4, rows of R and C aligned for one
// access of four elements): 16-byte loads from every plane.
template <typename T, bool VEC = false>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float* __restrict__ part, const T* R, T* C, int M, int N,
                                                                 int splits, int64_t ldr, int64_t ldc) {
  constexpr int V = VEC ? 4 : 1;
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
  if (i >= (int64_t)M * N) return;
  const int row = (int)(i / N), col = (int)(i - (int64_t)row * N);
  const int64_t plane = (int64_t)M * N;
  float v[V];
#pragma unroll
  for (int e = 0; e < V; e++) v[e] = 0.f;
  auto load = [&](int z, float (&t)[V]) {
    if constexpr (VEC) {
      const float4 q = *reinterpret_cast<const float4*>(part + z * plane + i);
      t[0] = q.x; t[1] = q.y; t[2] = q.z; t[3] = q.w;
    } else {
      t[0] = part[z * plane + i];
    }
  };
  int z = 0;
  for (; z + 8 <= splits; z += 8) {                       // eight loads in flight, added in plane order
    float t[8][V];
#pragma unroll
    for (int u = 0; u < 8; u++) load(z + u, t[u]);
#pragma unroll
    for (int u = 0; u < 8; u++)
#pragma unroll
      for (int e = 0; e < V; e++) v[e] += t[u][e];
  }
  if (z + 4 <= splits) {
    float t[4][V];
#pragma unroll
    for (int u = 0; u < 4; u++) load(z + u, t[u]);
#pragma unroll
    for (int u = 0; u < 4; u++)
#pragma unroll
      for (int e = 0; e < V; e++) v[e] += t[u][e];
    z += 4;
  }
  for (; z < splits; z++) {
    float t[V];
    load(z, t);
#pragma unroll
    for (int e = 0; e < V; e++) v[e] += t[e];
  }
  if constexpr (VEC) {
    if (R != nullptr) {
      if constexpr (sizeof(T) == 2) {
        const u32x2_t r = *reinterpret_cast<const u32x2_t*>(R + (int64_t)row * ldr + col);
        v[0] += __uint_as_float(r[0] << 16); v[1] += __uint_as_float(r[0] & 0xffff0000u);
        v[2] += __uint_as_float(r[1] << 16); v[3] += __uint_as_float(r[1] & 0xffff0000u);
      } else {
        const float4 r = *reinterpret_cast<const float4*>(R + (int64_t)row * ldr + col);
        v[0] += r.x; v[1] += r.y; v[2] += r.z; v[3] += r.w;
      }
    }
    if constexpr (sizeof(T) == 2) {
      u32x2_t o;
      o[0] = pack_bf16x2(v[0], v[1]);
      o[1] = pack_bf16x2(v[2], v[3]);
      *reinterpret_cast<u32x2_t*>(C + (int64_t)row * ldc + col) = o;
    } else {
      *reinterpret_cast<float4*>(C + (int64_t)row * ldc + col) = make_float4(v[0], v[1], v[2], v[3]);
    }
  } else {
    if (R != nullptr) v[0] += to_f32(R[(int64_t)row * ldr + col]);
    C[(int64_t)row * ldc + col] = from_f32<T>(v[0]);
  }
}

// Launches the reduction of `splits` fp32 planes [M, N] (+ R) into C.
template <typename T>
static void launch_splitk_reduce(hipStream_t st, const float* part, const void* R, void* C, int M, int N, int splits, int64_t ldr,
                                 int64_t ldc) {
  const uintptr_t al = 4 * sizeof(T) - 1;
  const bool vec = N % 4 == 0 && ldc % 4 == 0 && (reinterpret_cast<uintptr_t>(C) & al) == 0 && (reinterpret_cast<uintptr_t>(part) & 15) == 0 &&
                   (R == nullptr || (ldr % 4 == 0 && (reinterpret_cast<uintptr_t>(R) & al) == 0));
  const int64_t items = vec ? (int64_t)M * N / 4 : (int64_t)M * N;
  const dim3 grid((unsigned)((items + 255) / 256));
  if (vec)
    hipLaunchKernelGGL((gemm_splitk_reduce_kernel<T, true>), grid, dim3(256), 0, st, part, static_cast<const T*>(R), static_cast<T*>(C), M,
                       N, splits, ldr, ldc);
  else
    hipLaunchKernelGGL((gemm_splitk_reduce_kernel<T, false>), grid, dim3(256), 0, st, part, static_cast<const T*>(R), static_cast<T*>(C), M,
                       N, splits, ldr, ldc);
}

// Few output tiles and a long contraction (the logits adjoint dX = dY . Wcls of a small batch:
// 6 tiles, K = 32000): split K over enough blocks to fill the chip.
static int generic_tile(int64_t M, int64_t N) {          // block tile edge: 64 while 128 would leave most CUs idle
  return ((M + 127) / 128) * ((N + 127) / 128) < 64 ? 64 : 128;
}
static int generic_splits(int64_t M, int64_t N, int64_t K) {
  const int t = generic_tile(M, N);
  const int64_t tiles = ((M + t - 1) / t) * ((N + t - 1) / t);
  if (tiles >= 128 || K < 2048) return 1;
  int64_t s = (t == 64 ? 1024 : 512) / tiles;          // about four (two) resident blocks per CU
  if (s > K / 256) s = K / 256;
  return (int)(s < 2 ? 1 : (s > 256 ? 256 : s));
}

template <int BM, int BN, int BK, int NSTAGE, int WM, int WN, bool AK, bool BKM>
static int launch_bf16(hipStream_t st, const void* A, const void* B, const void* R, void* C, int M, int N, int K, int lda,
                       int ldb, int ldr, int ldc, uint32_t a_bytes, uint32_t b_bytes, float* part = nullptr, int splits = 1) {
  // 16-byte epilogue accesses need aligned rows of C (and R)
  const int vec_ok = ((reinterpret_cast<uintptr_t>(C) & 15) == 0 && ldc % 8 == 0 &&
                      (R == nullptr || ((reinterpret_cast<uintptr_t>(R) & 15) == 0 && ldr % 8 == 0)))
                         ? 1 : 0;
  auto kern = gemm_bf16_kernel<BM, BN, BK, NSTAGE, WM, WN, AK, BKM>;
  constexpr int smem = NSTAGE * (BM + BN) * BK * 2;
  static bool configured = false;   // idempotent; a race only repeats the call
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return emi_fail(EMI_INTERNAL, "emi_gemm: cannot reserve %d bytes of LDS: %s", smem, hipGetErrorString(e));
    configured = true;
  }
  const int tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  if (part != nullptr && splits > 1) {
    const int kps = (((K + splits - 1) / splits) + BK - 1) / BK * BK;
    const int nz = (K + kps - 1) / kps;
    hipLaunchKernelGGL(kern, dim3(tiles * nz), dim3(WM * WN * 64), smem, st, static_cast<const uint16_t*>(A),
                       static_cast<const uint16_t*>(B), static_cast<const uint16_t*>(R), static_cast<uint16_t*>(C), M, N, K,
                       lda, ldb, ldr, ldc, a_bytes, b_bytes, vec_ok, part, kps, GemmGroup{});
    EMI_CHECK_LAUNCH("emi_gemm(split-K)");
    launch_splitk_reduce<bf16>(st, part, R, C, M, N, nz, (int64_t)ldr, (int64_t)ldc);
    EMI_CHECK_LAUNCH("emi_gemm(split-K reduce)");
    return EMI_OK;
  }
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(WM * WN * 64), smem, st, static_cast<const uint16_t*>(A),
                     static_cast<const uint16_t*>(B), static_cast<const uint16_t*>(R), static_cast<uint16_t*>(C), M, N, K,
                     lda, ldb, ldr, ldc, a_bytes, b_bytes, vec_ok, static_cast<float*>(nullptr), 0, GemmGroup{});
  EMI_CHECK_LAUNCH("emi_gemm");
  return EMI_OK;
}

// Splits of K for `count` independent products of one shape in one launch (see bf16_splits).
static int grouped_splits(int64_t M, int64_t N, int64_t K, int count) {
  const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128) * count;
  if (tiles > 128 || K < 2048) return 1;
  int64_t s = 512 / tiles;
  if (s > K / 1024) s = K / 1024;
  return (int)(s < 2 ? 1 : (s > 64 ? 64 : s));
}

// The 128x128 kernel on a group of products (GemmGroup): one launch, count times the tiles (or, summed, count times
// the contraction).
template <bool AK, bool BKM>
static int launch_bf16_grouped(hipStream_t st, const GemmGroup& g, int M, int N, int K, int lda, int ldb, int ldr, int ldc,
                               uint32_t a_bytes, uint32_t b_bytes, void* workspace, size_t workspace_bytes) {
  constexpr int BM = 128, BN = 128, BK = 64;
  int vec_ok = (ldc % 8 == 0 && ldr % 8 == 0) ? 1 : 0;
  const int nout = g.sum ? 1 : g.count;
  for (int i = 0; i < nout; i++)
    if ((reinterpret_cast<uintptr_t>(g.C[i]) & 15) || (g.R[i] != nullptr && (reinterpret_cast<uintptr_t>(g.R[i]) & 15))) vec_ok = 0;
  auto kern = gemm_bf16_kernel<BM, BN, BK, 2, 2, 2, AK, BKM>;
  constexpr int smem = 2 * (BM + BN) * BK * 2;
  static bool configured = false;   // idempotent; a race only repeats the call
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return emi_fail(EMI_INTERNAL, "emi_gemm_grouped: cannot reserve %d bytes of LDS: %s", smem, hipGetErrorString(e));
    configured = true;
  }
  const int big_tiles = ((M + 255) / 256) * ((N + 255) / 256);
  const int64_t group_tiles = (int64_t)big_tiles * g.count, rounds = (group_tiles + 255) / 256;
  if (!g.sum && group_tiles >= 192 && (4 * group_tiles >= 3 * rounds * 256 || K >= 4096)) {
    // enough 256x256 tiles over the whole group to fill the chip: the ping-pong kernel, product-major.  With a short
    // contraction a last round that leaves most CUs idle costs more than the larger tile gains (3 x [8192, 768] x 768:
    // 288 tiles, 48 us against 43 us on 128x128 tiles); with a long one it does not (12 x [768, 2048] x 8192: 351 vs 462 us).
    constexpr int smem_pp = 2 * 65536;
    static bool configured_pp = false;
    if (!configured_pp) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_pingpong_kernel<AK, BKM, true>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, smem_pp);
      if (e != hipSuccess) return emi_fail(EMI_INTERNAL, "emi_gemm_grouped: cannot reserve %d bytes of LDS: %s", smem_pp, hipGetErrorString(e));
      configured_pp = true;
    }
    hipLaunchKernelGGL((gemm_bf16_pingpong_kernel<AK, BKM, true>), dim3(big_tiles * g.count), dim3(512), smem_pp, st, g.A[0], g.B[0],
                       g.R[0], g.C[0], M, N, K, lda, ldb, ldr, ldc, a_bytes, b_bytes, vec_ok, g);
    EMI_CHECK_LAUNCH("emi_gemm_grouped(256-tiles)");
    return EMI_OK;
  }
  const int tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  const int splits = g.sum ? 1 : grouped_splits(M, N, K, g.count);
  if (splits > 1 && workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0 &&
      workspace_bytes >= (size_t)g.count * splits * M * N * sizeof(float)) {
    float* part = static_cast<float*>(workspace);
    const int kps = (((K + splits - 1) / splits) + BK - 1) / BK * BK;
    const int nz = (K + kps - 1) / kps;
    hipLaunchKernelGGL(kern, dim3(tiles * g.count * nz), dim3(256), smem, st, g.A[0], g.B[0], g.R[0], g.C[0], M, N, K, lda, ldb,
                       ldr, ldc, a_bytes, b_bytes, vec_ok, part, kps, g);
    EMI_CHECK_LAUNCH("emi_gemm_grouped(split-K)");
    for (int i = 0; i < g.count; i++) {
      launch_splitk_reduce<bf16>(st, part + (int64_t)i * nz * M * N, g.R[i], g.C[i], M, N, nz, (int64_t)ldr, (int64_t)ldc);
      EMI_CHECK_LAUNCH("emi_gemm_grouped(split-K reduce)");
    }
    return EMI_OK;
  }
  hipLaunchKernelGGL(kern, dim3(tiles * nout), dim3(256), smem, st, g.A[0], g.B[0], g.R[0], g.C[0], M, N, K, lda, ldb, ldr, ldc,
                     a_bytes, b_bytes, vec_ok, static_cast<float*>(nullptr), 0, g);
  EMI_CHECK_LAUNCH("emi_gemm_grouped");
  return EMI_OK;
}

template <bool AKM, bool BKM>
static int launch_bf16_pingpong(hipStream_t st, const void* A, const void* B, const void* R, void* C, int M, int N, int K,
                                int lda, int ldb, int ldr, int ldc, uint32_t a_bytes, uint32_t b_bytes) {
  const int vec_ok = ((reinterpret_cast<uintptr_t>(C) & 15) == 0 && ldc % 8 == 0 &&
                      (R == nullptr || ((reinterpret_cast<uintptr_t>(R) & 15) == 0 && ldr % 8 == 0)))
                         ? 1 : 0;
  constexpr int smem = 2 * 65536;
  static bool configured = false;   // idempotent; a race only repeats the call
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_pingpong_kernel<AKM, BKM>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return emi_fail(EMI_INTERNAL, "emi_gemm: cannot reserve %d bytes of LDS: %s", smem, hipGetErrorString(e));
    configured = true;
  }
  const int tiles = ((M + 255) / 256) * ((N + 255) / 256);
  if (vec_ok && M % 256 == 0 && N % 256 == 0) {
    static bool configured_full = false;
    if (!configured_full) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_pingpong_kernel<AKM, BKM, false, 4>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, smem);
      if (e != hipSuccess) return emi_fail(EMI_INTERNAL, "emi_gemm: cannot reserve %d bytes of LDS: %s", smem, hipGetErrorString(e));
      configured_full = true;
    }
    hipLaunchKernelGGL((gemm_bf16_pingpong_kernel<AKM, BKM, false, 4>), dim3(tiles), dim3(512), smem, st,
                       static_cast<const uint16_t*>(A), static_cast<const uint16_t*>(B), static_cast<const uint16_t*>(R),
                       static_cast<uint16_t*>(C), M, N, K, lda, ldb, ldr, ldc, a_bytes, b_bytes, 1, NoGroup{}, NoEpi{});
    EMI_CHECK_LAUNCH("emi_gemm");
    return EMI_OK;
  }
  hipLaunchKernelGGL((gemm_bf16_pingpong_kernel<AKM, BKM>), dim3(tiles), dim3(512), smem, st, static_cast<const uint16_t*>(A),
                     static_cast<const uint16_t*>(B), static_cast<const uint16_t*>(R), static_cast<uint16_t*>(C), M, N, K,
                     lda, ldb, ldr, ldc, a_bytes, b_bytes, vec_ok, NoGroup{});
  EMI_CHECK_LAUNCH("emi_gemm");
  return EMI_OK;
}

// C = A . B^T with a SwiGLU epilogue (MODE 1: P0 = a in, Q0 = b, Q1 = g out; MODE 2: P0 = a, P1 = b in, Q0 = da, Q1 = db
// out).  Returns -1 when the shape is not one the fused kernel serves (the caller then runs the two passes).
template <int MODE>
static int launch_bf16_swiglu(hipStream_t st, const void* A, const void* B, const void* P0, const void* P1, void* Q0, void* Q1,
                              int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb) {
  auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const int64_t a_bytes = ((M - 1) * lda + K) * 2, b_bytes = ((N - 1) * ldb + K) * 2;
  if (M % 256 || N % 256 || K % 8 || K <= 0 || lda % 8 || ldb % 8 || (M / 256) * (N / 256) < 192 || !al16(A) || !al16(B) ||
      !al16(P0) || (MODE == 2 && !al16(P1)) || !al16(Q0) || !al16(Q1) || a_bytes >= 0x7fffff00LL || b_bytes >= 0x7fffff00LL ||
      M * N * 2 >= 0x7fffff00LL)
    return -1;
  constexpr int smem = 2 * 65536;
  auto kern = gemm_bf16_pingpong_kernel<false, false, false, MODE>;
  static bool configured = false;   // idempotent; a race only repeats the call
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return emi_fail(EMI_INTERNAL, "emi_gemm_swiglu: cannot reserve %d bytes of LDS: %s", smem, hipGetErrorString(e));
    configured = true;
  }
  const int tiles = (int)((M / 256) * (N / 256));
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(512), smem, st, static_cast<const uint16_t*>(A), static_cast<const uint16_t*>(B),
                     static_cast<const uint16_t*>(P0), static_cast<uint16_t*>(Q0), (int)M, (int)N, (int)K, (int)lda, (int)ldb, (int)N,
                     (int)N, (uint32_t)a_bytes, (uint32_t)b_bytes, 1, NoGroup{},
                     SwigluEpi{static_cast<const uint16_t*>(P1), static_cast<uint16_t*>(Q1)});
  EMI_CHECK_LAUNCH("emi_gemm_swiglu");
  return EMI_OK;
}

// C = rope(A . B^T): returns -1 when the shape is not one the fused kernel serves (the caller then runs the two passes).
static int launch_bf16_rope(hipStream_t st, const void* A, const void* B, void* C, const float* table, int64_t M, int64_t N,
                            int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t seq, int64_t head_dim) {
  auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const int64_t a_bytes = ((M - 1) * lda + K) * 2, b_bytes = ((N - 1) * ldb + K) * 2;
  // a head is a whole number of the lanes' 4-column quads
  if (M % 256 || N % 256 || K % 8 || K <= 0 || lda % 8 || ldb % 8 || ldc % 8 || ldc < N || (M / 256) * (N / 256) < 192 ||
      !al16(A) || !al16(B) || !al16(C) || !al16(table) || a_bytes >= 0x7fffff00LL || b_bytes >= 0x7fffff00LL ||
      ((M - 1) * ldc + N) * 2 >= 0x7fffff00LL || head_dim % 4 || seq > 0x7fffffff)
    return -1;
  constexpr int smem = 2 * 65536;
  auto kern = gemm_bf16_pingpong_kernel<false, false, false, 3>;
  static bool configured = false;   // idempotent; a race only repeats the call
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return emi_fail(EMI_INTERNAL, "emi_gemm_rope: cannot reserve %d bytes of LDS: %s", smem, hipGetErrorString(e));
    configured = true;
  }
  const int tiles = (int)((M / 256) * (N / 256));
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(512), smem, st, static_cast<const uint16_t*>(A), static_cast<const uint16_t*>(B),
                     static_cast<const uint16_t*>(nullptr), static_cast<uint16_t*>(C), (int)M, (int)N, (int)K, (int)lda, (int)ldb,
                     (int)ldc, (int)ldc, (uint32_t)a_bytes, (uint32_t)b_bytes, 1, NoGroup{},
                     RopeEpi{table, (int)seq, (int)head_dim});
  EMI_CHECK_LAUNCH("emi_gemm_rope");
  return EMI_OK;
}

// Split-K on the 256x256 ping-pong kernel: k-contiguous products with too few 256-tiles for that kernel, too many
// 128-tiles for bf16_splits and a long contraction (dX of the classifier of a small model, [8192, 32000] x [32000, 768]:
// 96 tiles of 256, 384 of 128).  The 128-tile kernel runs those at 0.75 PFLOP/s (two blocks on half the CUs, one on the
// others); four splits are 384 ping-pong blocks at 1.1 PFLOP/s plus the reduction of 4 x M x N fp32 partials.
static int pingpong_splits(int64_t M, int64_t N, int64_t K, bool k_contiguous) {
  if (!k_contiguous || K < 8192) return 1;
  const int64_t big = ((M + 255) / 256) * ((N + 255) / 256), t128 = ((M + 127) / 128) * ((N + 127) / 128);
  if (big >= 192 || t128 <= 128 || big > 128) return 1;
  int64_t s = (320 + big - 1) / big;
  if (s > 8) s = 8;
  while (s > 1 && K / s < 2048) s--;
  return (int)s;
}

static int launch_bf16_pingpong_splitk(hipStream_t st, const void* A, const void* B, const void* R, void* C, int M, int N, int K,
                                       int lda, int ldb, int ldr, int ldc, uint32_t a_bytes, uint32_t b_bytes, float* part,
                                       int splits) {
  auto kern = gemm_bf16_pingpong_kernel<false, false, false, 5>;
  constexpr int smem = 2 * 65536;
  static bool configured = false;   // idempotent; a race only repeats the call
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return emi_fail(EMI_INTERNAL, "emi_gemm: cannot reserve %d bytes of LDS: %s", smem, hipGetErrorString(e));
    configured = true;
  }
  const int tiles = ((M + 255) / 256) * ((N + 255) / 256);
  const int kps = (((K + splits - 1) / splits) + 63) / 64 * 64;
  const int nz = (K + kps - 1) / kps;
  hipLaunchKernelGGL(kern, dim3(tiles * nz), dim3(512), smem, st, static_cast<const uint16_t*>(A), static_cast<const uint16_t*>(B),
                     static_cast<const uint16_t*>(nullptr), static_cast<uint16_t*>(nullptr), M, N, K, lda, ldb, ldr, ldc, a_bytes,
                     b_bytes, 0, NoGroup{}, SplitEpi{part, kps});
  EMI_CHECK_LAUNCH("emi_gemm(split-K, 256-tiles)");
  launch_splitk_reduce<bf16>(st, part, R, C, M, N, nz, (int64_t)ldr, (int64_t)ldc);
  EMI_CHECK_LAUNCH("emi_gemm(split-K reduce)");
  return EMI_OK;
}

// The 128x128 bf16 kernel on few tiles and a long contraction (the weight gradients of a small model:
// dW[768, 768] over 8192 tokens is 36 tiles): two blocks per CU, at least 1024 of K per block.
static int bf16_splits(int64_t M, int64_t N, int64_t K) {
  if (((M + 255) / 256) * ((N + 255) / 256) >= 192) return 1;         // the 256x256 ping-pong kernel takes these
  const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
  if (tiles > 128 || K < 2048) return 1;
  int64_t s = 512 / tiles;
  if (s > K / 1024) s = K / 1024;
  return (int)(s < 2 ? 1 : (s > 64 ? 64 : s));
}

template <bool AK, bool BKM>
static int launch_bf16_layout(hipStream_t st, const void* A, const void* B, const void* R, void* C, int M, int N, int K,
                              int lda, int ldb, int ldr, int ldc, uint32_t a_bytes, uint32_t b_bytes, void* workspace,
                              size_t workspace_bytes) {
  const int splits = bf16_splits(M, N, K);
  if (splits > 1 && workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0 &&
      workspace_bytes >= (size_t)splits * M * N * sizeof(float))
    return launch_bf16<128, 128, 64, 2, 2, 2, AK, BKM>(st, A, B, R, C, M, N, K, lda, ldb, ldr, ldc, a_bytes, b_bytes,
                                                      static_cast<float*>(workspace), splits);
  if constexpr (!AK && !BKM) {
    const int pps = pingpong_splits(M, N, K, true);
    if (pps > 1 && workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0 &&
        workspace_bytes >= (size_t)pps * M * N * sizeof(float))
      return launch_bf16_pingpong_splitk(st, A, B, R, C, M, N, K, lda, ldb, ldr, ldc, a_bytes, b_bytes,
                                         static_cast<float*>(workspace), pps);
  }
  // 256x256 tiles (the ping-pong kernel) when they fill the chip, else 128x128.
  const int64_t big_tiles = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
  if (big_tiles >= 192) return launch_bf16_pingpong<AK, BKM>(st, A, B, R, C, M, N, K, lda, ldb, ldr, ldc, a_bytes, b_bytes);
  return launch_bf16<128, 128, 64, 2, 2, 2, AK, BKM>(st, A, B, R, C, M, N, K, lda, ldb, ldr, ldc, a_bytes, b_bytes);
}

template <typename T>
static int launch_generic(hipStream_t st, const void* A, const void* B, const void* R, void* C, int M, int N, int K,
                          int64_t lda, int64_t ldb, int64_t ldr, int64_t ldc, int trans_a, int trans_b, void* workspace, size_t workspace_bytes) {
  const int tile = generic_tile(M, N);
  dim3 grid((N + tile - 1) / tile, (M + tile - 1) / tile);
  if (grid.y > 65535) return emi_fail(EMI_INVALID_ARGUMENT, "emi_gemm: M=%d too large for the generic path", M);
  const int splits = generic_splits(M, N, K);
#define EMI_GENERIC(PART, KPS)                                                                                          \
  do {                                                                                                                   \
    if (tile == 64)                                                                                                      \
      hipLaunchKernelGGL((gemm_generic_kernel<T, 1>), grid, dim3(256), 0, st, static_cast<const T*>(A), static_cast<const T*>(B), \
                         static_cast<const T*>(R), static_cast<T*>(C), M, N, K, lda, ldb, ldr, ldc, trans_a, trans_b, PART, KPS); \
    else                                                                                                                 \
      hipLaunchKernelGGL((gemm_generic_kernel<T, 2>), grid, dim3(256), 0, st, static_cast<const T*>(A), static_cast<const T*>(B), \
                         static_cast<const T*>(R), static_cast<T*>(C), M, N, K, lda, ldb, ldr, ldc, trans_a, trans_b, PART, KPS); \
  } while (0)
  if (splits > 1 && workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0 &&
      workspace_bytes >= (size_t)splits * M * N * sizeof(float)) {
    const int kps = (((K + splits - 1) / splits) + 15) / 16 * 16;
    grid.z = (K + kps - 1) / kps;
    float* part = static_cast<float*>(workspace);
    EMI_GENERIC(part, kps);
    EMI_CHECK_LAUNCH("emi_gemm(generic split-K)");
    launch_splitk_reduce<T>(st, part, R, C, M, N, (int)grid.z, ldr, ldc);
    EMI_CHECK_LAUNCH("emi_gemm(generic split-K reduce)");
    return EMI_OK;
  }
  EMI_GENERIC(static_cast<float*>(nullptr), 0);
#undef EMI_GENERIC
  EMI_CHECK_LAUNCH("emi_gemm(generic)");
  return EMI_OK;
}

// gemm_skinny.hip
int launch_skinny(hipStream_t st, const void* A, const void* B, const void* R, void* C, void* workspace, size_t workspace_bytes,
                  int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldr, int64_t ldc, int trans_a, int trans_b,
                  int dtype);
size_t skinny_workspace_bytes(int64_t M, int64_t N, int64_t K, int trans_a, int trans_b, int dtype);

}  // namespace emi

using namespace emi;


extern "C" size_t emi_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int trans_a, int trans_b, int dtype) {
  const size_t skinny = skinny_workspace_bytes(M, N, K, trans_a, trans_b, dtype);
  if (skinny) return skinny;
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  // few tiles and a long contraction: split-K partials (the larger of what the fp32 / odd-shape path and the
  // 128x128 bf16 kernel would use, since alignment decides between them at launch time)
  int splits = generic_splits(M, N, K);
  if (dtype == EMI_BF16 && bf16_splits(M, N, K) > splits) splits = bf16_splits(M, N, K);
  if (dtype == EMI_BF16 && pingpong_splits(M, N, K, !trans_a && trans_b) > splits) splits = pingpong_splits(M, N, K, true);
  return splits > 1 ? (size_t)splits * M * N * sizeof(float) : 0;
}

extern "C" int emi_gemm(emi_stream_t stream, const void* A, const void* B, const void* R, void* C, int64_t M, int64_t N,
                        int64_t K, int64_t lda, int64_t ldb, int64_t ldr, int64_t ldc, int trans_a, int trans_b,
                        int dtype) {
  return emi_gemm_ws(stream, A, B, R, C, nullptr, 0, M, N, K, lda, ldb, ldr, ldc, trans_a, trans_b, dtype);
}

extern "C" int emi_gemm_ws(emi_stream_t stream, const void* A, const void* B, const void* R, void* C, void* workspace,
                           size_t workspace_bytes, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldr,
                           int64_t ldc, int trans_a, int trans_b, int dtype) {
  EMI_REQUIRE(M >= 0 && N >= 0 && K >= 0, "emi_gemm: negative dimension M=%lld N=%lld K=%lld", (long long)M, (long long)N,
              (long long)K);
  EMI_REQUIRE(M <= 0x7fffffff && N <= 0x7fffffff && K <= 0x7fffffff, "emi_gemm: dimension exceeds 2^31-1");
  EMI_REQUIRE(dtype == EMI_F32 || dtype == EMI_BF16, "emi_gemm: unsupported dtype code %d (want 11=f32 or 16=bf16)", dtype);
  if (M == 0 || N == 0) return EMI_OK;
  EMI_REQUIRE(A && B && C, "emi_gemm: null buffer");
  EMI_REQUIRE(lda >= (trans_a ? M : K) && ldb >= (trans_b ? K : N) && ldc >= N && (R == nullptr || ldr >= N),
              "emi_gemm: leading dimension smaller than the row length (lda=%lld ldb=%lld ldr=%lld ldc=%lld)",
              (long long)lda, (long long)ldb, (long long)ldr, (long long)ldc);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (K > 0 && (R == nullptr || ldr >= N)) {
    // single-token forms (mat-vec and its adjoints): weight-bandwidth-bound kernels
    const int rc = launch_skinny(st, A, B, R, C, workspace, workspace_bytes, M, N, K, lda, ldb, ldr, ldc, trans_a, trans_b, dtype);
    if (rc >= 0) return rc;
  }
  if (dtype == EMI_BF16) {
    const int64_t a_rows = trans_a ? K : M, b_rows = trans_b ? N : K;
    const int64_t a_bytes = ((a_rows - 1) * lda + (trans_a ? M : K)) * 2;
    const int64_t b_bytes = ((b_rows - 1) * ldb + (trans_b ? K : N)) * 2;
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    // The fast path moves 16-byte chunks: rows must start 16-byte aligned and
    // row lengths in the contiguous dimension must be multiples of 8 elements.
    const bool fast = K > 0 && al16(A) && al16(B) && (lda % 8 == 0) && (ldb % 8 == 0) && (K % 8 == 0) &&
                      (!trans_a || M % 8 == 0) && (trans_b || N % 8 == 0) && a_bytes < 0x7fffff00LL &&
                      b_bytes < 0x7fffff00LL && ldr <= 0x7fffffff && ldc <= 0x7fffffff;
    if (fast) {
      const int m = (int)M, n = (int)N, k = (int)K;
      const uint32_t ab = (uint32_t)a_bytes, bb = (uint32_t)b_bytes;
      if (!trans_a && trans_b)
        return launch_bf16_layout<false, false>(st, A, B, R, C, m, n, k, (int)lda, (int)ldb, (int)ldr, (int)ldc, ab, bb, workspace, workspace_bytes);
      if (!trans_a && !trans_b)
        return launch_bf16_layout<false, true>(st, A, B, R, C, m, n, k, (int)lda, (int)ldb, (int)ldr, (int)ldc, ab, bb, workspace, workspace_bytes);
      if (trans_a && !trans_b)
        return launch_bf16_layout<true, true>(st, A, B, R, C, m, n, k, (int)lda, (int)ldb, (int)ldr, (int)ldc, ab, bb, workspace, workspace_bytes);
      return launch_bf16_layout<true, false>(st, A, B, R, C, m, n, k, (int)lda, (int)ldb, (int)ldr, (int)ldc, ab, bb, workspace, workspace_bytes);
    }
    return launch_generic<bf16>(st, A, B, R, C, (int)M, (int)N, (int)K, lda, ldb, ldr, ldc, trans_a, trans_b, workspace, workspace_bytes);
  }
  // fp32 on 16-byte aligned k-contiguous rows: 32x32 tiles, K split over the block's wavefronts, operands straight from global memory (at every size measured
  // this beats the LDS-staged kernel, whose loads are element-wise: 1024^3 45 vs 3 TFLOP/s, 2048^3 55 vs 13)
  if (K > 0 && (M + 31) / 32 <= 65535 &&
      (trans_a || ((reinterpret_cast<uintptr_t>(A) & 15) == 0 && lda % 4 == 0)) &&
      (!trans_b || ((reinterpret_cast<uintptr_t>(B) & 15) == 0 && ldb % 4 == 0))) {
    dim3 grid((unsigned)((N + 31) / 32), (unsigned)((M + 31) / 32));
    const int splits = generic_splits(M, N, K);
    // 128 x 128 tiles staged through LDS once they fill the chip (alone or as planes of K)
    const bool tiled_ok = (reinterpret_cast<uintptr_t>(A) & 15) == 0 && (reinterpret_cast<uintptr_t>(B) & 15) == 0 &&
                          lda % 4 == 0 && ldb % 4 == 0;
    const int64_t tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
    if (splits > 1 && workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0 &&
        workspace_bytes >= (size_t)splits * M * N * sizeof(float)) {
      // few tiles and a long contraction (dX = dY . Wcls of a small batch): planes of K on the same kernel, partials
      // added in fixed order by the reduce kernel (256 x 288 x 32000: 130 us on the LDS-staged kernel)
      int kps = (int)((((K + splits - 1) / splits) + 31) / 32 * 32);
      grid.z = (unsigned)((K + kps - 1) / kps);
      float* part = static_cast<float*>(workspace);
      if (tiled_ok && tiles128 * grid.z >= 192) {
        // one block per CU and no second round: at most 256 / tiles planes (never more than the workspace holds)
        const int64_t want = 256 / tiles128 < splits ? 256 / tiles128 : splits;
        kps = (int)((((K + want - 1) / want) + 31) / 32 * 32);
        grid.z = (unsigned)((K + kps - 1) / kps);
        const dim3 gridt((unsigned)((N + 127) / 128), (unsigned)((M + 127) / 128), grid.z);
#define EMI_F32_TILED_SPLIT(AKM, BKM)                                                                                      \
  hipLaunchKernelGGL((gemm_f32_tiled_kernel<AKM, BKM>), gridt, dim3(256), 0, st, static_cast<const float*>(A),             \
                     static_cast<const float*>(B), static_cast<const float*>(nullptr), static_cast<float*>(C), (int)M,     \
                     (int)N, (int)K, lda, ldb, ldr, ldc, part, kps)
        if (!trans_a && trans_b) EMI_F32_TILED_SPLIT(false, false);
        else if (!trans_a && !trans_b) EMI_F32_TILED_SPLIT(false, true);
        else if (trans_a && !trans_b) EMI_F32_TILED_SPLIT(true, true);
        else EMI_F32_TILED_SPLIT(true, false);
#undef EMI_F32_TILED_SPLIT
        EMI_CHECK_LAUNCH("emi_gemm(fp32 tiled split-K)");
        launch_splitk_reduce<float>(st, part, R, C, (int)M, (int)N, (int)grid.z, ldr, ldc);
        EMI_CHECK_LAUNCH("emi_gemm(fp32 split-K reduce)");
        return EMI_OK;
      }
#define EMI_F32_SPLIT(AKM, BKM)                                                                                            \
  hipLaunchKernelGGL((gemm_f32_small_kernel<AKM, BKM, false, 4, 4, false>), grid, dim3(256), 0, st,                        \
                     static_cast<const float*>(A), static_cast<const float*>(B), static_cast<const float*>(nullptr),       \
                     static_cast<float*>(C), (int)M, (int)N, (int)K, lda, ldb, ldr, ldc, NoGroup{}, part, kps)
      if (!trans_a && trans_b) EMI_F32_SPLIT(false, false);
      else if (!trans_a && !trans_b) EMI_F32_SPLIT(false, true);
      else if (trans_a && !trans_b) EMI_F32_SPLIT(true, true);
      else EMI_F32_SPLIT(true, false);
#undef EMI_F32_SPLIT
      EMI_CHECK_LAUNCH("emi_gemm(fp32 split-K)");
      launch_splitk_reduce<float>(st, part, R, C, (int)M, (int)N, (int)grid.z, ldr, ldc);
      EMI_CHECK_LAUNCH("emi_gemm(fp32 split-K reduce)");
      return EMI_OK;
    }
#define EMI_F32_SMALL_V(AKM, BKM, NWV, UV, ONCEV)                                                                          \
  hipLaunchKernelGGL((gemm_f32_small_kernel<AKM, BKM, false, NWV, UV, ONCEV>), grid, dim3(NWV * 64), 0, st,                \
                     static_cast<const float*>(A), static_cast<const float*>(B), static_cast<const float*>(R),             \
                     static_cast<float*>(C), (int)M, (int)N, (int)K, lda, ldb, ldr, ldc, NoGroup{})
    if (tiled_ok && tiles128 >= 192) {
      const dim3 gridt((unsigned)((N + 127) / 128), (unsigned)((M + 127) / 128));
#define EMI_F32_TILED(AKM, BKM)                                                                                            \
  hipLaunchKernelGGL((gemm_f32_tiled_kernel<AKM, BKM>), gridt, dim3(256), 0, st, static_cast<const float*>(A),             \
                     static_cast<const float*>(B), static_cast<const float*>(R), static_cast<float*>(C), (int)M, (int)N,   \
                     (int)K, lda, ldb, ldr, ldc, static_cast<float*>(nullptr), 0)
      if (!trans_a && trans_b) EMI_F32_TILED(false, false);
      else if (!trans_a && !trans_b) EMI_F32_TILED(false, true);
      else if (trans_a && !trans_b) EMI_F32_TILED(true, true);
      else EMI_F32_TILED(true, false);
#undef EMI_F32_TILED
      EMI_CHECK_LAUNCH("emi_gemm(fp32 tiled)");
      return EMI_OK;
    }
    // few blocks: latency decides, everything is requested at once; many blocks: the stepped form, whose smaller
    // register footprint keeps more wavefronts resident
    const bool few = (int64_t)grid.x * grid.y <= 1024;
#define EMI_F32_SMALL(AKM, BKM)                                            \
  do {                                                                     \
    if (few && K <= 384) EMI_F32_SMALL_V(AKM, BKM, 4, 12, true);           \
    else if (few && K <= 768) EMI_F32_SMALL_V(AKM, BKM, 8, 12, true);      \
    else EMI_F32_SMALL_V(AKM, BKM, 4, 4, false);                           \
  } while (0)
    if (!trans_a && trans_b) EMI_F32_SMALL(false, false);
    else if (!trans_a && !trans_b) EMI_F32_SMALL(false, true);
    else if (trans_a && !trans_b) EMI_F32_SMALL(true, true);
    else EMI_F32_SMALL(true, false);
#undef EMI_F32_SMALL
#undef EMI_F32_SMALL_V
    EMI_CHECK_LAUNCH("emi_gemm(fp32 small)");
    return EMI_OK;
  }
  return launch_generic<float>(st, A, B, R, C, (int)M, (int)N, (int)K, lda, ldb, ldr, ldc, trans_a, trans_b, workspace, workspace_bytes);
}

extern "C" int emi_swiglu_fwd(emi_stream_t stream, const void* a, const void* b, void* g, int64_t n, int dtype);
extern "C" int emi_swiglu_bwd(emi_stream_t stream, const void* a, const void* b, const void* dg, void* da, void* db, int64_t n,
                              int dtype);

extern "C" int emi_gemm_swiglu_fwd(emi_stream_t stream, const void* X, const void* W3, const void* A, void* B_out, void* G_out,
                                   int64_t M, int64_t N, int64_t K, int dtype) {
  EMI_REQUIRE(M >= 0 && N >= 0 && K >= 0, "emi_gemm_swiglu_fwd: negative dimension");
  EMI_REQUIRE(dtype == EMI_F32 || dtype == EMI_BF16, "emi_gemm_swiglu_fwd: unsupported dtype code %d", dtype);
  if (M == 0 || N == 0) return EMI_OK;
  EMI_REQUIRE(X && W3 && A && B_out && G_out, "emi_gemm_swiglu_fwd: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == EMI_BF16) {
    const int rc = launch_bf16_swiglu<1>(st, X, W3, A, nullptr, B_out, G_out, M, N, K, K, K);
    if (rc >= 0) return rc;
  }
  const int rc = emi_gemm(stream, X, W3, nullptr, B_out, M, N, K, K, K, N, N, 0, 1, dtype);
  if (rc != EMI_OK) return rc;
  return emi_swiglu_fwd(stream, A, B_out, G_out, M * N, dtype);
}

extern "C" size_t emi_gemm_swiglu_bwd_workspace_bytes(int64_t M, int64_t N, int64_t K, int dtype) {
  if (M <= 0 || N <= 0) return 0;
  return (size_t)M * N * (dtype == EMI_BF16 ? 2 : 4);           // dg, when the two passes run
}

extern "C" int emi_gemm_swiglu_bwd(emi_stream_t stream, const void* dY, const void* W2T, const void* A, const void* B, void* dA,
                                   void* dB, void* workspace, size_t workspace_bytes, int64_t M, int64_t N, int64_t K, int dtype) {
  EMI_REQUIRE(M >= 0 && N >= 0 && K >= 0, "emi_gemm_swiglu_bwd: negative dimension");
  EMI_REQUIRE(dtype == EMI_F32 || dtype == EMI_BF16, "emi_gemm_swiglu_bwd: unsupported dtype code %d", dtype);
  if (M == 0 || N == 0) return EMI_OK;
  EMI_REQUIRE(dY && W2T && A && B && dA && dB, "emi_gemm_swiglu_bwd: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == EMI_BF16) {
    const int rc = launch_bf16_swiglu<2>(st, dY, W2T, A, B, dA, dB, M, N, K, K, K);
    if (rc >= 0) return rc;
  }
  const size_t need = emi_gemm_swiglu_bwd_workspace_bytes(M, N, K, dtype);
  EMI_REQUIRE(workspace != nullptr && workspace_bytes >= need && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0,
              "emi_gemm_swiglu_bwd: this shape runs as two passes and needs a 16-byte aligned workspace of %zu bytes (got %zu)",
              need, workspace_bytes);
  const int rc = emi_gemm(stream, dY, W2T, nullptr, workspace, M, N, K, K, K, N, N, 0, 1, dtype);
  if (rc != EMI_OK) return rc;
  return emi_swiglu_bwd(stream, A, B, workspace, dA, dB, M * N, dtype);
}

extern "C" int emi_rope(emi_stream_t stream, const void* x, const float* table, void* y, int64_t batch, int64_t seq,
                        int64_t heads, int64_t head_dim, int inverse, int dtype);

extern "C" int emi_gemm_rope(emi_stream_t stream, const void* X, const void* W, void* Y, const float* rope_table, int64_t M,
                             int64_t N, int64_t K, int64_t seq, int64_t head_dim, int dtype) {
  EMI_REQUIRE(M >= 0 && N >= 0 && K >= 0 && seq > 0 && head_dim > 0 && head_dim % 2 == 0 && N % head_dim == 0 && M % seq == 0,
              "emi_gemm_rope: bad shape M=%lld N=%lld K=%lld seq=%lld head_dim=%lld (rows are whole sequences, columns whole heads)",
              (long long)M, (long long)N, (long long)K, (long long)seq, (long long)head_dim);
  if (M == 0 || N == 0) return EMI_OK;
  EMI_REQUIRE(X && W && Y && rope_table, "emi_gemm_rope: null buffer");
  if (dtype == EMI_BF16) {
    const int rc = launch_bf16_rope(static_cast<hipStream_t>(stream), X, W, Y, rope_table, M, N, K, K, K, N, seq, head_dim);
    if (rc >= 0) return rc;
  }
  const int rc = emi_gemm(stream, X, W, nullptr, Y, M, N, K, K, K, N, N, 0, 1, dtype);
  if (rc != EMI_OK) return rc;
  return emi_rope(stream, Y, rope_table, Y, M / seq, seq, N / head_dim, head_dim, 0, dtype);
}

extern "C" size_t emi_gemm_grouped_workspace_bytes(int count, int64_t M, int64_t N, int64_t K, int trans_a, int trans_b, int sum,
                                                    int dtype) {
  size_t need = emi_gemm_workspace_bytes(M, N, K, trans_a, trans_b, dtype);          // the one-by-one fallback
  if (count >= 2 && count <= kMaxGroup && !sum && dtype == EMI_BF16 && M > 0 && N > 0 && K > 0) {
    const int splits = grouped_splits(M, N, K, count);
    const size_t grouped = splits > 1 ? (size_t)count * splits * M * N * sizeof(float) : 0;
    if (grouped > need) need = grouped;
  }
  return need;
}

extern "C" int emi_gemm_grouped(emi_stream_t stream, int count, const void* const* A, const void* const* B, const void* const* R,
                                void* const* C, void* workspace, size_t workspace_bytes, int64_t M, int64_t N, int64_t K,
                                int64_t lda, int64_t ldb, int64_t ldr, int64_t ldc, int trans_a, int trans_b, int sum, int dtype) {
  EMI_REQUIRE(count >= 1 && count <= kMaxGroup, "emi_gemm_grouped: count %d not in 1..%d", count, kMaxGroup);
  EMI_REQUIRE(A && B && C, "emi_gemm_grouped: null pointer table");
  EMI_REQUIRE(M >= 0 && N >= 0 && K >= 0 && M <= 0x7fffffff && N <= 0x7fffffff && K <= 0x7fffffff,
              "emi_gemm_grouped: bad dimensions M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  EMI_REQUIRE(dtype == EMI_F32 || dtype == EMI_BF16, "emi_gemm_grouped: unsupported dtype code %d (want 11=f32 or 16=bf16)", dtype);
  const int nout = sum ? 1 : count;
  for (int i = 0; i < count; i++) EMI_REQUIRE(A[i] && B[i], "emi_gemm_grouped: null operand %d", i);
  for (int i = 0; i < nout; i++) EMI_REQUIRE(C[i], "emi_gemm_grouped: null result %d", i);
  if (M == 0 || N == 0) return EMI_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  bool fast = dtype == EMI_BF16 && count >= 2 && K > 0 && M > 8;
  if (fast) {
    const int64_t a_rows = trans_a ? K : M, b_rows = trans_b ? N : K;
    const int64_t a_bytes = ((a_rows - 1) * lda + (trans_a ? M : K)) * 2;
    const int64_t b_bytes = ((b_rows - 1) * ldb + (trans_b ? K : N)) * 2;
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    fast = lda >= (trans_a ? M : K) && ldb >= (trans_b ? K : N) && ldc >= N && (lda % 8 == 0) && (ldb % 8 == 0) && (K % 8 == 0) &&
           (!trans_a || M % 8 == 0) && (trans_b || N % 8 == 0) && a_bytes < 0x7fffff00LL && b_bytes < 0x7fffff00LL &&
           ldr <= 0x7fffffff && ldc <= 0x7fffffff && ((M + 255) / 256) * ((N + 255) / 256) < 192;
    for (int i = 0; i < count && fast; i++) fast = al16(A[i]) && al16(B[i]);
    // a residual on some results only would need a null check per product: all or none
    bool any_r = false, all_r = true;
    for (int i = 0; i < nout; i++) {
      const bool has = R != nullptr && R[i] != nullptr;
      any_r = any_r || has;
      all_r = all_r && has;
    }
    if (any_r && (!all_r || ldr < N)) fast = false;
    if (fast) {
      GemmGroup g{};
      g.count = count;
      g.sum = sum ? 1 : 0;
      for (int i = 0; i < count; i++) {
        g.A[i] = static_cast<const uint16_t*>(A[i]);
        g.B[i] = static_cast<const uint16_t*>(B[i]);
      }
      for (int i = 0; i < nout; i++) {
        g.R[i] = any_r ? static_cast<const uint16_t*>(R[i]) : nullptr;
        g.C[i] = static_cast<uint16_t*>(C[i]);
      }
      const int m = (int)M, n = (int)N, k = (int)K;
      const uint32_t ab = (uint32_t)a_bytes, bb = (uint32_t)b_bytes;
      if (!trans_a && trans_b)
        return launch_bf16_grouped<false, false>(st, g, m, n, k, (int)lda, (int)ldb, (int)ldr, (int)ldc, ab, bb, workspace, workspace_bytes);
      if (!trans_a && !trans_b)
        return launch_bf16_grouped<false, true>(st, g, m, n, k, (int)lda, (int)ldb, (int)ldr, (int)ldc, ab, bb, workspace, workspace_bytes);
      if (trans_a && !trans_b)
        return launch_bf16_grouped<true, true>(st, g, m, n, k, (int)lda, (int)ldb, (int)ldr, (int)ldc, ab, bb, workspace, workspace_bytes);
      return launch_bf16_grouped<true, false>(st, g, m, n, k, (int)lda, (int)ldb, (int)ldr, (int)ldc, ab, bb, workspace, workspace_bytes);
    }
  }
  if (dtype == EMI_F32 && count >= 2 && !sum && K > 0 && M > 8 && (M + 31) / 32 <= 65535 && lda >= (trans_a ? M : K) &&
      ldb >= (trans_b ? K : N) && ldc >= N && (trans_a || lda % 4 == 0) && (!trans_b || ldb % 4 == 0) &&
      !(generic_splits(M, N, K) > 1 && (int64_t)count * ((M + 63) / 64) * ((N + 63) / 64) < 128)) {
    bool ok = true, any_r = false, all_r = true;
    for (int i = 0; i < count && ok; i++)
      ok = (trans_a || (reinterpret_cast<uintptr_t>(A[i]) & 15) == 0) && (!trans_b || (reinterpret_cast<uintptr_t>(B[i]) & 15) == 0);
    for (int i = 0; i < count; i++) {
      const bool has = R != nullptr && R[i] != nullptr;
      any_r = any_r || has;
      all_r = all_r && has;
    }
    if (ok && (!any_r || (all_r && ldr >= N))) {
      // the fp32 kernel, one grid plane per product
      GemmGroup g{};
      g.count = count;
      for (int i = 0; i < count; i++) {
        g.A[i] = static_cast<const uint16_t*>(A[i]);
        g.B[i] = static_cast<const uint16_t*>(B[i]);
        g.R[i] = any_r ? static_cast<const uint16_t*>(R[i]) : nullptr;
        g.C[i] = static_cast<uint16_t*>(C[i]);
      }
      const dim3 grid((unsigned)((N + 31) / 32), (unsigned)((M + 31) / 32), (unsigned)count);
#define EMI_F32_GROUPED_V(AKM, BKM, NWV, UV, ONCEV)                                                                        \
  hipLaunchKernelGGL((gemm_f32_small_kernel<AKM, BKM, true, NWV, UV, ONCEV>), grid, dim3(NWV * 64), 0, st,                 \
                     static_cast<const float*>(A[0]), static_cast<const float*>(B[0]), static_cast<const float*>(nullptr), \
                     static_cast<float*>(C[0]), (int)M, (int)N, (int)K, lda, ldb, ldr, ldc, g)
      const bool few = (int64_t)grid.x * grid.y * grid.z <= 1024;
#define EMI_F32_GROUPED(AKM, BKM)                                          \
  do {                                                                     \
    if (few && K <= 384) EMI_F32_GROUPED_V(AKM, BKM, 4, 12, true);         \
    else if (few && K <= 768) EMI_F32_GROUPED_V(AKM, BKM, 8, 12, true);    \
    else EMI_F32_GROUPED_V(AKM, BKM, 4, 4, false);                         \
  } while (0)
      if (!trans_a && trans_b) EMI_F32_GROUPED(false, false);
      else if (!trans_a && !trans_b) EMI_F32_GROUPED(false, true);
      else if (trans_a && !trans_b) EMI_F32_GROUPED(true, true);
      else EMI_F32_GROUPED(true, false);
#undef EMI_F32_GROUPED
#undef EMI_F32_GROUPED_V
      EMI_CHECK_LAUNCH("emi_gemm_grouped(fp32)");
      return EMI_OK;
    }
  }
  // one product after the other; summed: each launch adds onto the result of the one before
  for (int i = 0; i < count; i++) {
    const void* r = sum ? (i == 0 ? (R ? R[0] : nullptr) : C[0]) : (R ? R[i] : nullptr);
    void* c = sum ? C[0] : C[i];
    const int rc = emi_gemm_ws(stream, A[i], B[i], r, c, workspace, workspace_bytes, M, N, K, lda, ldb, (sum && i > 0) ? ldc : ldr, ldc,
                               trans_a, trans_b, dtype);
    if (rc != EMI_OK) return rc;
  }
  return EMI_OK;
}
