/* emi.h - C ABI of the MI355X (gfx950) llama forward + reverse-mode kernels.
 *
 * Boundary: these entry points are what an XLA custom-call handler for the
 * llama path binds.  The reference hands its optimized StableHLO to XLA's own
 * code generator (src/enzyme_ad/jax/primitives.py:626-692) and its only native
 * handlers are the typed-FFI cuBLAS wrappers (src/enzyme_ad/jax/xla_ffi/cuda/
 * blas.cc:286-313) and the kernel_call bundle (src/enzyme_ad/jax/gpu.cc:35-173);
 * each function below cites the reference item whose arithmetic it replaces.
 *
 * Conventions
 *  - plain pointers and sizes only; every pointer is DEVICE memory unless said
 *    otherwise; `stream` is a hipStream_t passed as void* (NULL = default stream);
 *  - work is enqueued on `stream`, no host synchronisation, no allocation;
 *    scratch space is an explicit `workspace` argument sized by the matching
 *    `*_workspace_bytes` query (the reference passes scratch as an extra
 *    result buffer, primitives.py:712-727);
 *  - row-major tensors, innermost dimension contiguous;
 *  - `dtype` is an XLA PrimitiveType code: EMI_F32 (11) or EMI_BF16 (16); all
 *    reductions, softmax statistics and GEMM accumulators are fp32;
 *  - return value 0 = success, otherwise an absl/XLA status code
 *    (EMI_INVALID_ARGUMENT = 3, EMI_UNIMPLEMENTED = 12, EMI_INTERNAL = 13) and a
 *    message retrievable with emi_last_error(); nothing is launched on error
 *    and nothing ever aborts or throws across this boundary.
 */
#ifndef EMI_H_
#define EMI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* emi_stream_t;

enum { EMI_F32 = 11, EMI_BF16 = 16 };
enum { EMI_OK = 0, EMI_INVALID_ARGUMENT = 3, EMI_UNIMPLEMENTED = 12, EMI_INTERNAL = 13 };

#define EMI_ABI_VERSION 1

/* ABI version of the loaded library (EMI_ABI_VERSION at build time). */
int emi_abi_version(void);
/* Message of the last failing call on this thread ("" if none). Host pointer. */
const char* emi_last_error(void);

/* RMSNorm forward: y = gamma * x * rsqrt(mean(x^2) + eps) over the last dim.
 * Replaces rmsnorm() of test/llama.py:6-10.  x,y: [rows, dim]; gamma: [dim]. */
int emi_rmsnorm_fwd(emi_stream_t stream, const void* x, const void* gamma, void* y,
                    int64_t rows, int64_t dim, float eps, int dtype);

/* RMSNorm adjoint (recomputes rstd from x, like the reference's combined
 * reverse program): dx = [dx_add +] r*g - x*r^3*mean(g*x), g = dy*gamma;
 * dgamma = sum_rows dy*x*r.  Replaces the Mul/Div/Sqrt/DotGeneral/Reduce
 * rules of HLODerivatives.td:1221,1133,1320,1166 applied to llama.py:6-10.
 * dx_add (nullable): residual-stream cotangent added into dx (Add rule, :964).
 * dgamma: [dim] in `dtype`.  workspace: emi_rmsnorm_bwd_workspace_bytes(). */
size_t emi_rmsnorm_bwd_workspace_bytes(int64_t rows, int64_t dim);
int emi_rmsnorm_bwd(emi_stream_t stream, const void* x, const void* gamma, const void* dy,
                    const void* dx_add, void* dx, void* dgamma, void* workspace,
                    size_t workspace_bytes, int64_t rows, int64_t dim, float eps, int dtype);

/* emi_rmsnorm_bwd without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid it).  No counterpart in the reference.  The dgamma
 * partial rows go to an array of EMI_RMSNORM_BWD_NOALLOC_MAX_BYTES that the library holds on every device it
 * has been called on, until the process ends; the call allocates and frees nothing (its first call on a device
 * looks the array's address up).  Fails with EMI_INVALID_ARGUMENT when emi_rmsnorm_bwd_workspace_bytes(rows, dim)
 * exceeds the array (any row count with dim <= 8192 and a multiple of 8 fits).  All calls on one device share
 * the array: calls that overlap on one device (two streams, two threads) race; serialise them. */
#define EMI_RMSNORM_BWD_NOALLOC_MAX_BYTES ((size_t)(512 + 1) * 8192 * 4)
int emi_rmsnorm_bwd_noalloc(emi_stream_t stream, const void* x, const void* gamma, const void* dy,
                            const void* dx_add, void* dx, void* dgamma, int64_t rows, int64_t dim,
                            float eps, int dtype);

/* RoPE angle table: table[s][j] = (cos, sin)(pos * theta^(-2j/head_dim)),
 * pos = pos0 + s, computed in float64 and rounded to fp32.  In the reference
 * these are trace-time constants (test/llama.py:127-140).
 * table: float[seq, head_dim/2, 2]. */
int emi_rope_table(emi_stream_t stream, float* table, int64_t seq, int64_t head_dim,
                   double theta, int64_t pos0);

/* RoPE apply: rotate adjacent pairs (2p, 2p+1) of every head by +angle, or by
 * -angle when inverse != 0 (the adjoint).  Replaces the einsum of
 * test/llama.py:161-168 and its DotGeneral adjoint (HLODerivatives.td:1166).
 * x,y: [batch, seq, heads, head_dim] contiguous; y may alias x. */
int emi_rope(emi_stream_t stream, const void* x, const float* table, void* y, int64_t batch,
             int64_t seq, int64_t heads, int64_t head_dim, int inverse, int dtype);

/* SwiGLU forward g = a * sigmoid(a) * b and adjoint
 * da = dg*b*s*(1 + a*(1-s)), db = dg*a*s.  Replaces silu()/sigmoid() of
 * test/llama.py:21-28,229-231 and the Neg/Exp/Add/Div/Mul rules.  n elements. */
int emi_swiglu_fwd(emi_stream_t stream, const void* a, const void* b, void* g, int64_t n, int dtype);
int emi_swiglu_bwd(emi_stream_t stream, const void* a, const void* b, const void* dg, void* da,
                   void* db, int64_t n, int dtype);

/* Elementwise y = a + b (residual add / cotangent fan-in, Add rule
 * HLODerivatives.td:964; test/llama.py:215,233).  y may alias a or b. */
int emi_add(emi_stream_t stream, const void* a, const void* b, void* y, int64_t n, int dtype);

/* out[cols, rows] = in[rows, cols]^T (Transpose rule HLODerivatives.td:1334: the adjoint
 * dots of the DotGeneral rule :1166-1178 contract over the outer index of their
 * row-major operands; transposing first puts the contraction index innermost).
 * `out` must not alias `in`. */
int emi_transpose(emi_stream_t stream, const void* in, void* out, int64_t rows, int64_t cols, int dtype);

/* GEMM: C[M,N] = op(A) . op(B) [+ R], fp32 accumulate, result rounded once.
 *   trans_a == 0: A is [M,K] (lda >= K);  trans_a != 0: A is [K,M] (lda >= M)
 *   trans_b == 0: B is [K,N] (ldb >= N);  trans_b != 0: B is [N,K] (ldb >= K)
 * Replaces the dot_general projections of test/llama.py:149-157,211,224-233
 * (Y = X.W^T: trans_a=0, trans_b=1) and their adjoints from the DotGeneral
 * rule HLODerivatives.td:1166-1178 (dX = dY.W: 0,0;  dW = dY^T.X: 1,0).
 * R (nullable, [M,N], ldr): added in the epilogue (residual add / fan-in sum).
 * C may alias R.  Leading dimensions in elements. */
int emi_gemm(emi_stream_t stream, const void* A, const void* B, const void* R, void* C,
             int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldr, int64_t ldc,
             int trans_a, int trans_b, int dtype);

/* The same with an optional scratch buffer of emi_gemm_workspace_bytes() bytes (0
 * for shapes that need none).  With it, the single-token adjoint dX = dY.W
 * (trans_a = trans_b = 0, M <= 8) sums row bands of W in many blocks (about 3x
 * faster), and products with few output tiles and a long contraction split K
 * over more blocks, each leaving an fp32 partial [M,N] plane: the weight
 * gradients of a small model on the 128x128 kernel, and in the bf16
 * Y = X.W^T form the shapes with more than 128 tiles of 128x128 but fewer than
 * 192 of 256x256 and K >= 8192 (the classifier adjoint [8192,32000].[32000,768]
 * of a 110M model) on the 256x256 kernel.  The planes are added in a fixed
 * order, with R, before the single rounding.  Without the buffer, or for any
 * other shape, the call is emi_gemm. */
size_t emi_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int trans_a, int trans_b, int dtype);
int emi_gemm_ws(emi_stream_t stream, const void* A, const void* B, const void* R, void* C,
                void* workspace, size_t workspace_bytes, int64_t M, int64_t N, int64_t K,
                int64_t lda, int64_t ldb, int64_t ldr, int64_t ldc, int trans_a, int trans_b,
                int dtype);

/* Up to EMI_GEMM_GROUP_MAX products of one shape in one launch: the q, k and v projections of one activation (test/llama.py:149-157),
 * w1 and w3 (:224-227), the weight gradients of such a group, and -- with `sum` -- the fan-in of their input gradients,
 * dX = sum_i dY_i . W_i (the DotGeneral rule HLODerivatives.td:1166-1178 followed by the additions of the Add rule :964).
 * A, B, R, C: tables of `count` pointers (R null, or one entry per result, all set or all null).
 *   sum == 0:  C[i] = op(A[i]) . op(B[i]) [+ R[i]]            (entries may repeat: one X against three weights)
 *   sum == 1:  C[0] = sum_i op(A[i]) . op(B[i]) [+ R[0]]      (products added in index order)
 * Shapes, leading dimensions and flags as for emi_gemm, the same for every product.  Small aligned bf16 products run
 * as one launch of the 128x128 kernel; anything else runs as `count` emi_gemm_ws calls with the same results up to the
 * rounding of the intermediate sums (sum == 1 then rounds C[0] to its type between products).  The workspace (size
 * from emi_gemm_grouped_workspace_bytes, may be null) holds split-K partials. */
#define EMI_GEMM_GROUP_MAX 48
size_t emi_gemm_grouped_workspace_bytes(int count, int64_t M, int64_t N, int64_t K, int trans_a, int trans_b, int sum,
                                        int dtype);
int emi_gemm_grouped(emi_stream_t stream, int count, const void* const* A, const void* const* B, const void* const* R,
                     void* const* C, void* workspace, size_t workspace_bytes, int64_t M, int64_t N, int64_t K, int64_t lda,
                     int64_t ldb, int64_t ldr, int64_t ldc, int trans_a, int trans_b, int sum, int dtype);

/* The SwiGLU of the FFN (test/llama.py:224-231: hb = w1 @ xb; hb2 = w3 @ xb; hb = hb * sigmoid(hb) * hb2) applied in the
 * epilogue of the product next to it, so that the elementwise pass over [tokens, hidden] disappears; same results as
 * the product followed by emi_swiglu_fwd / emi_swiglu_bwd (the product is rounded to its type before the elementwise
 * arithmetic, as it is when it goes through memory).  All matrices contiguous.
 *   emi_gemm_swiglu_fwd:  B_out[M, N] = X[M, K] . W3[N, K]^T ;  G_out = A * sigmoid(A) * B_out   (A = X . W1^T, given)
 *   emi_gemm_swiglu_bwd:  dG = dY[M, K] . W2T[N, K]^T (never stored) ;  (dA, dB) = adjoint of SwiGLU at (A, B) on dG
 *                         (W2T = the transposed down projection, [hidden, dim]; Mul / Div / Exp rules
 *                         HLODerivatives.td:1221,1133,1182 behind the DotGeneral rule :1166-1178)
 * bf16 products of whole 256 x 256 tiles (M, N multiples of 256, at least 192 tiles, 16-byte aligned buffers) run as
 * one launch; anything else as the product followed by the elementwise kernel, for which emi_gemm_swiglu_bwd needs a
 * workspace of emi_gemm_swiglu_bwd_workspace_bytes (dG) and fails without it. */
int emi_gemm_swiglu_fwd(emi_stream_t stream, const void* X, const void* W3, const void* A, void* B_out, void* G_out, int64_t M,
                        int64_t N, int64_t K, int dtype);
size_t emi_gemm_swiglu_bwd_workspace_bytes(int64_t M, int64_t N, int64_t K, int dtype);
int emi_gemm_swiglu_bwd(emi_stream_t stream, const void* dY, const void* W2T, const void* A, const void* B, void* dA, void* dB,
                        void* workspace, size_t workspace_bytes, int64_t M, int64_t N, int64_t K, int dtype);

/* A projection with RoPE in its epilogue (test/llama.py:149-157 followed by :161-168 for q and k):
 * Y[M, N] = rope(X[M, K] . W[N, K]^T), all contiguous.  Rows are tokens, `seq` consecutive rows one sequence (M a
 * multiple of seq), columns are heads of `head_dim`; rope_table as emi_rope_table writes it ([seq, head_dim/2] of
 * (cos, sin)).  The product is rotated in fp32 and rounded once.  bf16 products of whole 256 x 256 tiles (M, N
 * multiples of 256, at least 192 tiles, head_dim a multiple of 4) run as one launch; anything else as emi_gemm
 * followed by emi_rope in place. */
int emi_gemm_rope(emi_stream_t stream, const void* X, const void* W, void* Y, const float* rope_table, int64_t M, int64_t N,
                  int64_t K, int64_t seq, int64_t head_dim, int dtype);

/* Causal softmax attention, forward.  Replaces the per-head loop of
 * test/llama.py:178-206 with softmax of :13-18 (scale applied after the dot,
 * max-subtracted, fp32 statistics).  Element (b, h, s, i) of q/k/v/o lives at
 * b*stride_b + h*stride_h + s*stride_s + i.  lse: float[batch, heads, seq]
 * = log-sum-exp of the scaled scores (saved for the adjoint). */
int emi_attn_fwd(emi_stream_t stream, const void* q, const void* k, const void* v, void* o,
                 float* lse, int64_t batch, int64_t heads, int64_t seq, int64_t head_dim,
                 int64_t stride_b, int64_t stride_h, int64_t stride_s, float scale, int causal,
                 int dtype);

/* The same with a scratch argument, kept for callers that pass one: the forward
 * kernels need no scratch (V is transposed by the LDS reads inside the kernel; a
 * separate V^T pass cost more than it saved), emi_attn_fwd_workspace_bytes() returns 0
 * and `workspace` may be null. */
size_t emi_attn_fwd_workspace_bytes(int64_t batch, int64_t heads, int64_t seq, int64_t head_dim);
int emi_attn_fwd_ws(emi_stream_t stream, const void* q, const void* k, const void* v, void* o,
                    float* lse, void* workspace, size_t workspace_bytes, int64_t batch,
                    int64_t heads, int64_t seq, int64_t head_dim, int64_t stride_b,
                    int64_t stride_h, int64_t stride_s, float scale, int causal, int dtype);

/* Attention adjoint: dV = P^T dO, dP = dO V^T, dS = P*(dP - rowsum(dO*O)),
 * dQ = dS K scale, dK = dS^T Q scale; P is recomputed from q, k and lse.
 * Rules: Exp :1182, Div :1133, Sub :1312, Reduce(max/add)
 * StableHLOAutoDiffOpInterfaceImpl.cpp:1833-1916, DotGeneral :1166.
 * All of q,k,v,o,dO,dq,dk,dv share the strides. */
size_t emi_attn_bwd_workspace_bytes(int64_t batch, int64_t heads, int64_t seq, int64_t head_dim);
int emi_attn_bwd(emi_stream_t stream, const void* q, const void* k, const void* v, const void* o,
                 const float* lse, const void* d_o, void* dq, void* dk, void* dv, void* workspace,
                 size_t workspace_bytes, int64_t batch, int64_t heads, int64_t seq,
                 int64_t head_dim, int64_t stride_b, int64_t stride_h, int64_t stride_s,
                 float scale, int causal, int dtype);

/* emi_attn_bwd for q and k that are RoPE outputs (test/llama.py:161-168 in front of :178-206): dq and dk are the
 * cotangents of the vectors BEFORE the rotation, i.e. emi_attn_bwd followed by emi_rope(inverse) on dq and dk, with
 * the rotation applied as the MFMA kernels (bf16, head_dim 64 or 128) store their results, in fp32 before the one
 * rounding.  Other shapes run emi_attn_bwd and two emi_rope passes in place and need contiguous
 * [batch, seq, heads, head_dim] operands.  rope_table: [seq, head_dim/2] of (cos, sin), 16-byte aligned. */
int emi_attn_bwd_rope(emi_stream_t stream, const void* q, const void* k, const void* v, const void* o, const float* lse,
                      const void* d_o, void* dq, void* dk, void* dv, const float* rope_table, void* workspace,
                      size_t workspace_bytes, int64_t batch, int64_t heads, int64_t seq, int64_t head_dim, int64_t stride_b,
                      int64_t stride_h, int64_t stride_s, float scale, int causal, int dtype);

/* Attention of the single-token step exactly as the reference writes it
 * (test/llama.py:178-206, softmax :13-18): one query per (batch, head) against
 * the seq_kv rows of that head's key / value cache (the cache already holds the
 * row of the current token, :170-175).  Element (b, h, i) of q / o / dO / dq
 * lives at b*q_stride_b + h*q_stride_h + i; element (b, h, s, i) of k / v / dk /
 * dv at b*kv_stride_b + h*kv_stride_h + s*kv_stride_s + i.  lse: float[batch,
 * heads].  The adjoint (rules as for emi_attn_bwd) returns the cotangent of
 * every cache row.  The keys of a head are split over several blocks whose
 * partial results meet in `workspace` (emi_attn_step_workspace_bytes, the same
 * size forward and backward).  Query heads and key/value heads are equal in
 * number, as in the reference (:162,171). */
size_t emi_attn_step_workspace_bytes(int64_t batch, int64_t heads, int64_t seq_kv, int64_t head_dim);
int emi_attn_step_fwd(emi_stream_t stream, const void* q, const void* k, const void* v, void* o,
                      float* lse, void* workspace, size_t workspace_bytes, int64_t batch,
                      int64_t heads, int64_t seq_kv, int64_t head_dim, int64_t q_stride_b,
                      int64_t q_stride_h, int64_t kv_stride_b, int64_t kv_stride_h,
                      int64_t kv_stride_s, float scale, int dtype);
int emi_attn_step_bwd(emi_stream_t stream, const void* q, const void* k, const void* v,
                      const void* o, const float* lse, const void* d_o, void* dq, void* dk,
                      void* dv, void* workspace, size_t workspace_bytes, int64_t batch,
                      int64_t heads, int64_t seq_kv, int64_t head_dim, int64_t q_stride_b,
                      int64_t q_stride_h, int64_t kv_stride_b, int64_t kv_stride_h,
                      int64_t kv_stride_s, float scale, int dtype);

/* Forward mode (tangents), the other half of the reference API (enzyme_jvp,
 * src/enzyme_ad/jax/primitives.py:1147-1245).  Linear operators (emi_gemm, emi_rope,
 * emi_add, emi_embedding_fwd) carry tangents through their own forward entry
 * points; the three below are the nonlinear ones.  A null tangent pointer is a
 * zero tangent.
 *   rmsnorm:  ty = gamma (r tx - x r^3 mean(x tx)) + tgamma x r
 *   swiglu:   tg = ta b s (1 + a (1 - s)) + tb a s,  s = sigmoid(a)
 *   attention (strides and lse as emi_attn_fwd):
 *             tS = scale (tq k^T + q tk^T), tP = P (tS - rowsum(P tS)), to = tP v + P tv */
int emi_rmsnorm_jvp(emi_stream_t stream, const void* x, const void* gamma, const void* tx,
                    const void* tgamma, void* ty, int64_t rows, int64_t dim, float eps, int dtype);
int emi_swiglu_jvp(emi_stream_t stream, const void* a, const void* b, const void* ta,
                   const void* tb, void* tg, int64_t n, int dtype);
int emi_attn_jvp(emi_stream_t stream, const void* q, const void* k, const void* v, const float* lse,
                 const void* tq, const void* tk, const void* tv, void* to, int64_t batch,
                 int64_t heads, int64_t seq, int64_t head_dim, int64_t stride_b, int64_t stride_h,
                 int64_t stride_s, float scale, int causal, int dtype);

/* Forward mode of the single-token attention (emi_attn_step_fwd's layout, o and lse from
 * it): to = sum_s p_s (tS_s v_s + tv_s) - (sum_s p_s tS_s) o with tS_s = scale (tq.k_s + q.tk_s).
 * Null tq / tk / tv = zero tangent.  workspace: emi_attn_step_workspace_bytes(). */
int emi_attn_step_jvp(emi_stream_t stream, const void* q, const void* k, const void* v, const void* o,
                      const float* lse, const void* tq, const void* tk, const void* tv, void* to,
                      void* workspace, size_t workspace_bytes, int64_t batch, int64_t heads,
                      int64_t seq_kv, int64_t head_dim, int64_t q_stride_b, int64_t q_stride_h,
                      int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, float scale,
                      int dtype);

/* ---- generic tensor operators -------------------------------------------
 * What is left of a StableHLO module that arrives as text (hlo_call,
 * src/enzyme_ad/jax/primitives.py:1052-1108; in the reference XLA's own code
 * generator compiles these operators) once the llama clusters have been
 * matched to the fused kernels above.  Operator codes: */
enum {
  /* binary: y = op(a, b) */
  EMI_OP_ADD = 0, EMI_OP_SUB, EMI_OP_MUL, EMI_OP_DIV, EMI_OP_MAX, EMI_OP_MIN,
  EMI_OP_GE,        /* 1.0 where a >= b else 0.0 (Max rule HLODerivatives.td:1205: ties go to a) */
  EMI_OP_EQ,        /* 1.0 where a == b else 0.0 (reduce-max rule, StableHLOAutoDiffOpInterfaceImpl.cpp:1881-1916) */
  EMI_OP_NMUL,      /* -(a * b) */
  EMI_OP_POW,
  /* binary derivative factors, a = incoming (co)tangent, b = the operator's saved value */
  EMI_OP_D_SQRT,     /* b = sqrt(x):     b == 0 ? 0 : a / (2 b)   (Sqrt rule :1320 with its zero guard) */
  EMI_OP_D_RSQRT,    /* b = rsqrt(x):    -a b^3 / 2               (Rsqrt rule :1283) */
  EMI_OP_D_LOGISTIC, /* b = logistic(x): a b (1 - b) */
  EMI_OP_D_TANH,     /* b = tanh(x):     a (1 - b^2) */
  EMI_OP_D_SIN,      /* b = x:           a cos(b) */
  EMI_OP_D_COS,      /* b = x:           -a sin(b) */
  /* factors of the Pow rule (HLODerivatives.td:1237-1242) on the operands themselves */
  EMI_OP_D_POW_A,    /* b pow(a, b - 1) */
  EMI_OP_D_POW_B,    /* pow(a, b) log(a) */
  /* further derivative factors (HLODerivatives.td: Abs :1244, Log1p :1201, Expm1 :1184, Cbrt :1085) */
  EMI_OP_D_ABS,      /* b = x:           b >= 0 ? a : -a */
  EMI_OP_D_LOG1P,    /* b = x:           a / (b + 1) */
  EMI_OP_D_EXPM1,    /* b = x:           a exp(b) */
  EMI_OP_D_CBRT,     /* b = cbrt(x):     a / (3 b^2) */
  EMI_OP_ATAN2,      /* atan2(a, b): the angle of the point (b, a) */
  /* unary: y = op(x) */
  EMI_OP_NEG = 32, EMI_OP_EXP, EMI_OP_LOG, EMI_OP_SQRT, EMI_OP_RSQRT, EMI_OP_LOGISTIC, EMI_OP_TANH,
  EMI_OP_SIN, EMI_OP_COS, EMI_OP_ABS, EMI_OP_COPY, EMI_OP_LOG1P, EMI_OP_EXPM1, EMI_OP_CBRT
};

/* y[i] = op(a[i], b[i]) for i < n, computed in fp32.  An operand flagged
 * *_is_scalar is a single element broadcast to all i (a folded
 * broadcast_in_dim of a rank-0 tensor).  y must not overlap a or b. */
int emi_map_binary(emi_stream_t stream, int op, const void* a, const void* b, void* y, int64_t n,
                   int a_is_scalar, int b_is_scalar, int dtype);
/* y[i] = op(x[i]).  y must not overlap x. */
int emi_map_unary(emi_stream_t stream, int op, const void* x, void* y, int64_t n, int dtype);
/* stablehlo.convert between EMI_F32 and EMI_BF16 (round to nearest even). */
int emi_convert(emi_stream_t stream, const void* x, void* y, int64_t n, int from_dtype, int to_dtype);
/* stablehlo.compare on floating-point operands: mask[i] = direction(a[i], b[i]) as one byte
 * (0 or 1, the storage of an i1 tensor); stablehlo.select: y[i] = mask[i] ? a[i] : b[i]
 * (Select rule HLODerivatives.td:1297; the guards of the Sqrt :1320 and Max :1205 rules are
 * selects on compares).  *_is_scalar operands are one element broadcast to all i. */
enum { EMI_CMP_EQ = 0, EMI_CMP_NE, EMI_CMP_GE, EMI_CMP_GT, EMI_CMP_LE, EMI_CMP_LT };
int emi_compare(emi_stream_t stream, int direction, const void* a, const void* b, void* mask, int64_t n,
                int a_is_scalar, int b_is_scalar, int dtype);
int emi_select(emi_stream_t stream, const void* mask, const void* a, const void* b, void* y, int64_t n,
               int mask_is_scalar, int a_is_scalar, int b_is_scalar, int dtype);
/* out[out_offset + sum_d i_d out_strides[d]] = in[in_offset + sum_d i_d in_strides[d]] for every
 * index 0 <= i_d < dims[d]: transpose (permuted strides), broadcast_in_dim
 * (zero in_strides), slice (offset and strides; Slice rule
 * StableHLOAutoDiffOpInterfaceImpl.cpp:1586-1620) and one operand of
 * concatenate (Concatenate rule :2015-2059).  rank <= 8; strides and offsets in
 * elements of elem_bytes (1, 2, 4 or 8) bytes; dims / strides are HOST arrays.
 * The boxes must not overlap. */
int emi_strided_copy(emi_stream_t stream, const void* in, void* out, int rank, const int64_t* dims,
                     const int64_t* in_strides, int64_t in_offset, const int64_t* out_strides,
                     int64_t out_offset, int elem_bytes);
/* y[o, i] = sum or max over r of x[o, r, i] (op = EMI_OP_ADD or EMI_OP_MAX), fp32
 * accumulation (stablehlo.reduce with an add / maximum body; Reduce rule
 * StableHLOAutoDiffOpInterfaceImpl.cpp:1833-1916).  x: [outer, red, inner] contiguous.
 * Shapes with few results and long reductions run in two stages through fp32
 * partials in `workspace` (emi_reduce_workspace_bytes(); 0 when one stage is used);
 * with a null or short workspace the single-stage kernel runs (same result, slower).
 * outer <= 65535 when inner > 1. */
size_t emi_reduce_workspace_bytes(int64_t outer, int64_t red, int64_t inner, int dtype);
int emi_reduce(emi_stream_t stream, int op, const void* x, void* y, void* workspace,
               size_t workspace_bytes, int64_t outer, int64_t red, int64_t inner, int dtype);

/* Embedding gather x[t,:] = table[tokens[t],:] and its adjoint (scatter-add of
 * dx rows into a zero-initialised dtable; fp32 accumulation in workspace when
 * dtype is bf16).  The lookup is commented out in the reference
 * (test/llama.py:109-113); adjoint per HLODerivatives.td:1022-1046.
 * tokens: int32[n_tokens]. */
int emi_embedding_fwd(emi_stream_t stream, const int32_t* tokens, const void* table, void* x,
                      int64_t n_tokens, int64_t vocab, int64_t dim, int dtype);
size_t emi_embedding_bwd_workspace_bytes(int64_t vocab, int64_t dim, int dtype);
int emi_embedding_bwd(emi_stream_t stream, const int32_t* tokens, const void* dx, void* dtable,
                      void* workspace, size_t workspace_bytes, int64_t n_tokens, int64_t vocab,
                      int64_t dim, int dtype);

/* Softmax cross-entropy of logits[tokens, vocab] against integer targets, the loss
 * that follows the classifier (the classifier is commented out at test/llama.py:236;
 * the reference's llama test stops at the final RMSNorm, so this operator has no
 * reference call site: its definition is the standard one, per token
 *   loss = logsumexp(z) - z[target]).
 * fwd writes loss and lse (both f32[tokens]); bwd writes
 *   dlogits = (exp(z - lse) - onehot(target)) * dloss      (dloss f32[tokens], dlogits in dtype);
 * jvp writes tloss = sum_v exp(z_v - lse) tz_v - tz[target] (f32[tokens]).
 * A token whose target lies outside [0, vocab) is masked: zero loss, gradient and
 * tangent.  targets: int32[tokens]; vocab <= 2^24.  Rows that are not whole 16-byte
 * chunks (vocab % 8 for bf16, % 4 for f32) take a scalar path. */
int emi_cross_entropy_fwd(emi_stream_t stream, const void* logits, const int32_t* targets, float* loss,
                          float* lse, int64_t tokens, int64_t vocab, int dtype);
int emi_cross_entropy_bwd(emi_stream_t stream, const void* logits, const int32_t* targets,
                          const float* lse, const float* dloss, void* dlogits, int64_t tokens,
                          int64_t vocab, int dtype);
int emi_cross_entropy_jvp(emi_stream_t stream, const void* logits, const int32_t* targets,
                          const float* lse, const void* tlogits, float* tloss, int64_t tokens,
                          int64_t vocab, int dtype);

#ifdef __cplusplus
}
#endif
#endif /* EMI_H_ */
