/* emi_ffi.h - XLA typed-FFI entry points of the MI355X llama kernels.
 *
 * These are the symbols a JAX/XLA process binds for platform "ROCM": one
 * `XLA_FFI_Error* handler(XLA_FFI_CallFrame*)` per custom-call target, in the
 * style of the reference's own handlers (execute-stage handler answering the
 * metadata-extension probe, src/enzyme_ad/jax/gpu.cc:95-156; typed handlers
 * registered per platform, src/enzyme_ad/jax/xla_ffi/cuda/blas.cc:481-492;
 * one registration call guarded by a once-flag, xla_ffi/register.cc:21-27).
 * Each handler validates dtypes, ranks and dimensions of the call frame, takes
 * the stream from the execution context and forwards to the plain launcher of
 * the same name in emi.h.  On any mismatch it returns an error created through
 * the API table (INVALID_ARGUMENT) and launches nothing.
 *
 * Wire format (stablehlo.custom_call, api_version = 4, attributes in the
 * `backend_config` dictionary, as emitted by the reference at
 * Passes/LowerEnzymeXLABLAS.cpp:463-479):
 *
 *  target             operands                         results                           attributes
 *  emi_rmsnorm_fwd    x[..,D], gamma[D]                y[..,D]                           eps:f32
 *  emi_rmsnorm_bwd    x, gamma, dy [, dx_add]          dx, dgamma[D], workspace:u8[n]    eps:f32
 *  emi_rope_table     -                                table f32[S, d/2, 2]              theta:f32|f64, pos0:s64
 *  emi_rope           x[B,S,h,d], table                y[B,S,h,d]                        inverse:pred
 *  emi_swiglu_fwd     a, b                             g                                 -
 *  emi_swiglu_bwd     a, b, dg                         da, db                            -
 *  emi_add            a, b                             y                                 -
 *  emi_gemm           A[.,.], B[.,.] [, R[M,N]]        C[M,N] [, workspace:u8[n]]        trans_a:pred, trans_b:pred
 *  emi_gemm_grouped   A0..An-1, B0..Bn-1 [, R...]      C0..Cn-1 (C0 alone if sum) [, workspace:u8[n]]  count:i64 (2-4), sum:pred, trans_a:pred, trans_b:pred
 *  emi_gemm_swiglu_fwd  x[M,K], w3[N,K], a[M,N]       b[M,N] = x.w3^T, g[M,N] = a*sigmoid(a)*b   -
 *  emi_gemm_swiglu_bwd  dy[M,K], w2t[N,K], a, b[M,N]  da, db[M,N] [, workspace:u8[n]]          -
 *  emi_gemm_rope      x[M,K], w[N,K], table f32[S,d/2,2]  y[M,N] = rope(x.w^T)             -
 *  emi_attn_bwd_rope  q, k, v, o, lse, do, table       dq, dk (before RoPE), dv, workspace:u8[n]  scale:f32, causal:pred, bshd:pred
 *  emi_attn_fwd       q, k, v  (rank 4)                o, lse f32[B,h,S] [, unused:u8[n]]     scale:f32, causal:pred, bshd:pred
 *  emi_attn_bwd       q, k, v, o, lse, do              dq, dk, dv, workspace:u8[n]       scale:f32, causal:pred, bshd:pred
 *  emi_attn_step_fwd  q[B,h,d], k, v [B,S,h,d]         o[B,h,d], lse f32[B,h], workspace:u8[n]  scale:f32
 *  emi_attn_step_bwd  q, k, v, o, lse, do              dq, dk, dv, workspace:u8[n]       scale:f32
 *  emi_rmsnorm_jvp    x, gamma, tx, tgamma             ty                                eps:f32
 *  emi_swiglu_jvp     a, b, ta, tb                     tg                                -
 *  emi_attn_jvp       q, k, v, lse, tq, tk, tv         to                                scale:f32, causal:pred, bshd:pred
 *  emi_attn_step_jvp  q, k, v, o, lse, tq, tk, tv      to, workspace:u8[n]               scale:f32
 *  emi_embedding_fwd  tokens s32[..], table[V,D]       x[..,D]                           -
 *  emi_embedding_bwd  tokens s32[..], dx[..,D]         dtable[V,D] [, workspace:u8[n]]   -
 *  emi_cross_entropy_fwd  logits[..,V], targets s32[..]  loss f32[..], lse f32[..]         -
 *  emi_cross_entropy_bwd  logits, targets, lse, dloss f32[..]  dlogits[..,V]               -
 *  emi_cross_entropy_jvp  logits, targets, lse, tlogits  tloss f32[..]                     -
 *
 * `bshd` true: rank-4 operands are [batch, seq, heads, head_dim]; false:
 * [batch, heads, seq, head_dim].  Workspace results must be at least as large as
 * the matching emi_*_workspace_bytes() query; XLA owns every buffer.
 */
#ifndef EMI_FFI_H_
#define EMI_FFI_H_

#ifdef __cplusplus
extern "C" {
#endif

struct XLA_FFI_CallFrame;
struct XLA_FFI_Error;
struct XLA_FFI_Api;

struct XLA_FFI_Error* emi_rmsnorm_fwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_rmsnorm_bwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_rope_table_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_rope_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_swiglu_fwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_swiglu_bwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_add_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_gemm_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_gemm_grouped_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_gemm_swiglu_fwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_gemm_swiglu_bwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_gemm_rope_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_attn_bwd_rope_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_attn_fwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_attn_bwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_attn_step_fwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_attn_step_bwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_rmsnorm_jvp_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_swiglu_jvp_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_attn_jvp_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_attn_step_jvp_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_embedding_fwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_embedding_bwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_cross_entropy_fwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_cross_entropy_bwd_ffi(struct XLA_FFI_CallFrame*);
struct XLA_FFI_Error* emi_cross_entropy_jvp_ffi(struct XLA_FFI_CallFrame*);

/* Number of targets and the i-th (name, handler); for registration from Python
 * with jax.ffi.register_ffi_target(name, capsule(handler), platform="ROCM"). */
int emi_ffi_target_count(void);
const char* emi_ffi_target_name(int i);
void* emi_ffi_target_handler(int i);

/* Registers every target for platform "ROCM" through api->XLA_FFI_Handler_Register
 * (counterpart of registerEnzymeJaXXLAFFI, src/enzyme_ad/jax/xla_ffi/register.cc:21-27).
 * Runs once per process; returns 0 on success, an emi status code otherwise. */
int emi_register_ffi(const struct XLA_FFI_Api* api);

#ifdef __cplusplus
}
#endif
#endif /* EMI_FFI_H_ */
