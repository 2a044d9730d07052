// XLA typed-FFI handlers (platform "ROCM") over the plain launchers of emi.h.
// Host code only: decode and validate the call frame, fetch the stream, forward.
#include <mutex>
#include <stdio.h>
#include <string.h>

#include "../../include/emi.h"
#include "../../include/emi_ffi.h"
#include "xla_ffi_abi.h"

namespace {

struct Frame {
  XLA_FFI_CallFrame* cf;
  const char* target;
  char msg[384];

  XLA_FFI_Error* fail(XLA_FFI_Error_Code code, const char* text) {
    const XLA_FFI_Api* api = cf->api;
    if (api == nullptr || api->XLA_FFI_Error_Create == nullptr) return reinterpret_cast<XLA_FFI_Error*>(1);
    XLA_FFI_Error_Create_Args a;
    a.struct_size = sizeof(a);
    a.extension_start = nullptr;
    a.message = text;
    a.errc = code;
    return api->XLA_FFI_Error_Create(&a);
  }
  XLA_FFI_Error* invalid(const char* fmt, long long a = 0, long long b = 0, long long c = 0) {
    char body[300];
    snprintf(body, sizeof(body), fmt, a, b, c);
    snprintf(msg, sizeof(msg), "%s: %s", target, body);
    return fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, msg);
  }
  XLA_FFI_Error* from_status(int rc) {
    if (rc == EMI_OK) return nullptr;
    snprintf(msg, sizeof(msg), "%s", emi_last_error());
    return fail(rc == EMI_INVALID_ARGUMENT ? XLA_FFI_Error_Code_INVALID_ARGUMENT
                : rc == EMI_UNIMPLEMENTED  ? XLA_FFI_Error_Code_UNIMPLEMENTED
                                           : XLA_FFI_Error_Code_INTERNAL,
                msg);
  }

  const XLA_FFI_Buffer* arg(int i) const { return static_cast<const XLA_FFI_Buffer*>(cf->args.args[i]); }
  const XLA_FFI_Buffer* ret(int i) const { return static_cast<const XLA_FFI_Buffer*>(cf->rets.rets[i]); }

  // named scalar attribute (attrs are sorted by name, but a linear scan is fine)
  const XLA_FFI_Scalar* scalar(const char* name) const {
    const size_t n = strlen(name);
    for (int64_t i = 0; i < cf->attrs.size; i++) {
      const XLA_FFI_ByteSpan* nm = cf->attrs.names[i];
      if (nm && nm->len == n && memcmp(nm->ptr, name, n) == 0 && cf->attrs.types[i] == XLA_FFI_AttrType_SCALAR)
        return static_cast<const XLA_FFI_Scalar*>(cf->attrs.attrs[i]);
    }
    return nullptr;
  }
  bool get_f(const char* name, double* out) const {
    const XLA_FFI_Scalar* s = scalar(name);
    if (!s || !s->value) return false;
    if (s->dtype == XLA_FFI_DataType_F32) *out = *static_cast<const float*>(s->value);
    else if (s->dtype == XLA_FFI_DataType_F64) *out = *static_cast<const double*>(s->value);
    else return false;
    return true;
  }
  bool get_i(const char* name, int64_t* out) const {
    const XLA_FFI_Scalar* s = scalar(name);
    if (!s || !s->value) return false;
    switch (s->dtype) {
      case XLA_FFI_DataType_PRED: case XLA_FFI_DataType_U8: *out = *static_cast<const uint8_t*>(s->value); return true;
      case XLA_FFI_DataType_S32: *out = *static_cast<const int32_t*>(s->value); return true;
      case XLA_FFI_DataType_S64: *out = *static_cast<const int64_t*>(s->value); return true;
      default: return false;
    }
  }
};

// Answers the metadata probe and filters the non-execute stages.  Returns true
// when the handler should return `*out` immediately.
bool prologue(XLA_FFI_CallFrame* cf, XLA_FFI_Error** out) {
  *out = nullptr;
  if (cf == nullptr) {
    *out = reinterpret_cast<XLA_FFI_Error*>(1);
    return true;
  }
  if (cf->extension_start != nullptr && cf->extension_start->type == XLA_FFI_Extension_Metadata) {
    auto* ext = reinterpret_cast<XLA_FFI_Metadata_Extension*>(cf->extension_start);
    if (ext->metadata != nullptr) {
      XLA_FFI_Api_Version v;
      v.struct_size = sizeof(XLA_FFI_Api_Version);
      v.extension_start = nullptr;
      v.major_version = XLA_FFI_API_MAJOR;
      v.minor_version = XLA_FFI_API_MINOR;
      ext->metadata->api_version = v;
    }
    return true;
  }
  return cf->stage != XLA_FFI_ExecutionStage_EXECUTE;   // instantiate / prepare / initialize: nothing to do
}

XLA_FFI_Error* get_stream(Frame& f, void** stream) {
  const XLA_FFI_Api* api = f.cf->api;
  *stream = nullptr;
  if (api == nullptr) return f.invalid("call frame has no API table");
  if (api->struct_size < offsetof(XLA_FFI_Api, XLA_FFI_Stream_Get) + sizeof(void*) || api->XLA_FFI_Stream_Get == nullptr)
    return f.invalid("API table (struct_size %lld) has no XLA_FFI_Stream_Get", (long long)api->struct_size);
  XLA_FFI_Stream_Get_Args a;
  a.struct_size = sizeof(a);
  a.extension_start = nullptr;
  a.ctx = f.cf->ctx;
  a.stream = nullptr;
  if (XLA_FFI_Error* e = api->XLA_FFI_Stream_Get(&a)) return e;
  *stream = a.stream;
  return nullptr;
}

int64_t numel(const XLA_FFI_Buffer* b) {
  int64_t n = 1;
  for (int64_t i = 0; i < b->rank; i++) n *= b->dims[i];
  return n;
}
bool same_shape(const XLA_FFI_Buffer* a, const XLA_FFI_Buffer* b) {
  if (a->rank != b->rank) return false;
  for (int64_t i = 0; i < a->rank; i++)
    if (a->dims[i] != b->dims[i]) return false;
  return true;
}
bool is_float(const XLA_FFI_Buffer* b) { return b->dtype == XLA_FFI_DataType_F32 || b->dtype == XLA_FFI_DataType_BF16; }
size_t elem_size(XLA_FFI_DataType t) {
  switch (t) {
    case XLA_FFI_DataType_F32: case XLA_FFI_DataType_S32: case XLA_FFI_DataType_U32: return 4;
    case XLA_FFI_DataType_BF16: case XLA_FFI_DataType_F16: case XLA_FFI_DataType_S16: case XLA_FFI_DataType_U16: return 2;
    case XLA_FFI_DataType_F64: case XLA_FFI_DataType_S64: case XLA_FFI_DataType_U64: return 8;
    default: return 1;
  }
}
size_t byte_size(const XLA_FFI_Buffer* b) { return (size_t)numel(b) * elem_size(b->dtype); }

#define EMI_FFI_BEGIN(NAME, NARGS_MIN, NARGS_MAX, NRETS_MIN, NRETS_MAX)                                      \
  XLA_FFI_Error* early;                                                                                      \
  if (prologue(cf, &early)) return early;                                                                    \
  Frame f;                                                                                                   \
  f.cf = cf;                                                                                                 \
  f.target = NAME;                                                                                           \
  if (cf->args.size < (NARGS_MIN) || cf->args.size > (NARGS_MAX) || cf->rets.size < (NRETS_MIN) ||           \
      cf->rets.size > (NRETS_MAX))                                                                           \
    return f.invalid("expected %lld operand(s) and %lld result(s), got %lld operand(s)", NARGS_MIN, NRETS_MIN, \
                     (long long)cf->args.size);                                                              \
  for (int64_t i_ = 0; i_ < cf->args.size; i_++)                                                             \
    if (cf->args.args[i_] == nullptr || f.arg((int)i_)->data == nullptr) return f.invalid("operand %lld is null", i_); \
  for (int64_t i_ = 0; i_ < cf->rets.size; i_++)                                                             \
    if (cf->rets.rets[i_] == nullptr || f.ret((int)i_)->data == nullptr) return f.invalid("result %lld is null", i_);

#define EMI_FFI_STREAM()                                   \
  void* stream;                                            \
  if (XLA_FFI_Error* e_ = get_stream(f, &stream)) return e_;

}  // namespace

extern "C" XLA_FFI_Error* emi_rmsnorm_fwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_rmsnorm_fwd", 2, 2, 1, 1)
  const XLA_FFI_Buffer *x = f.arg(0), *g = f.arg(1), *y = f.ret(0);
  if (!is_float(x) || g->dtype != x->dtype || y->dtype != x->dtype)
    return f.invalid("x, gamma and y must share one dtype, f32 or bf16 (got codes %lld, %lld, %lld)", x->dtype, g->dtype, y->dtype);
  if (x->rank < 1 || g->rank != 1 || g->dims[0] != x->dims[x->rank - 1])
    return f.invalid("gamma must be rank 1 with the last dimension of x (x rank %lld, gamma rank %lld)", x->rank, g->rank);
  if (!same_shape(x, y)) return f.invalid("y must have the shape of x");
  double eps;
  if (!f.get_f("eps", &eps)) return f.invalid("missing f32/f64 attribute 'eps'");
  EMI_FFI_STREAM()
  const int64_t D = g->dims[0];
  return f.from_status(emi_rmsnorm_fwd(stream, x->data, g->data, y->data, D ? numel(x) / D : 0, D, (float)eps, x->dtype));
}

extern "C" XLA_FFI_Error* emi_rmsnorm_bwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_rmsnorm_bwd", 3, 4, 3, 3)
  const XLA_FFI_Buffer *x = f.arg(0), *g = f.arg(1), *dy = f.arg(2), *add = cf->args.size == 4 ? f.arg(3) : nullptr;
  const XLA_FFI_Buffer *dx = f.ret(0), *dg = f.ret(1), *ws = f.ret(2);
  if (!is_float(x) || g->dtype != x->dtype || dy->dtype != x->dtype || dx->dtype != x->dtype || dg->dtype != x->dtype ||
      (add && add->dtype != x->dtype))
    return f.invalid("all tensors must share one dtype, f32 or bf16 (x has code %lld)", x->dtype);
  if (x->rank < 1 || g->rank != 1 || g->dims[0] != x->dims[x->rank - 1])
    return f.invalid("gamma must be rank 1 with the last dimension of x (x rank %lld, gamma rank %lld)", x->rank, g->rank);
  if (!same_shape(x, dy) || !same_shape(x, dx) || !same_shape(g, dg) || (add && !same_shape(x, add)))
    return f.invalid("dy, dx (and dx_add) must have the shape of x, dgamma the shape of gamma");
  double eps;
  if (!f.get_f("eps", &eps)) return f.invalid("missing f32/f64 attribute 'eps'");
  const int64_t D = g->dims[0], rows = D ? numel(x) / D : 0;
  const size_t need = emi_rmsnorm_bwd_workspace_bytes(rows, D);
  if (byte_size(ws) < need) return f.invalid("workspace result has %lld bytes, %lld needed", (long long)byte_size(ws), (long long)need);
  EMI_FFI_STREAM()
  return f.from_status(emi_rmsnorm_bwd(stream, x->data, g->data, dy->data, add ? add->data : nullptr, dx->data, dg->data,
                                       ws->data, byte_size(ws), rows, D, (float)eps, x->dtype));
}

extern "C" XLA_FFI_Error* emi_rope_table_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_rope_table", 0, 0, 1, 1)
  const XLA_FFI_Buffer* t = f.ret(0);
  if (t->dtype != XLA_FFI_DataType_F32 || t->rank != 3 || t->dims[2] != 2)
    return f.invalid("table must be f32[seq, head_dim/2, 2] (rank %lld)", t->rank);
  double theta;
  int64_t pos0 = 0;
  if (!f.get_f("theta", &theta)) return f.invalid("missing f32/f64 attribute 'theta'");
  f.get_i("pos0", &pos0);
  EMI_FFI_STREAM()
  return f.from_status(emi_rope_table(stream, static_cast<float*>(t->data), t->dims[0], t->dims[1] * 2, theta, pos0));
}

extern "C" XLA_FFI_Error* emi_rope_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_rope", 2, 2, 1, 1)
  const XLA_FFI_Buffer *x = f.arg(0), *t = f.arg(1), *y = f.ret(0);
  if (!is_float(x) || y->dtype != x->dtype) return f.invalid("x and y must share one dtype, f32 or bf16 (code %lld)", x->dtype);
  if (x->rank != 4 || !same_shape(x, y)) return f.invalid("x and y must be [batch, seq, heads, head_dim] (rank %lld)", x->rank);
  if (t->dtype != XLA_FFI_DataType_F32 || t->rank != 3 || t->dims[0] != x->dims[1] || t->dims[1] * 2 != x->dims[3] || t->dims[2] != 2)
    return f.invalid("table must be f32[seq, head_dim/2, 2] matching x (table rank %lld)", t->rank);
  int64_t inverse = 0;
  f.get_i("inverse", &inverse);
  EMI_FFI_STREAM()
  return f.from_status(emi_rope(stream, x->data, static_cast<const float*>(t->data), y->data, x->dims[0], x->dims[1],
                                x->dims[2], x->dims[3], (int)inverse, x->dtype));
}

extern "C" XLA_FFI_Error* emi_swiglu_fwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_swiglu_fwd", 2, 2, 1, 1)
  const XLA_FFI_Buffer *a = f.arg(0), *b = f.arg(1), *g = f.ret(0);
  if (!is_float(a) || b->dtype != a->dtype || g->dtype != a->dtype) return f.invalid("a, b, g must share one dtype, f32 or bf16 (code %lld)", a->dtype);
  if (!same_shape(a, b) || !same_shape(a, g)) return f.invalid("a, b and g must have one shape");
  EMI_FFI_STREAM()
  return f.from_status(emi_swiglu_fwd(stream, a->data, b->data, g->data, numel(a), a->dtype));
}

extern "C" XLA_FFI_Error* emi_swiglu_bwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_swiglu_bwd", 3, 3, 2, 2)
  const XLA_FFI_Buffer *a = f.arg(0), *b = f.arg(1), *dg = f.arg(2), *da = f.ret(0), *db = f.ret(1);
  if (!is_float(a) || b->dtype != a->dtype || dg->dtype != a->dtype || da->dtype != a->dtype || db->dtype != a->dtype)
    return f.invalid("all tensors must share one dtype, f32 or bf16 (code %lld)", a->dtype);
  if (!same_shape(a, b) || !same_shape(a, dg) || !same_shape(a, da) || !same_shape(a, db)) return f.invalid("all tensors must have one shape");
  EMI_FFI_STREAM()
  return f.from_status(emi_swiglu_bwd(stream, a->data, b->data, dg->data, da->data, db->data, numel(a), a->dtype));
}

extern "C" XLA_FFI_Error* emi_add_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_add", 2, 2, 1, 1)
  const XLA_FFI_Buffer *a = f.arg(0), *b = f.arg(1), *y = f.ret(0);
  if (!is_float(a) || b->dtype != a->dtype || y->dtype != a->dtype) return f.invalid("a, b, y must share one dtype, f32 or bf16 (code %lld)", a->dtype);
  if (!same_shape(a, b) || !same_shape(a, y)) return f.invalid("a, b and y must have one shape");
  EMI_FFI_STREAM()
  return f.from_status(emi_add(stream, a->data, b->data, y->data, numel(a), a->dtype));
}

extern "C" XLA_FFI_Error* emi_gemm_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_gemm", 2, 3, 1, 2)
  const XLA_FFI_Buffer *A = f.arg(0), *B = f.arg(1), *R = cf->args.size == 3 ? f.arg(2) : nullptr, *C = f.ret(0);
  const XLA_FFI_Buffer* ws = cf->rets.size == 2 ? f.ret(1) : nullptr;      // optional scratch (emi_gemm_workspace_bytes)
  if (!is_float(A) || B->dtype != A->dtype || C->dtype != A->dtype || (R && R->dtype != A->dtype))
    return f.invalid("A, B, C (and R) must share one dtype, f32 or bf16 (code %lld)", A->dtype);
  if (A->rank != 2 || B->rank != 2 || C->rank != 2 || (R && R->rank != 2)) return f.invalid("operands must be rank 2 (A rank %lld, B rank %lld)", A->rank, B->rank);
  int64_t ta = 0, tb = 0;
  f.get_i("trans_a", &ta);
  f.get_i("trans_b", &tb);
  const int64_t M = ta ? A->dims[1] : A->dims[0], K = ta ? A->dims[0] : A->dims[1];
  const int64_t Kb = tb ? B->dims[1] : B->dims[0], N = tb ? B->dims[0] : B->dims[1];
  if (K != Kb) return f.invalid("contraction sizes differ: %lld vs %lld", K, Kb);
  if (C->dims[0] != M || C->dims[1] != N || (R && !same_shape(R, C))) return f.invalid("C (and R) must be [%lld, %lld]", M, N);
  EMI_FFI_STREAM()
  return f.from_status(emi_gemm_ws(stream, A->data, B->data, R ? R->data : nullptr, C->data, ws ? ws->data : nullptr,
                                   ws ? byte_size(ws) : 0, M, N, K, A->dims[1], B->dims[1], N, N, (int)ta, (int)tb, A->dtype));
}

// x[M, K], w3[N, K], a[M, N] -> b[M, N], g[M, N]
extern "C" XLA_FFI_Error* emi_gemm_swiglu_fwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_gemm_swiglu_fwd", 3, 3, 2, 2)
  const XLA_FFI_Buffer *X = f.arg(0), *W = f.arg(1), *A = f.arg(2), *B = f.ret(0), *G = f.ret(1);
  if (!is_float(X) || W->dtype != X->dtype || A->dtype != X->dtype || B->dtype != X->dtype || G->dtype != X->dtype)
    return f.invalid("x, w3, a, b, g must share one dtype, f32 or bf16 (code %lld)", X->dtype);
  if (X->rank != 2 || W->rank != 2 || A->rank != 2) return f.invalid("operands must be rank 2");
  const int64_t M = X->dims[0], K = X->dims[1], N = W->dims[0];
  if (W->dims[1] != K) return f.invalid("contraction sizes differ: %lld vs %lld", K, W->dims[1]);
  if (A->dims[0] != M || A->dims[1] != N || !same_shape(A, B) || !same_shape(A, G)) return f.invalid("a, b, g must be [%lld, %lld]", M, N);
  EMI_FFI_STREAM()
  return f.from_status(emi_gemm_swiglu_fwd(stream, X->data, W->data, A->data, B->data, G->data, M, N, K, X->dtype));
}

// x[M, K], w[N, K], table[seq, head_dim/2, 2] -> y[M, N] = rope(x . w^T); rows are whole sequences of `seq` positions
extern "C" XLA_FFI_Error* emi_gemm_rope_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_gemm_rope", 3, 3, 1, 1)
  const XLA_FFI_Buffer *X = f.arg(0), *W = f.arg(1), *T = f.arg(2), *Y = f.ret(0);
  if (!is_float(X) || W->dtype != X->dtype || Y->dtype != X->dtype)
    return f.invalid("x, w, y must share one dtype, f32 or bf16 (code %lld)", X->dtype);
  if (X->rank != 2 || W->rank != 2 || Y->rank != 2) return f.invalid("x, w, y must be rank 2");
  const int64_t M = X->dims[0], K = X->dims[1], N = W->dims[0];
  if (W->dims[1] != K) return f.invalid("contraction sizes differ: %lld vs %lld", K, W->dims[1]);
  if (Y->dims[0] != M || Y->dims[1] != N) return f.invalid("y must be [%lld, %lld]", M, N);
  if (T->dtype != XLA_FFI_DataType_F32 || T->rank != 3 || T->dims[2] != 2 || T->dims[0] <= 0 || T->dims[1] <= 0)
    return f.invalid("the angle table must be f32[seq, head_dim/2, 2]");
  EMI_FFI_STREAM()
  return f.from_status(emi_gemm_rope(stream, X->data, W->data, Y->data, static_cast<const float*>(T->data), M, N, K, T->dims[0],
                                     2 * T->dims[1], X->dtype));
}

// dy[M, K], w2t[N, K], a[M, N], b[M, N] -> da[M, N], db[M, N] [, workspace]
extern "C" XLA_FFI_Error* emi_gemm_swiglu_bwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_gemm_swiglu_bwd", 4, 4, 2, 3)
  const XLA_FFI_Buffer *dY = f.arg(0), *W = f.arg(1), *A = f.arg(2), *B = f.arg(3), *dA = f.ret(0), *dB = f.ret(1);
  const XLA_FFI_Buffer* ws = cf->rets.size == 3 ? f.ret(2) : nullptr;
  if (!is_float(dY) || W->dtype != dY->dtype || A->dtype != dY->dtype || B->dtype != dY->dtype || dA->dtype != dY->dtype || dB->dtype != dY->dtype)
    return f.invalid("dy, w2t, a, b, da, db must share one dtype, f32 or bf16 (code %lld)", dY->dtype);
  if (dY->rank != 2 || W->rank != 2 || A->rank != 2) return f.invalid("operands must be rank 2");
  const int64_t M = dY->dims[0], K = dY->dims[1], N = W->dims[0];
  if (W->dims[1] != K) return f.invalid("contraction sizes differ: %lld vs %lld", K, W->dims[1]);
  if (A->dims[0] != M || A->dims[1] != N || !same_shape(A, B) || !same_shape(A, dA) || !same_shape(A, dB))
    return f.invalid("a, b, da, db must be [%lld, %lld]", M, N);
  EMI_FFI_STREAM()
  return f.from_status(emi_gemm_swiglu_bwd(stream, dY->data, W->data, A->data, B->data, dA->data, dB->data, ws ? ws->data : nullptr,
                                           ws ? byte_size(ws) : 0, M, N, K, dY->dtype));
}

// count A operands, count B operands, then no residual or one per result; count results (one when `sum`), then an
// optional scratch result for split-K partials.
extern "C" XLA_FFI_Error* emi_gemm_grouped_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_gemm_grouped", 4, 12, 1, 5)
  int64_t count = 0, sum = 0, ta = 0, tb = 0;
  if (!f.get_i("count", &count) || count < 2 || count > 4) return f.invalid("attribute 'count' must be 2, 3 or 4 (got %lld)", count);
  f.get_i("sum", &sum);
  f.get_i("trans_a", &ta);
  f.get_i("trans_b", &tb);
  const int64_t nout = sum ? 1 : count;
  const int64_t nargs = cf->args.size, nrets = cf->rets.size;
  if (nargs != 2 * count && nargs != 2 * count + nout)
    return f.invalid("expected %lld operands (A..., B...) or %lld (with residuals), got %lld", 2 * count, 2 * count + nout, nargs);
  if (nrets != nout && nrets != nout + 1) return f.invalid("expected %lld result(s) plus an optional workspace, got %lld", nout, nrets);
  const bool has_r = nargs == 2 * count + nout;
  const XLA_FFI_Buffer* A0 = f.arg(0);
  const XLA_FFI_Buffer* B0 = f.arg((int)count);
  if (!is_float(A0) || A0->rank != 2 || B0->rank != 2) return f.invalid("operands must be rank-2 f32 or bf16 (A rank %lld, B rank %lld)", A0->rank, B0->rank);
  const int64_t M = ta ? A0->dims[1] : A0->dims[0], K = ta ? A0->dims[0] : A0->dims[1];
  const int64_t Kb = tb ? B0->dims[1] : B0->dims[0], N = tb ? B0->dims[0] : B0->dims[1];
  if (K != Kb) return f.invalid("contraction sizes differ: %lld vs %lld", K, Kb);
  const void *a[4], *b[4], *r[4] = {nullptr, nullptr, nullptr, nullptr};
  void* c[4];
  for (int64_t i = 0; i < count; i++) {
    const XLA_FFI_Buffer *Ai = f.arg((int)i), *Bi = f.arg((int)(count + i));
    if (Ai->dtype != A0->dtype || Bi->dtype != A0->dtype || !same_shape(Ai, A0) || !same_shape(Bi, B0))
      return f.invalid("product %lld: operands must have the dtype and shapes of product 0", i);
    a[i] = Ai->data;
    b[i] = Bi->data;
  }
  for (int64_t i = 0; i < nout; i++) {
    const XLA_FFI_Buffer* Ci = f.ret((int)i);
    const XLA_FFI_Buffer* Ri = has_r ? f.arg((int)(2 * count + i)) : nullptr;
    if (Ci->dtype != A0->dtype || Ci->rank != 2 || Ci->dims[0] != M || Ci->dims[1] != N || (Ri && (Ri->dtype != A0->dtype || !same_shape(Ri, Ci))))
      return f.invalid("result %lld (and its residual) must be [%lld, %lld] of the operands' dtype", i, M, N);
    c[i] = Ci->data;
    r[i] = Ri ? Ri->data : nullptr;
  }
  const XLA_FFI_Buffer* ws = nrets == nout + 1 ? f.ret((int)nout) : nullptr;
  EMI_FFI_STREAM()
  return f.from_status(emi_gemm_grouped(stream, (int)count, a, b, has_r ? r : nullptr, c, ws ? ws->data : nullptr,
                                        ws ? byte_size(ws) : 0, M, N, K, A0->dims[1], B0->dims[1], N, N, (int)ta, (int)tb,
                                        sum ? 1 : 0, A0->dtype));
}

namespace {
struct AttnDims {
  int64_t B, H, S, D, sb, sh, ss;
};
bool attn_dims(const XLA_FFI_Buffer* q, int64_t bshd, AttnDims* d) {
  if (q->rank != 4) return false;
  d->B = q->dims[0];
  d->D = q->dims[3];
  if (bshd) {
    d->S = q->dims[1]; d->H = q->dims[2];
    d->sb = d->S * d->H * d->D; d->sh = d->D; d->ss = d->H * d->D;
  } else {
    d->H = q->dims[1]; d->S = q->dims[2];
    d->sb = d->H * d->S * d->D; d->sh = d->S * d->D; d->ss = d->D;
  }
  return true;
}
}  // namespace

extern "C" XLA_FFI_Error* emi_attn_fwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_attn_fwd", 3, 3, 2, 3)
  const XLA_FFI_Buffer *q = f.arg(0), *k = f.arg(1), *v = f.arg(2), *o = f.ret(0), *lse = f.ret(1);
  const XLA_FFI_Buffer* ws = cf->rets.size == 3 ? f.ret(2) : nullptr;
  if (!is_float(q) || k->dtype != q->dtype || v->dtype != q->dtype || o->dtype != q->dtype)
    return f.invalid("q, k, v, o must share one dtype, f32 or bf16 (code %lld)", q->dtype);
  int64_t causal = 1, bshd = 0;
  double scale;
  f.get_i("causal", &causal);
  f.get_i("bshd", &bshd);
  if (!f.get_f("scale", &scale)) return f.invalid("missing f32/f64 attribute 'scale'");
  AttnDims d;
  if (!attn_dims(q, bshd, &d) || !same_shape(q, k) || !same_shape(q, v) || !same_shape(q, o))
    return f.invalid("q, k, v, o must be rank 4 with one shape (q rank %lld)", q->rank);
  if (lse->dtype != XLA_FFI_DataType_F32 || lse->rank != 3 || lse->dims[0] != d.B || lse->dims[1] != d.H || lse->dims[2] != d.S)
    return f.invalid("lse must be f32[batch, heads, seq] = [%lld, %lld, %lld]", d.B, d.H, d.S);
  // An optional third result (scratch of earlier versions of this target) is accepted and left untouched.
  (void)ws;
  EMI_FFI_STREAM()
  return f.from_status(emi_attn_fwd_ws(stream, q->data, k->data, v->data, o->data, static_cast<float*>(lse->data),
                                       nullptr, 0, d.B, d.H, d.S, d.D, d.sb, d.sh, d.ss, (float)scale, (int)causal,
                                       q->dtype));
}

extern "C" XLA_FFI_Error* emi_attn_bwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_attn_bwd", 6, 6, 4, 4)
  const XLA_FFI_Buffer *q = f.arg(0), *k = f.arg(1), *v = f.arg(2), *o = f.arg(3), *lse = f.arg(4), *d_o = f.arg(5);
  const XLA_FFI_Buffer *dq = f.ret(0), *dk = f.ret(1), *dv = f.ret(2), *ws = f.ret(3);
  const XLA_FFI_Buffer* same[] = {k, v, o, d_o, dq, dk, dv};
  if (!is_float(q)) return f.invalid("q must be f32 or bf16 (code %lld)", q->dtype);
  for (const XLA_FFI_Buffer* b : same)
    if (b->dtype != q->dtype || !same_shape(q, b)) return f.invalid("q, k, v, o, do, dq, dk, dv must share dtype and shape");
  int64_t causal = 1, bshd = 0;
  double scale;
  f.get_i("causal", &causal);
  f.get_i("bshd", &bshd);
  if (!f.get_f("scale", &scale)) return f.invalid("missing f32/f64 attribute 'scale'");
  AttnDims d;
  if (!attn_dims(q, bshd, &d)) return f.invalid("q must be rank 4 (rank %lld)", q->rank);
  if (lse->dtype != XLA_FFI_DataType_F32 || lse->rank != 3 || lse->dims[0] != d.B || lse->dims[1] != d.H || lse->dims[2] != d.S)
    return f.invalid("lse must be f32[batch, heads, seq] = [%lld, %lld, %lld]", d.B, d.H, d.S);
  const size_t need = emi_attn_bwd_workspace_bytes(d.B, d.H, d.S, d.D);
  if (byte_size(ws) < need) return f.invalid("workspace result has %lld bytes, %lld needed", (long long)byte_size(ws), (long long)need);
  EMI_FFI_STREAM()
  return f.from_status(emi_attn_bwd(stream, q->data, k->data, v->data, o->data, static_cast<const float*>(lse->data), d_o->data,
                                    dq->data, dk->data, dv->data, ws->data, byte_size(ws), d.B, d.H, d.S, d.D, d.sb, d.sh, d.ss,
                                    (float)scale, (int)causal, q->dtype));
}

// emi_attn_bwd with a seventh operand, the RoPE angle table f32[seq, head_dim/2, 2]: dq and dk come out as the
// cotangents of q and k before their rotation.
extern "C" XLA_FFI_Error* emi_attn_bwd_rope_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_attn_bwd_rope", 7, 7, 4, 4)
  const XLA_FFI_Buffer *q = f.arg(0), *k = f.arg(1), *v = f.arg(2), *o = f.arg(3), *lse = f.arg(4), *d_o = f.arg(5), *T = f.arg(6);
  const XLA_FFI_Buffer *dq = f.ret(0), *dk = f.ret(1), *dv = f.ret(2), *ws = f.ret(3);
  const XLA_FFI_Buffer* same[] = {k, v, o, d_o, dq, dk, dv};
  if (!is_float(q)) return f.invalid("q must be f32 or bf16 (code %lld)", q->dtype);
  for (const XLA_FFI_Buffer* b : same)
    if (b->dtype != q->dtype || !same_shape(q, b)) return f.invalid("q, k, v, o, do, dq, dk, dv must share dtype and shape");
  int64_t causal = 1, bshd = 0;
  double scale;
  f.get_i("causal", &causal);
  f.get_i("bshd", &bshd);
  if (!f.get_f("scale", &scale)) return f.invalid("missing f32/f64 attribute 'scale'");
  AttnDims d;
  if (!attn_dims(q, bshd, &d)) return f.invalid("q must be rank 4 (rank %lld)", q->rank);
  if (lse->dtype != XLA_FFI_DataType_F32 || lse->rank != 3 || lse->dims[0] != d.B || lse->dims[1] != d.H || lse->dims[2] != d.S)
    return f.invalid("lse must be f32[batch, heads, seq] = [%lld, %lld, %lld]", d.B, d.H, d.S);
  if (T->dtype != XLA_FFI_DataType_F32 || T->rank != 3 || T->dims[0] != d.S || 2 * T->dims[1] != d.D || T->dims[2] != 2)
    return f.invalid("the angle table must be f32[seq, head_dim/2, 2] = [%lld, %lld, 2]", d.S, d.D / 2);
  const size_t need = emi_attn_bwd_workspace_bytes(d.B, d.H, d.S, d.D);
  if (byte_size(ws) < need) return f.invalid("workspace result has %lld bytes, %lld needed", (long long)byte_size(ws), (long long)need);
  EMI_FFI_STREAM()
  return f.from_status(emi_attn_bwd_rope(stream, q->data, k->data, v->data, o->data, static_cast<const float*>(lse->data),
                                         d_o->data, dq->data, dk->data, dv->data, static_cast<const float*>(T->data), ws->data,
                                         byte_size(ws), d.B, d.H, d.S, d.D, d.sb, d.sh, d.ss, (float)scale, (int)causal, q->dtype));
}

// Forward mode: tangents are ordinary operands (a zero tangent is passed as zeros).
extern "C" XLA_FFI_Error* emi_rmsnorm_jvp_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_rmsnorm_jvp", 4, 4, 1, 1)
  const XLA_FFI_Buffer *x = f.arg(0), *g = f.arg(1), *tx = f.arg(2), *tg = f.arg(3), *ty = f.ret(0);
  if (!is_float(x) || g->dtype != x->dtype || tx->dtype != x->dtype || tg->dtype != x->dtype || ty->dtype != x->dtype)
    return f.invalid("all tensors must share one dtype, f32 or bf16 (x has code %lld)", x->dtype);
  if (x->rank < 1 || g->rank != 1 || g->dims[0] != x->dims[x->rank - 1])
    return f.invalid("gamma must be rank 1 with the last dimension of x (x rank %lld, gamma rank %lld)", x->rank, g->rank);
  if (!same_shape(x, tx) || !same_shape(x, ty) || !same_shape(g, tg)) return f.invalid("tx, ty must have the shape of x and tgamma that of gamma");
  double eps;
  if (!f.get_f("eps", &eps)) return f.invalid("missing f32/f64 attribute 'eps'");
  EMI_FFI_STREAM()
  const int64_t D = g->dims[0];
  return f.from_status(emi_rmsnorm_jvp(stream, x->data, g->data, tx->data, tg->data, ty->data, D ? numel(x) / D : 0, D, (float)eps,
                                       x->dtype));
}

extern "C" XLA_FFI_Error* emi_swiglu_jvp_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_swiglu_jvp", 4, 4, 1, 1)
  const XLA_FFI_Buffer *a = f.arg(0), *b = f.arg(1), *ta = f.arg(2), *tb = f.arg(3), *tg = f.ret(0);
  if (!is_float(a) || b->dtype != a->dtype || ta->dtype != a->dtype || tb->dtype != a->dtype || tg->dtype != a->dtype)
    return f.invalid("all tensors must share one dtype, f32 or bf16 (code %lld)", a->dtype);
  if (!same_shape(a, b) || !same_shape(a, ta) || !same_shape(a, tb) || !same_shape(a, tg)) return f.invalid("all tensors must have one shape");
  EMI_FFI_STREAM()
  return f.from_status(emi_swiglu_jvp(stream, a->data, b->data, ta->data, tb->data, tg->data, numel(a), a->dtype));
}

extern "C" XLA_FFI_Error* emi_attn_jvp_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_attn_jvp", 7, 7, 1, 1)
  const XLA_FFI_Buffer *q = f.arg(0), *k = f.arg(1), *v = f.arg(2), *lse = f.arg(3), *tq = f.arg(4), *tk = f.arg(5), *tv = f.arg(6);
  const XLA_FFI_Buffer* to = f.ret(0);
  if (!is_float(q)) return f.invalid("q must be f32 or bf16 (code %lld)", q->dtype);
  const XLA_FFI_Buffer* same[] = {k, v, tq, tk, tv, to};
  for (const XLA_FFI_Buffer* b : same)
    if (b->dtype != q->dtype || !same_shape(q, b)) return f.invalid("q, k, v, tq, tk, tv, to must share dtype and shape");
  int64_t causal = 1, bshd = 0;
  double scale;
  f.get_i("causal", &causal);
  f.get_i("bshd", &bshd);
  if (!f.get_f("scale", &scale)) return f.invalid("missing f32/f64 attribute 'scale'");
  AttnDims d;
  if (!attn_dims(q, bshd, &d)) return f.invalid("q must be rank 4 (rank %lld)", q->rank);
  if (lse->dtype != XLA_FFI_DataType_F32 || lse->rank != 3 || lse->dims[0] != d.B || lse->dims[1] != d.H || lse->dims[2] != d.S)
    return f.invalid("lse must be f32[batch, heads, seq] = [%lld, %lld, %lld]", d.B, d.H, d.S);
  EMI_FFI_STREAM()
  return f.from_status(emi_attn_jvp(stream, q->data, k->data, v->data, static_cast<const float*>(lse->data), tq->data, tk->data,
                                    tv->data, to->data, d.B, d.H, d.S, d.D, d.sb, d.sh, d.ss, (float)scale, (int)causal, q->dtype));
}

namespace {
// q / o / dO / dq: [B, h, d]; caches and their cotangents: [B, S, h, d] (rows of one token contiguous).
struct StepDims {
  int64_t B, H, S, D;
};
bool step_dims(const XLA_FFI_Buffer* q, const XLA_FFI_Buffer* kc, StepDims* d) {
  if (q->rank != 3 || kc->rank != 4) return false;
  d->B = q->dims[0]; d->H = q->dims[1]; d->D = q->dims[2]; d->S = kc->dims[1];
  return kc->dims[0] == d->B && kc->dims[2] == d->H && kc->dims[3] == d->D;
}
}  // namespace

extern "C" XLA_FFI_Error* emi_attn_step_fwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_attn_step_fwd", 3, 3, 3, 3)
  const XLA_FFI_Buffer *q = f.arg(0), *k = f.arg(1), *v = f.arg(2), *o = f.ret(0), *lse = f.ret(1), *ws = f.ret(2);
  if (!is_float(q) || k->dtype != q->dtype || v->dtype != q->dtype || o->dtype != q->dtype)
    return f.invalid("q, k, v, o must share one dtype, f32 or bf16 (code %lld)", q->dtype);
  double scale;
  if (!f.get_f("scale", &scale)) return f.invalid("missing f32/f64 attribute 'scale'");
  StepDims d;
  if (!step_dims(q, k, &d) || !same_shape(k, v) || !same_shape(q, o))
    return f.invalid("q, o must be [batch, heads, head_dim] and k, v [batch, seq_kv, heads, head_dim] (q rank %lld)", q->rank);
  if (lse->dtype != XLA_FFI_DataType_F32 || lse->rank != 2 || lse->dims[0] != d.B || lse->dims[1] != d.H)
    return f.invalid("lse must be f32[batch, heads] = [%lld, %lld]", d.B, d.H);
  const size_t need = emi_attn_step_workspace_bytes(d.B, d.H, d.S, d.D);
  if (byte_size(ws) < need) return f.invalid("workspace result has %lld bytes, %lld needed", (long long)byte_size(ws), (long long)need);
  EMI_FFI_STREAM()
  return f.from_status(emi_attn_step_fwd(stream, q->data, k->data, v->data, o->data, static_cast<float*>(lse->data), ws->data,
                                         byte_size(ws), d.B, d.H, d.S, d.D, d.H * d.D, d.D, d.S * d.H * d.D, d.D, d.H * d.D,
                                         (float)scale, q->dtype));
}

extern "C" XLA_FFI_Error* emi_attn_step_bwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_attn_step_bwd", 6, 6, 4, 4)
  const XLA_FFI_Buffer *q = f.arg(0), *k = f.arg(1), *v = f.arg(2), *o = f.arg(3), *lse = f.arg(4), *d_o = f.arg(5);
  const XLA_FFI_Buffer *dq = f.ret(0), *dk = f.ret(1), *dv = f.ret(2), *ws = f.ret(3);
  if (!is_float(q)) return f.invalid("q must be f32 or bf16 (code %lld)", q->dtype);
  const XLA_FFI_Buffer* qlike[] = {o, d_o, dq};
  const XLA_FFI_Buffer* klike[] = {v, dk, dv};
  for (const XLA_FFI_Buffer* b : qlike)
    if (b->dtype != q->dtype || !same_shape(q, b)) return f.invalid("q, o, do, dq must share dtype and shape");
  for (const XLA_FFI_Buffer* b : klike)
    if (b->dtype != q->dtype || !same_shape(k, b)) return f.invalid("k, v, dk, dv must share dtype and shape");
  double scale;
  if (!f.get_f("scale", &scale)) return f.invalid("missing f32/f64 attribute 'scale'");
  StepDims d;
  if (k->dtype != q->dtype || !step_dims(q, k, &d))
    return f.invalid("q must be [batch, heads, head_dim] and k [batch, seq_kv, heads, head_dim] (q rank %lld)", q->rank);
  if (lse->dtype != XLA_FFI_DataType_F32 || lse->rank != 2 || lse->dims[0] != d.B || lse->dims[1] != d.H)
    return f.invalid("lse must be f32[batch, heads] = [%lld, %lld]", d.B, d.H);
  const size_t need = emi_attn_step_workspace_bytes(d.B, d.H, d.S, d.D);
  if (byte_size(ws) < need) return f.invalid("workspace result has %lld bytes, %lld needed", (long long)byte_size(ws), (long long)need);
  EMI_FFI_STREAM()
  return f.from_status(emi_attn_step_bwd(stream, q->data, k->data, v->data, o->data, static_cast<const float*>(lse->data),
                                         d_o->data, dq->data, dk->data, dv->data, ws->data, byte_size(ws), d.B, d.H, d.S, d.D,
                                         d.H * d.D, d.D, d.S * d.H * d.D, d.D, d.H * d.D, (float)scale, q->dtype));
}

extern "C" XLA_FFI_Error* emi_attn_step_jvp_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_attn_step_jvp", 8, 8, 2, 2)
  const XLA_FFI_Buffer *q = f.arg(0), *k = f.arg(1), *v = f.arg(2), *o = f.arg(3), *lse = f.arg(4), *tq = f.arg(5), *tk = f.arg(6),
                       *tv = f.arg(7);
  const XLA_FFI_Buffer *to = f.ret(0), *ws = f.ret(1);
  if (!is_float(q)) return f.invalid("q must be f32 or bf16 (code %lld)", q->dtype);
  const XLA_FFI_Buffer* qlike[] = {o, tq, to};
  const XLA_FFI_Buffer* klike[] = {v, tk, tv};
  for (const XLA_FFI_Buffer* b : qlike)
    if (b->dtype != q->dtype || !same_shape(q, b)) return f.invalid("q, o, tq, to must share dtype and shape");
  for (const XLA_FFI_Buffer* b : klike)
    if (b->dtype != q->dtype || !same_shape(k, b)) return f.invalid("k, v, tk, tv must share dtype and shape");
  double scale;
  if (!f.get_f("scale", &scale)) return f.invalid("missing f32/f64 attribute 'scale'");
  StepDims d;
  if (k->dtype != q->dtype || !step_dims(q, k, &d))
    return f.invalid("q must be [batch, heads, head_dim] and k [batch, seq_kv, heads, head_dim] (q rank %lld)", q->rank);
  if (lse->dtype != XLA_FFI_DataType_F32 || lse->rank != 2 || lse->dims[0] != d.B || lse->dims[1] != d.H)
    return f.invalid("lse must be f32[batch, heads] = [%lld, %lld]", d.B, d.H);
  const size_t need = emi_attn_step_workspace_bytes(d.B, d.H, d.S, d.D);
  if (byte_size(ws) < need) return f.invalid("workspace result has %lld bytes, %lld needed", (long long)byte_size(ws), (long long)need);
  EMI_FFI_STREAM()
  return f.from_status(emi_attn_step_jvp(stream, q->data, k->data, v->data, o->data, static_cast<const float*>(lse->data),
                                         tq->data, tk->data, tv->data, to->data, ws->data, byte_size(ws), d.B, d.H, d.S, d.D,
                                         d.H * d.D, d.D, d.S * d.H * d.D, d.D, d.H * d.D, (float)scale, q->dtype));
}

extern "C" XLA_FFI_Error* emi_embedding_fwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_embedding_fwd", 2, 2, 1, 1)
  const XLA_FFI_Buffer *tok = f.arg(0), *tab = f.arg(1), *x = f.ret(0);
  if (tok->dtype != XLA_FFI_DataType_S32) return f.invalid("tokens must be s32 (code %lld)", tok->dtype);
  if (!is_float(tab) || x->dtype != tab->dtype || tab->rank != 2) return f.invalid("table must be rank-2 f32 or bf16 and x share its dtype");
  if (x->rank != tok->rank + 1 || x->dims[x->rank - 1] != tab->dims[1] || numel(x) != numel(tok) * tab->dims[1])
    return f.invalid("x must be tokens.shape + [dim]");
  EMI_FFI_STREAM()
  return f.from_status(emi_embedding_fwd(stream, static_cast<const int32_t*>(tok->data), tab->data, x->data, numel(tok),
                                         tab->dims[0], tab->dims[1], tab->dtype));
}

extern "C" XLA_FFI_Error* emi_embedding_bwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_embedding_bwd", 2, 2, 1, 2)
  const XLA_FFI_Buffer *tok = f.arg(0), *dx = f.arg(1), *dt = f.ret(0), *ws = cf->rets.size == 2 ? f.ret(1) : nullptr;
  if (tok->dtype != XLA_FFI_DataType_S32) return f.invalid("tokens must be s32 (code %lld)", tok->dtype);
  if (!is_float(dx) || dt->dtype != dx->dtype || dt->rank != 2) return f.invalid("dtable must be rank-2 f32 or bf16 and dx share its dtype");
  if (dx->rank != tok->rank + 1 || dx->dims[dx->rank - 1] != dt->dims[1] || numel(dx) != numel(tok) * dt->dims[1])
    return f.invalid("dx must be tokens.shape + [dim]");
  const size_t need = emi_embedding_bwd_workspace_bytes(dt->dims[0], dt->dims[1], dx->dtype);
  if (need > 0 && (ws == nullptr || byte_size(ws) < need))
    return f.invalid("workspace result of %lld bytes needed", (long long)need);
  EMI_FFI_STREAM()
  return f.from_status(emi_embedding_bwd(stream, static_cast<const int32_t*>(tok->data), dx->data, dt->data,
                                         ws ? ws->data : nullptr, ws ? byte_size(ws) : 0, numel(tok), dt->dims[0], dt->dims[1],
                                         dx->dtype));
}

namespace {
// logits[.., V] with per-token buffers shaped like its leading dimensions
const char* xent_shapes(const XLA_FFI_Buffer* z, const XLA_FFI_Buffer* tgt, const XLA_FFI_Buffer* const* per_token, int n) {
  if (!is_float(z) || z->rank < 1) return "logits must be f32 or bf16 of rank >= 1";
  if (tgt->dtype != XLA_FFI_DataType_S32) return "targets must be s32";
  const int64_t V = z->dims[z->rank - 1];
  const int64_t T = V ? numel(z) / V : 0;
  if (numel(tgt) != T) return "targets must have one entry per token";
  for (int i = 0; i < n; i++)
    if (per_token[i]->dtype != XLA_FFI_DataType_F32 || numel(per_token[i]) != T) return "loss, lse, dloss and tloss are f32 with one entry per token";
  return nullptr;
}
}  // namespace

extern "C" XLA_FFI_Error* emi_cross_entropy_fwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_cross_entropy_fwd", 2, 2, 2, 2)
  const XLA_FFI_Buffer *z = f.arg(0), *tgt = f.arg(1), *loss = f.ret(0), *lse = f.ret(1);
  const XLA_FFI_Buffer* pt[] = {loss, lse};
  if (const char* why = xent_shapes(z, tgt, pt, 2)) return f.invalid(why);
  EMI_FFI_STREAM()
  const int64_t V = z->dims[z->rank - 1];
  return f.from_status(emi_cross_entropy_fwd(stream, z->data, static_cast<const int32_t*>(tgt->data),
                                             static_cast<float*>(loss->data), static_cast<float*>(lse->data),
                                             V ? numel(z) / V : 0, V, z->dtype));
}

extern "C" XLA_FFI_Error* emi_cross_entropy_bwd_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_cross_entropy_bwd", 4, 4, 1, 1)
  const XLA_FFI_Buffer *z = f.arg(0), *tgt = f.arg(1), *lse = f.arg(2), *dl = f.arg(3), *dz = f.ret(0);
  const XLA_FFI_Buffer* pt[] = {lse, dl};
  if (const char* why = xent_shapes(z, tgt, pt, 2)) return f.invalid(why);
  if (dz->dtype != z->dtype || !same_shape(z, dz)) return f.invalid("dlogits must have the shape and dtype of logits");
  EMI_FFI_STREAM()
  const int64_t V = z->dims[z->rank - 1];
  return f.from_status(emi_cross_entropy_bwd(stream, z->data, static_cast<const int32_t*>(tgt->data),
                                             static_cast<const float*>(lse->data), static_cast<const float*>(dl->data),
                                             dz->data, V ? numel(z) / V : 0, V, z->dtype));
}

extern "C" XLA_FFI_Error* emi_cross_entropy_jvp_ffi(XLA_FFI_CallFrame* cf) {
  EMI_FFI_BEGIN("emi_cross_entropy_jvp", 4, 4, 1, 1)
  const XLA_FFI_Buffer *z = f.arg(0), *tgt = f.arg(1), *lse = f.arg(2), *tz = f.arg(3), *tl = f.ret(0);
  const XLA_FFI_Buffer* pt[] = {lse, tl};
  if (const char* why = xent_shapes(z, tgt, pt, 2)) return f.invalid(why);
  if (tz->dtype != z->dtype || !same_shape(z, tz)) return f.invalid("tlogits must have the shape and dtype of logits");
  EMI_FFI_STREAM()
  const int64_t V = z->dims[z->rank - 1];
  return f.from_status(emi_cross_entropy_jvp(stream, z->data, static_cast<const int32_t*>(tgt->data),
                                             static_cast<const float*>(lse->data), tz->data,
                                             static_cast<float*>(tl->data), V ? numel(z) / V : 0, V, z->dtype));
}

namespace {
struct Target {
  const char* name;
  XLA_FFI_Handler* handler;
};
const Target kTargets[] = {
    {"emi_rmsnorm_fwd", emi_rmsnorm_fwd_ffi}, {"emi_rmsnorm_bwd", emi_rmsnorm_bwd_ffi},
    {"emi_rope_table", emi_rope_table_ffi},   {"emi_rope", emi_rope_ffi},
    {"emi_swiglu_fwd", emi_swiglu_fwd_ffi},   {"emi_swiglu_bwd", emi_swiglu_bwd_ffi},
    {"emi_add", emi_add_ffi},                 {"emi_gemm", emi_gemm_ffi},
    {"emi_gemm_grouped", emi_gemm_grouped_ffi},
    {"emi_gemm_swiglu_fwd", emi_gemm_swiglu_fwd_ffi}, {"emi_gemm_swiglu_bwd", emi_gemm_swiglu_bwd_ffi},
    {"emi_gemm_rope", emi_gemm_rope_ffi},     {"emi_attn_bwd_rope", emi_attn_bwd_rope_ffi},
    {"emi_attn_fwd", emi_attn_fwd_ffi},       {"emi_attn_bwd", emi_attn_bwd_ffi},
    {"emi_attn_step_fwd", emi_attn_step_fwd_ffi}, {"emi_attn_step_bwd", emi_attn_step_bwd_ffi},
    {"emi_rmsnorm_jvp", emi_rmsnorm_jvp_ffi}, {"emi_swiglu_jvp", emi_swiglu_jvp_ffi}, {"emi_attn_jvp", emi_attn_jvp_ffi},
    {"emi_attn_step_jvp", emi_attn_step_jvp_ffi},
    {"emi_embedding_fwd", emi_embedding_fwd_ffi}, {"emi_embedding_bwd", emi_embedding_bwd_ffi},
    {"emi_cross_entropy_fwd", emi_cross_entropy_fwd_ffi}, {"emi_cross_entropy_bwd", emi_cross_entropy_bwd_ffi},
    {"emi_cross_entropy_jvp", emi_cross_entropy_jvp_ffi},
};
constexpr int kNumTargets = sizeof(kTargets) / sizeof(kTargets[0]);
XLA_FFI_Error* noop_stage(XLA_FFI_CallFrame*) { return nullptr; }
}  // namespace

extern "C" int emi_ffi_target_count(void) { return kNumTargets; }
extern "C" const char* emi_ffi_target_name(int i) { return (i >= 0 && i < kNumTargets) ? kTargets[i].name : nullptr; }
extern "C" void* emi_ffi_target_handler(int i) {
  return (i >= 0 && i < kNumTargets) ? reinterpret_cast<void*>(kTargets[i].handler) : nullptr;
}

extern "C" int emi_fail(int code, const char* fmt, ...);

extern "C" int emi_register_ffi(const XLA_FFI_Api* api) {
  static std::once_flag once;
  static int result = EMI_OK;
  if (api == nullptr) return emi_fail(EMI_INVALID_ARGUMENT, "emi_register_ffi: null API table");
  if (api->struct_size < offsetof(XLA_FFI_Api, XLA_FFI_Handler_Register) + sizeof(void*) || api->XLA_FFI_Handler_Register == nullptr)
    return emi_fail(EMI_INVALID_ARGUMENT, "emi_register_ffi: API table (struct_size %zu) has no XLA_FFI_Handler_Register",
                    api->struct_size);
  std::call_once(once, [&] {
    static const char kPlatform[] = "ROCM";
    for (int i = 0; i < kNumTargets; i++) {
      XLA_FFI_Handler_Register_Args a;
      memset(&a, 0, sizeof(a));
      a.struct_size = sizeof(a);
      a.name.ptr = kTargets[i].name;
      a.name.len = strlen(kTargets[i].name);
      a.platform.ptr = kPlatform;
      a.platform.len = sizeof(kPlatform) - 1;
      a.bundle.instantiate = noop_stage;
      a.bundle.prepare = noop_stage;
      a.bundle.initialize = noop_stage;
      a.bundle.execute = kTargets[i].handler;
      a.traits = 0;
      if (api->XLA_FFI_Handler_Register(&a) != nullptr) {
        result = emi_fail(EMI_INTERNAL, "emi_register_ffi: registering %s failed", kTargets[i].name);
        return;
      }
    }
  });
  return result;
}
