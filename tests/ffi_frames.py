"""Hand-built XLA FFI call frames (ctypes mirror of enzyme-jax_amd/csrc/xla_ffi_abi.h)
plus a fake API table, so the handlers can be driven without XLA."""
import ctypes as C

PRED, S32, S64, U8, F32, F64, BF16 = 1, 4, 5, 6, 11, 12, 16
ATTR_SCALAR = 3
STAGE_EXECUTE = 3
INVALID_ARGUMENT, INTERNAL = 3, 13


class ExtBase(C.Structure):
    pass


ExtBase._fields_ = [("struct_size", C.c_size_t), ("type", C.c_int), ("next", C.POINTER(ExtBase))]


class ApiVersion(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("major", C.c_int), ("minor", C.c_int)]


class Metadata(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("api_version", ApiVersion), ("traits", C.c_uint32)]


class MetadataExt(C.Structure):
    _fields_ = [("base", ExtBase), ("metadata", C.POINTER(Metadata))]


class Buffer(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("dtype", C.c_int), ("data", C.c_void_p),
                ("dims", C.POINTER(C.c_int64)), ("rank", C.c_int64)]


class ByteSpan(C.Structure):
    _fields_ = [("ptr", C.c_char_p), ("len", C.c_size_t)]


class Scalar(C.Structure):
    _fields_ = [("dtype", C.c_int), ("value", C.c_void_p)]


class Args(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("size", C.c_int64),
                ("types", C.POINTER(C.c_int)), ("args", C.POINTER(C.c_void_p))]


class Attrs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("size", C.c_int64),
                ("types", C.POINTER(C.c_int)), ("names", C.POINTER(C.POINTER(ByteSpan))), ("attrs", C.POINTER(C.c_void_p))]


class ErrorCreateArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("message", C.c_char_p), ("errc", C.c_int)]


class StreamGetArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("ctx", C.c_void_p), ("stream", C.c_void_p)]


class RegisterArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("name", ByteSpan), ("platform", ByteSpan),
                ("instantiate", C.c_void_p), ("prepare", C.c_void_p), ("initialize", C.c_void_p), ("execute", C.c_void_p),
                ("traits", C.c_uint32)]


ERR_CREATE = C.CFUNCTYPE(C.c_void_p, C.POINTER(ErrorCreateArgs))
VOID_FN = C.CFUNCTYPE(None, C.c_void_p)
REGISTER = C.CFUNCTYPE(C.c_void_p, C.POINTER(RegisterArgs))
STREAM_GET = C.CFUNCTYPE(C.c_void_p, C.POINTER(StreamGetArgs))


class Api(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("api_version", ApiVersion),
                ("internal_api", C.c_void_p), ("error_create", ERR_CREATE), ("error_get_message", VOID_FN),
                ("error_destroy", VOID_FN), ("handler_register", REGISTER), ("stream_get", STREAM_GET)]


class CallFrame(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.POINTER(ExtBase)), ("api", C.POINTER(Api)),
                ("ctx", C.c_void_p), ("stage", C.c_int), ("args", Args), ("rets", Args), ("attrs", Attrs),
                ("future", C.c_void_p)]


class FakeXla:
    """Fake API table: records created errors and registered handlers; hands out `stream`."""

    def __init__(self, stream=None):
        self.errors, self.registered, self.stream = [], [], stream
        self._keep = []

        def err_create(a):
            self.errors.append((a.contents.errc, a.contents.message.decode()))
            return 0xE770  # any non-null token

        def stream_get(a):
            a.contents.stream = self.stream
            return None

        def register(a):
            r = a.contents
            self.registered.append((r.name.ptr[: r.name.len].decode(), r.platform.ptr[: r.platform.len].decode(), r.execute))
            return None

        self._cbs = (ERR_CREATE(err_create), VOID_FN(lambda p: None), VOID_FN(lambda p: None), REGISTER(register),
                     STREAM_GET(stream_get))
        self.api = Api(C.sizeof(Api), None, ApiVersion(C.sizeof(ApiVersion), None, 0, 1), None, *self._cbs)

    def buffer(self, dtype, dims, data=0x1000):
        d = (C.c_int64 * max(len(dims), 1))(*dims)
        b = Buffer(C.sizeof(Buffer), None, dtype, data, d, len(dims))
        self._keep += [d, b]
        return b

    def frame(self, args, rets, attrs=None, stage=STAGE_EXECUTE):
        attrs = attrs or {}

        def pack(bufs):
            n = len(bufs)
            types = (C.c_int * max(n, 1))(*([1] * n))
            ptrs = (C.c_void_p * max(n, 1))(*[C.addressof(b) for b in bufs])
            self._keep += [types, ptrs]
            return Args(C.sizeof(Args), None, n, types, ptrs)

        names = sorted(attrs)
        n = len(names)
        types = (C.c_int * max(n, 1))(*([ATTR_SCALAR] * n))
        spans = (C.POINTER(ByteSpan) * max(n, 1))()
        vals = (C.c_void_p * max(n, 1))()
        for i, k in enumerate(names):
            dtype, v = attrs[k]
            ctype = {F32: C.c_float, F64: C.c_double, PRED: C.c_uint8, S64: C.c_int64, S32: C.c_int32}[dtype]
            box = ctype(v)
            sc = Scalar(dtype, C.addressof(box))
            sp = ByteSpan(k.encode(), len(k))
            self._keep += [box, sc, sp]
            spans[i] = C.pointer(sp)
            vals[i] = C.addressof(sc)
        self._keep += [types, spans, vals]
        at = Attrs(C.sizeof(Attrs), None, n, types, spans, vals)
        cf = CallFrame(C.sizeof(CallFrame), None, C.pointer(self.api), None, stage, pack(args), pack(rets), at, None)
        self._keep.append(cf)
        return cf
