"""ctypes binding of libemi_hip.so (the C ABI declared in include/emi.h).

The library is the only compute path: if it cannot be loaded the import of
any operator fails with an error; there is no CPU or eager fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(os.path.dirname(_HERE)), "lib", "libemi_hip.so")

EMI_F32, EMI_BF16 = 11, 16
EMI_ABI_VERSION = 1

c_void_p, c_i64, c_int, c_float, c_double, c_size_t = (
    ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_double, ctypes.c_size_t)

# name -> (restype, argtypes); mirrors include/emi.h one to one.
SIGNATURES = {
    "emi_abi_version": (c_int, []),
    "emi_last_error": (ctypes.c_char_p, []),
    "emi_rmsnorm_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_i64, c_float, c_int]),
    "emi_rmsnorm_bwd_workspace_bytes": (c_size_t, [c_i64, c_i64]),
    "emi_rmsnorm_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                c_size_t, c_i64, c_i64, c_float, c_int]),
    "emi_rmsnorm_bwd_noalloc": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_i64,
                                        c_float, c_int]),
    "emi_rope_table": (c_int, [c_void_p, c_void_p, c_i64, c_i64, c_double, c_i64]),
    "emi_rope": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_i64, c_i64, c_i64, c_int, c_int]),
    "emi_swiglu_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int]),
    "emi_swiglu_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int]),
    "emi_add": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int]),
    "emi_transpose": (c_int, [c_void_p, c_void_p, c_void_p, c_i64, c_i64, c_int]),
    "emi_map_binary": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int, c_int]),
    "emi_map_unary": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_i64, c_int]),
    "emi_compare": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int, c_int]),
    "emi_select": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int, c_int, c_int]),
    "emi_convert": (c_int, [c_void_p, c_void_p, c_void_p, c_i64, c_int, c_int]),
    "emi_strided_copy": (c_int, [c_void_p, c_void_p, c_void_p, c_int, ctypes.POINTER(c_i64), ctypes.POINTER(c_i64),
                                 c_i64, ctypes.POINTER(c_i64), c_i64, c_int]),
    "emi_reduce_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64, c_int]),
    "emi_reduce": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_i64, c_i64, c_i64, c_int]),
    "emi_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                         c_i64, c_int, c_int, c_int]),
    "emi_gemm_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64, c_int, c_int, c_int]),
    "emi_gemm_ws": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_i64, c_i64, c_i64, c_i64,
                            c_i64, c_i64, c_i64, c_int, c_int, c_int]),
    "emi_gemm_grouped_workspace_bytes": (c_size_t, [c_int, c_i64, c_i64, c_i64, c_int, c_int, c_int, c_int]),
    "emi_gemm_grouped": (c_int, [c_void_p, c_int, ctypes.POINTER(c_void_p), ctypes.POINTER(c_void_p), ctypes.POINTER(c_void_p),
                                 ctypes.POINTER(c_void_p), c_void_p, c_size_t, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                 c_int, c_int, c_int, c_int]),
    "emi_gemm_swiglu_fwd": (c_int, [c_void_p] * 6 + [c_i64, c_i64, c_i64, c_int]),
    "emi_gemm_swiglu_bwd_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64, c_int]),
    "emi_gemm_swiglu_bwd": (c_int, [c_void_p] * 8 + [c_size_t, c_i64, c_i64, c_i64, c_int]),
    "emi_attn_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_i64, c_i64, c_i64,
                             c_i64, c_i64, c_i64, c_float, c_int, c_int]),
    "emi_attn_fwd_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64, c_i64]),
    "emi_attn_fwd_ws": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_i64,
                                c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_float, c_int, c_int]),
    "emi_attn_bwd_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64, c_i64]),
    "emi_attn_bwd": (c_int, [c_void_p] * 10 + [c_void_p, c_size_t, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                               c_float, c_int, c_int]),
    "emi_attn_bwd_rope": (c_int, [c_void_p] * 11 + [c_void_p, c_size_t, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                                    c_float, c_int, c_int]),
    "emi_gemm_rope": (c_int, [c_void_p] * 5 + [c_i64, c_i64, c_i64, c_i64, c_i64, c_int]),
    "emi_attn_step_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64, c_i64]),
    "emi_attn_step_fwd": (c_int, [c_void_p] * 7 + [c_size_t] + [c_i64] * 9 + [c_float, c_int]),
    "emi_attn_step_bwd": (c_int, [c_void_p] * 11 + [c_size_t] + [c_i64] * 9 + [c_float, c_int]),
    "emi_attn_step_jvp": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_size_t, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                  c_float, c_int]),
    "emi_rmsnorm_jvp": (c_int, [c_void_p] * 6 + [c_i64, c_i64, c_float, c_int]),
    "emi_swiglu_jvp": (c_int, [c_void_p] * 6 + [c_i64, c_int]),
    "emi_attn_jvp": (c_int, [c_void_p] * 9 + [c_i64] * 7 + [c_float, c_int, c_int]),
    "emi_embedding_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_i64, c_i64, c_int]),
    "emi_embedding_bwd_workspace_bytes": (c_size_t, [c_i64, c_i64, c_int]),
    "emi_embedding_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_i64, c_i64, c_i64,
                                  c_int]),
    "emi_cross_entropy_fwd": (c_int, [c_void_p] * 5 + [c_i64, c_i64, c_int]),
    "emi_cross_entropy_bwd": (c_int, [c_void_p] * 6 + [c_i64, c_i64, c_int]),
    "emi_cross_entropy_jvp": (c_int, [c_void_p] * 6 + [c_i64, c_i64, c_int]),
}

_lib = None


class EmiError(RuntimeError):
    """A C-ABI call returned a non-zero status (code and message attached)."""

    def __init__(self, code, message):
        super().__init__("emi status %d: %s" % (code, message))
        self.code = code


def lib():
    """The loaded library with typed entry points (loaded once)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "libemi_hip.so is not built (%s); run `python enzyme-jax_amd/build.py`. "
                "There is no fallback path." % LIB_PATH)
        l = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype, fn.argtypes = res, args
        if l.emi_abi_version() != EMI_ABI_VERSION:
            raise ImportError("libemi_hip.so ABI %d != expected %d" % (l.emi_abi_version(), EMI_ABI_VERSION))
        _lib = l
    return _lib


def check(code):
    if code != 0:
        raise EmiError(code, lib().emi_last_error().decode("utf-8", "replace"))
