"""The modules optimize_module prints, executed the way an XLA client would: every
`stablehlo.custom_call @emi_*` goes through the library's XLA-FFI handler with a hand-built call
frame (operand / result buffers of the printed types, attributes of the printed types from
`backend_config`), the remaining operators through the generic kernels.  Checks that the printed
wire format - operand order, result shapes including lse and workspace sizes, attribute names
and types - is what the handlers accept, and that the results equal hlo_call's (bit for bit for the primal programs)."""
import ctypes as C

import numpy as np
import pytest
import torch

import ffi_frames as F
from gpu_util import dev
from enzyme_ad.jax.llama_text import WEIGHT_ORDER, llama_layer_text, llama_step_text

pytestmark = pytest.mark.gpu

CODES = {torch.float32: F.F32, torch.bfloat16: F.BF16, torch.int32: F.S32, torch.uint8: F.U8}


def _ffi_executable(text):
    from enzyme_ad.jax import _native, stablehlo as S

    xla = F.FakeXla(stream=torch.cuda.current_stream().cuda_stream)
    calls = []

    class FfiExecutable(S.Executable):
        def _custom_call(self, op, xs):
            xs = [S._packed(x) for x in xs]
            outs = [torch.empty(t.shape, dtype=torch.uint8 if t.dtype == "i8" else S.TORCH_DTYPES[t.dtype], device="cuda") for t in op.types]
            attrs = {}
            for k, v in op.attrs["config"].items():
                attrs[k] = (F.PRED, int(v)) if isinstance(v, bool) else (F.S64, v) if isinstance(v, int) else (F.F32, v)
            buf = lambda t: xla.buffer(CODES[t.dtype], list(t.shape), t.data_ptr())
            fn = getattr(_native.lib(), op.attrs["target"] + "_ffi")
            fn.restype, fn.argtypes = C.c_void_p, [C.POINTER(F.CallFrame)]
            cf = xla.frame([buf(x) for x in xs], [buf(o) for o in outs], attrs)
            err = fn(C.byref(cf))
            assert err is None, (op.attrs["target"], xla.errors)
            calls.append(op.attrs["target"])
            return outs

    return FfiExecutable(text, fuse=False), calls


def _close(a, b, tol):
    a, b = a.float(), b.float()
    return float((a - b).abs().max()) <= tol * max(float(b.abs().max()), 1e-30)


def _step_args(cfg, pos, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    L_, D, H = cfg["n_layers"], cfg["dim"], cfg["hidden_dim"]
    shapes = {"rms_att_weight": (L_, D), "wq": (L_, D, D), "wk": (L_, D, D), "wv": (L_, D, D), "wo": (L_, D, D), "rms_ffn_weight": (L_, D),
              "w1": (L_, H, D), "w2": (L_, D, H), "w3": (L_, H, D), "rms_final_weight": (D,)}
    w = [dev(rng.uniform(0.5, 1.5, shapes[k]) if k.startswith("rms") else rng.standard_normal(shapes[k]) * 0.05, "f32")[0] for k in WEIGHT_ORDER]
    x, dy = (dev(rng.standard_normal(D), "f32")[0] for _ in range(2))
    kc, vc = (dev(rng.standard_normal((L_, pos, D)), "f32")[0] for _ in range(2))
    return [x] + w + [kc, vc], dy


def test_step_modules_through_the_ffi_handlers():
    from enzyme_ad.jax import hlo_call, optimize_module, primitives as P

    cfg = dict(dim=288, hidden_dim=768, n_layers=2, n_heads=6, n_kv_heads=6)
    text, order = llama_step_text(cfg, 9)
    args, dy = _step_args(cfg, 9, 4)
    fwd_pipe = P.forward_mode_pipeline(P.JaXPipeline(), [True] * len(args), 1)
    programs = {"primal": (optimize_module(text), args),
                "reverse": (optimize_module(text, P.reverse_mode_pipeline(fwd_pipe, [True]).pass_pipeline()), args + [dy]),
                "forward": (optimize_module(text, fwd_pipe.pass_pipeline()), [v for a in args for v in (a, torch.ones_like(a) * 0.01)])}
    for name, (low, ins) in programs.items():
        exe, calls = _ffi_executable(low)
        got = exe.run(ins)
        torch.cuda.synchronize()
        want = hlo_call(*ins, source=low)
        assert len(got) == len(want) and len(calls) == low.count("stablehlo.custom_call"), name
        for a, b in zip(got, want):
            # the primal program is bit-identical; in the derivative programs the one-row NN products run
            # without the workspace hlo_call gives them (another summation order)
            assert torch.equal(a, b) if name == "primal" else _close(a, b, 1e-5), name
    assert {"emi_attn_step_jvp", "emi_rmsnorm_jvp", "emi_swiglu_jvp"} <= set(calls)            # the last program run: forward


def test_layer_modules_through_the_ffi_handlers():
    from enzyme_ad.jax import hlo_call, optimize_module, primitives as P

    cfg = {"dim": 256, "hidden_dim": 704, "n_heads": 2}
    text, order = llama_layer_text(cfg, 2, 130, "bf16")
    rng = np.random.Generator(np.random.PCG64(3))
    shapes = [(2, 130, 256), (256,), (256, 256), (256, 256), (256, 256), (256, 256), (256,), (704, 256), (256, 704), (704, 256)]
    args = [dev(rng.uniform(0.5, 1.5, s) if len(s) == 1 else rng.standard_normal(s) * (1.0 if len(s) == 3 else 0.05), "bf16")[0] for s in shapes]
    dy = dev(rng.standard_normal(shapes[0]), "bf16")[0]
    fwd_pipe = P.forward_mode_pipeline(P.JaXPipeline(), [True] * len(args), 1)
    for name, low, ins in (("primal", optimize_module(text), args),
                           ("reverse", optimize_module(text, P.reverse_mode_pipeline(fwd_pipe, [True]).pass_pipeline()), args + [dy])):
        exe, calls = _ffi_executable(low)
        got = exe.run(ins)
        torch.cuda.synchronize()
        want = hlo_call(*ins, source=low)
        assert len(calls) == low.count("stablehlo.custom_call") and set(calls) >= {"emi_gemm", "emi_attn_fwd", "emi_rope"}, name
        for a, b in zip(got, want):
            assert torch.equal(a, b) if name == "primal" else _close(a, b, 2e-2), name
