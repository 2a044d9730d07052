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
        assert len(calls) == low.count("stablehlo.custom_call") and set(calls) >= {"emi_gemm", "emi_attn_fwd", "emi_gemm_rope", "emi_gemm_swiglu_fwd"}, name
        for a, b in zip(got, want):
            assert torch.equal(a, b) if name == "primal" else _close(a, b, 2e-2), name


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_cross_entropy_and_gather_modules_through_the_ffi_handlers(dt):
    """The printed programs of a traced mean softmax cross-entropy and of a row lookup (the reference's gather.mlir
    input), primal, reverse and forward, with every custom call served by the library's FFI handler: the s32 operands
    (targets, indices), the f32 loss / log-sum-exp results and the scatter-add's table-shaped result are laid out as
    the handlers expect."""
    import json
    import os
    from enzyme_ad.jax import hlo_call, stablehlo_ad
    from enzyme_ad.jax import optimize_module
    from test_stablehlo_frontend import traced_cross_entropy_text

    rng = np.random.Generator(np.random.PCG64(12))
    tdt = torch.float32 if dt == "f32" else torch.bfloat16
    # cross-entropy
    rows, V = (6, 9), 520
    text = traced_cross_entropy_text(rows, V, dt=dt)
    z = dev(2.0 * rng.standard_normal(rows + (V,)), dt)[0]
    tz = dev(rng.standard_normal(rows + (V,)), dt)[0]
    tgt = torch.from_numpy(rng.integers(0, V, size=rows).astype(np.int32)).cuda()
    one = torch.ones((), device="cuda", dtype=tdt)
    programs = (("primal", optimize_module(text), [z, tgt], {"emi_cross_entropy_fwd"}),
                ("reverse", stablehlo_ad.reverse_module_text(text), [z, tgt, one], {"emi_cross_entropy_fwd", "emi_cross_entropy_bwd"}),
                ("forward", stablehlo_ad.forward_module_text(text), [z, tz, tgt], {"emi_cross_entropy_fwd", "emi_cross_entropy_jvp"}))
    for name, low, ins, targets in programs:
        exe, calls = _ffi_executable(low)
        got = exe.run(ins)
        torch.cuda.synchronize()
        want = hlo_call(*ins, source=low)
        assert set(calls) == targets and len(calls) == low.count("stablehlo.custom_call"), (name, calls)
        for a, b in zip(got, want):
            assert torch.equal(a, b), name
    # gather
    fixture = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "lit_primal_functions.json")))
    (fn_text,) = fixture["gather.mlir"]
    gtext = "module {\n" + fn_text.replace("f32", "f32" if dt == "f32" else "bf16") + "\n}"
    table = dev(rng.standard_normal((64, 3)), dt)[0]
    ttab = dev(rng.standard_normal((64, 3)), dt)[0]
    c = dev(rng.standard_normal((45, 3)), dt)[0]
    idx = torch.from_numpy(rng.integers(0, 64, size=(45, 1)).astype(np.int32)).cuda()
    rev = stablehlo_ad.reverse_module_text(gtext, arg_active=[True, False])
    exe, calls = _ffi_executable(rev)
    got = exe.run([table, idx, c])
    torch.cuda.synchronize()
    want = hlo_call(table, idx, c, source=rev)
    assert "emi_embedding_bwd" in calls
    assert _close(got[0], want[0], 1e-6 if dt == "f32" else 2e-2)          # fp32 atomics: the order of repeated rows differs
