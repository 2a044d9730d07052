"""GPU: the XLA-FFI handlers, driven with hand-built call frames that carry real
device buffers, produce bit-identical results to the plain C-ABI launchers."""
import ctypes as C

import numpy as np
import pytest
import torch

import ffi_frames as F
from oracle import llama_ref as L
from gpu_util import dev, host, check

pytestmark = pytest.mark.gpu


def _call(name, xla, args, rets, attrs):
    from enzyme_ad.jax import _native
    fn = getattr(_native.lib(), name)
    fn.restype, fn.argtypes = C.c_void_p, [C.POINTER(F.CallFrame)]
    cf = xla.frame(args, rets, attrs)
    err = fn(C.byref(cf))
    assert err is None, xla.errors
    torch.cuda.synchronize()


def _buf(xla, t):
    code = {torch.float32: F.F32, torch.bfloat16: F.BF16, torch.int32: F.S32, torch.uint8: F.U8}[t.dtype]
    return xla.buffer(code, list(t.shape), t.data_ptr())


def test_ffi_handlers_launch_on_the_frame_stream():
    from enzyme_ad.jax import ops, _native
    lib = _native.lib()
    side = torch.cuda.Stream()
    xla = F.FakeXla(stream=side.cuda_stream)
    rng = np.random.default_rng(0)
    with torch.cuda.stream(side):
        # rmsnorm fwd + bwd
        x, xr = dev(rng.standard_normal((6, 512)), "bf16")
        g, gr = dev(rng.uniform(0.5, 1.5, 512), "bf16")
        dy, dyr = dev(rng.standard_normal((6, 512)), "bf16")
        y = torch.empty_like(x)
        _call("emi_rmsnorm_fwd_ffi", xla, [_buf(xla, x), _buf(xla, g)], [_buf(xla, y)], {"eps": (F.F32, 1e-5)})
        assert torch.equal(y, ops.rmsnorm(x, g))
        dx, dg = torch.empty_like(x), torch.empty_like(g)
        ws = torch.empty(lib.emi_rmsnorm_bwd_workspace_bytes(6, 512), dtype=torch.uint8, device="cuda")
        _call("emi_rmsnorm_bwd_ffi", xla, [_buf(xla, x), _buf(xla, g), _buf(xla, dy)], [_buf(xla, dx), _buf(xla, dg), _buf(xla, ws)],
              {"eps": (F.F64, 1e-5)})
        rdx, rdg = L.rmsnorm_bwd(xr, gr, dyr)
        check(dx, rdx, "bf16", "ffi rmsnorm dx")
        check(dg, rdg, "bf16", "ffi rmsnorm dgamma")
        # rope table + rope
        B, S, h, d = 1, 40, 2, 64
        tab = torch.empty((S, d // 2, 2), dtype=torch.float32, device="cuda")
        _call("emi_rope_table_ffi", xla, [], [_buf(xla, tab)], {"theta": (F.F32, 10000.0), "pos0": (F.S64, 0)})
        q, qr = dev(rng.standard_normal((B, S, h, d)), "f32")
        qo = torch.empty_like(q)
        _call("emi_rope_ffi", xla, [_buf(xla, q), _buf(xla, tab)], [_buf(xla, qo)], {"inverse": (F.PRED, 0)})
        cos, sin = L.rope_angles(S, d)
        check(qo, L.rope_fwd(qr, cos, sin), "f32", "ffi rope")
        # gemm NT with residual
        a, ar = dev(rng.standard_normal((128, 256)), "bf16")
        w, wr = dev(rng.standard_normal((192, 256)) * 0.1, "bf16")
        r, rr = dev(rng.standard_normal((128, 192)), "bf16")
        c = torch.empty((128, 192), dtype=torch.bfloat16, device="cuda")
        _call("emi_gemm_ffi", xla, [_buf(xla, a), _buf(xla, w), _buf(xla, r)], [_buf(xla, c)],
              {"trans_a": (F.PRED, 0), "trans_b": (F.PRED, 1)})
        assert torch.equal(c, ops.gemm(a, w, False, True, r))
        check(c, ar @ wr.T + rr, "bf16", "ffi gemm")
        # grouped gemm: three weights against one activation, then the three adjoints summed into one dX
        ws3 = [dev(rng.standard_normal((192, 256)) * 0.1, "bf16") for _ in range(3)]
        cs3 = [torch.empty((128, 192), dtype=torch.bfloat16, device="cuda") for _ in range(3)]
        _call("emi_gemm_grouped_ffi", xla, [_buf(xla, a)] * 3 + [_buf(xla, w_) for w_, _ in ws3], [_buf(xla, c_) for c_ in cs3],
              {"count": (F.S64, 3), "sum": (F.PRED, 0), "trans_a": (F.PRED, 0), "trans_b": (F.PRED, 1)})
        for c_, (w_, wr_) in zip(cs3, ws3):
            check(c_, ar @ wr_.T, "bf16", "ffi grouped gemm")
        dx = torch.empty((128, 256), dtype=torch.bfloat16, device="cuda")
        _call("emi_gemm_grouped_ffi", xla, [_buf(xla, c_) for c_ in cs3] + [_buf(xla, w_) for w_, _ in ws3], [_buf(xla, dx)],
              {"count": (F.S64, 3), "sum": (F.PRED, 1), "trans_a": (F.PRED, 0), "trans_b": (F.PRED, 0)})
        check(dx, sum(host(c_) @ wr_ for c_, (_, wr_) in zip(cs3, ws3)), "bf16", "ffi grouped gemm, summed")
        # attention fwd + bwd, [B, S, h, d] layout
        B, S, h, d = 1, 96, 2, 128
        (q, qr), (k, kr), (v, vr), (do, dor) = (dev(rng.standard_normal((B, S, h, d)), "bf16") for _ in range(4))
        o = torch.empty_like(q)
        lse = torch.empty((B, h, S), dtype=torch.float32, device="cuda")
        at = {"scale": (F.F32, d ** -0.5), "causal": (F.PRED, 1), "bshd": (F.PRED, 1)}
        _call("emi_attn_fwd_ffi", xla, [_buf(xla, q), _buf(xla, k), _buf(xla, v)], [_buf(xla, o), _buf(xla, lse)], at)
        tr = lambda z: z.transpose(0, 2, 1, 3)
        ro, _ = L.attention_fwd(tr(qr), tr(kr), tr(vr))
        check(tr(host(o)), ro, "bf16", "ffi attention")
        dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
        ws = torch.empty(lib.emi_attn_bwd_workspace_bytes(B, h, S, d), dtype=torch.uint8, device="cuda")
        _call("emi_attn_bwd_ffi", xla, [_buf(xla, t) for t in (q, k, v, o, lse, do)], [_buf(xla, t) for t in (dq, dk, dv, ws)], at)
        rdq, rdk, rdv = L.attention_bwd(tr(qr), tr(kr), tr(vr), tr(dor))
        check(tr(host(dq)), rdq, "bf16", "ffi dq")
        check(tr(host(dk)), rdk, "bf16", "ffi dk")
        check(tr(host(dv)), rdv, "bf16", "ffi dv")
        # forward with the optional third result (scratch; unused now), long enough for the MFMA ping-pong kernel
        B, S, h, d = 1, 320, 2, 128
        (q, qr), (k, kr), (v, vr) = (dev(rng.standard_normal((B, S, h, d)), "bf16") for _ in range(3))
        o = torch.empty_like(q)
        lse = torch.empty((B, h, S), dtype=torch.float32, device="cuda")
        assert lib.emi_attn_fwd_workspace_bytes(B, h, S, d) == 0
        ws = torch.empty(64, dtype=torch.uint8, device="cuda")
        _call("emi_attn_fwd_ffi", xla, [_buf(xla, q), _buf(xla, k), _buf(xla, v)], [_buf(xla, o), _buf(xla, lse), _buf(xla, ws)], at)
        ro, _ = L.attention_fwd(tr(qr), tr(kr), tr(vr))
        check(tr(host(o)), ro, "bf16", "ffi attention with workspace")
        # single-token attention over a cache: q [B, h, d], caches [B, S, h, d]
        B, S, h, d = 2, 700, 3, 64
        (q, qr), (do, dor) = (dev(rng.standard_normal((B, h, d)), "bf16") for _ in range(2))
        (kc, kcr), (vc, vcr) = (dev(rng.standard_normal((B, S, h, d)), "bf16") for _ in range(2))
        o, dq = torch.empty_like(q), torch.empty_like(q)
        dk, dv = torch.empty_like(kc), torch.empty_like(vc)
        lse = torch.empty((B, h), dtype=torch.float32, device="cuda")
        ws = torch.empty(lib.emi_attn_step_workspace_bytes(B, h, S, d), dtype=torch.uint8, device="cuda")
        at = {"scale": (F.F32, d ** -0.5)}
        _call("emi_attn_step_fwd_ffi", xla, [_buf(xla, t) for t in (q, kc, vc)], [_buf(xla, t) for t in (o, lse, ws)], at)
        q4, k4, v4, do4 = qr[:, :, None, :], kcr.transpose(0, 2, 1, 3), vcr.transpose(0, 2, 1, 3), dor[:, :, None, :]
        ro, _ = L.attention_fwd(q4, k4, v4, causal=False)
        check(o, ro[:, :, 0, :], "bf16", "ffi step attention")
        _call("emi_attn_step_bwd_ffi", xla, [_buf(xla, t) for t in (q, kc, vc, o, lse, do)],
              [_buf(xla, t) for t in (dq, dk, dv, ws)], at)
        rdq, rdk, rdv = L.attention_bwd(q4, k4, v4, do4, causal=False)
        check(dq, rdq[:, :, 0, :], "bf16", "ffi step dq")
        check(dk, rdk.transpose(0, 2, 1, 3), "bf16", "ffi step dk")
        check(dv, rdv.transpose(0, 2, 1, 3), "bf16", "ffi step dv")
        # tangent of the step attention: same layout, tangents are ordinary operands
        (tq, tqr), = (dev(rng.standard_normal((B, h, d)), "bf16"),)
        (tkc, tkcr), (tvc, tvcr) = (dev(rng.standard_normal((B, S, h, d)), "bf16") for _ in range(2))
        to = torch.empty_like(q)
        _call("emi_attn_step_jvp_ffi", xla, [_buf(xla, t) for t in (q, kc, vc, o, lse, tq, tkc, tvc)],
              [_buf(xla, to), _buf(xla, ws)], at)
        rto = L.attention_jvp(q4, k4, v4, tqr[:, :, None, :], tkcr.transpose(0, 2, 1, 3), tvcr.transpose(0, 2, 1, 3), causal=False)
        check(to, rto[:, :, 0, :], "bf16", "ffi step attention tangent")
        # forward-mode targets: tangents are ordinary operands
        x4, x4r = dev(rng.standard_normal((6, 512)), "bf16")
        g4, g4r = dev(rng.uniform(0.5, 1.5, 512), "bf16")
        tx4, tx4r = dev(rng.standard_normal((6, 512)), "bf16")
        tg4, tg4r = dev(rng.standard_normal(512), "bf16")
        ty4 = torch.empty_like(x4)
        _call("emi_rmsnorm_jvp_ffi", xla, [_buf(xla, t) for t in (x4, g4, tx4, tg4)], [_buf(xla, ty4)], {"eps": (F.F32, 1e-5)})
        check(ty4, L.rmsnorm_jvp(x4r, g4r, tx4r, tg4r), "bf16", "ffi rmsnorm tangent")
        b4, b4r = dev(rng.standard_normal((6, 512)), "bf16")
        tb4, tb4r = dev(rng.standard_normal((6, 512)), "bf16")
        _call("emi_swiglu_jvp_ffi", xla, [_buf(xla, t) for t in (x4, b4, tx4, tb4)], [_buf(xla, ty4)], {})
        check(ty4, L.swiglu_jvp(x4r, b4r, tx4r, tb4r), "bf16", "ffi swiglu tangent")
        B, S, h, d = 1, 200, 2, 128
        (q, qr), (k, kr), (v, vr), (tq, tqr), (tk, tkr), (tv, tvr) = (dev(rng.standard_normal((B, S, h, d)), "bf16") for _ in range(6))
        o, to = torch.empty_like(q), torch.empty_like(q)
        lse = torch.empty((B, h, S), dtype=torch.float32, device="cuda")
        at = {"scale": (F.F32, d ** -0.5), "causal": (F.PRED, 1), "bshd": (F.PRED, 1)}
        _call("emi_attn_fwd_ffi", xla, [_buf(xla, q), _buf(xla, k), _buf(xla, v)], [_buf(xla, o), _buf(xla, lse)], at)
        _call("emi_attn_jvp_ffi", xla, [_buf(xla, t) for t in (q, k, v, lse, tq, tk, tv)], [_buf(xla, to)], at)
        check(tr(host(to)), L.attention_jvp(tr(qr), tr(kr), tr(vr), tr(tqr), tr(tkr), tr(tvr)), "bf16", "ffi attention tangent")
        # swiglu, add, embedding
        a, ar = dev(rng.standard_normal(1000), "f32")
        b, br = dev(rng.standard_normal(1000), "f32")
        gg = torch.empty_like(a)
        _call("emi_swiglu_fwd_ffi", xla, [_buf(xla, a), _buf(xla, b)], [_buf(xla, gg)], {})
        check(gg, L.swiglu_fwd(ar, br), "f32", "ffi swiglu")
        tok = torch.tensor([[1, 3, 3]], dtype=torch.int32, device="cuda")
        tabl, tablr = dev(rng.standard_normal((5, 8)), "bf16")
        xo = torch.empty((1, 3, 8), dtype=torch.bfloat16, device="cuda")
        _call("emi_embedding_fwd_ffi", xla, [_buf(xla, tok), _buf(xla, tabl)], [_buf(xla, xo)], {})
        assert np.array_equal(host(xo)[0], tablr[[1, 3, 3]])
    assert xla.errors == []
