"""GPU: softmax cross-entropy on the logits (emi_cross_entropy_fwd / bwd / jvp through the C ABI) against the
numpy oracle: per-token losses, logsumexp, the adjoint and the tangent, in fp32 (1e-4) and bf16 (2e-2), on rows that
are whole 16-byte chunks and rows that are not, with masked targets; the mean loss of the whole model with all its
gradients; the XLA-FFI handlers."""
import ctypes as C

import numpy as np
import pytest
import torch

import ffi_frames as F
from oracle import llama_ref as L
from gpu_util import dev, host, check, rel_err, TOL

pytestmark = pytest.mark.gpu

SHAPES = [((7,), 53), ((2, 5), 4104), ((64,), 32000), ((3,), 100003), ((1, 1), 8)]


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("lead,V", SHAPES)
def test_cross_entropy_matches_oracle(lead, V, dt):
    from enzyme_ad.jax import ops, jvp, vjp

    rng = np.random.default_rng(V)
    z, zr = dev(rng.standard_normal(lead + (V,)) * 4.0, dt)
    tz, tzr = dev(rng.standard_normal(lead + (V,)), dt)
    tn = rng.integers(0, V, size=lead).astype(np.int32)
    if tn.size > 2:
        tn.reshape(-1)[1] = -1                     # masked tokens
        tn.reshape(-1)[2] = V
    t = torch.from_numpy(tn).cuda()
    dl = rng.standard_normal(lead).astype(np.float32)

    fn = lambda logits: ops.cross_entropy(logits, t)
    loss, tl = jvp(fn, (z,), (tz,))
    assert loss.dtype == torch.float32 and tuple(loss.shape) == lead
    ref_loss, ref_lse = L.cross_entropy_fwd(zr, tn)
    # bf16 logits are rounded inputs, the arithmetic is fp32 for both dtypes
    np.testing.assert_allclose(host(loss), ref_loss, rtol=2e-6, atol=2e-5)
    np.testing.assert_allclose(host(tl), L.cross_entropy_jvp(zr, tn, tzr), rtol=1e-4, atol=2e-5)
    out, f_vjp = vjp(fn, z)
    assert torch.equal(out, loss)
    (dz,) = f_vjp(torch.from_numpy(dl).cuda())
    ref_dz = L.cross_entropy_bwd(zr, tn, dl)
    assert dz.dtype == z.dtype and dz.shape == z.shape
    check(dz, ref_dz, dt, "dlogits")
    if tn.size > 2:
        flat = host(dz).reshape(-1, V)
        assert not flat[1].any() and not flat[2].any() and float(host(loss).reshape(-1)[1]) == 0.0
    # <J v, w> = <v, J^T w> on the device results
    lhs = float((host(tl) * dl).sum())
    rhs = float((tzr * host(dz)).sum())
    assert abs(lhs - rhs) <= (5e-4 if dt == "f32" else 3e-2) * max(1.0, abs(lhs))


def test_cross_entropy_closed_forms_and_large_logits():
    from enzyme_ad.jax import ops

    V = 32000
    z = torch.full((4, V), 1.75, device="cuda")
    t = torch.tensor([0, 5, V - 1, 17], dtype=torch.int32, device="cuda")
    np.testing.assert_allclose(host(ops.cross_entropy(z, t)), np.log(V), rtol=1e-6)
    big = torch.zeros((2, 16), device="cuda")
    big[:, 3] = 1000.0                                              # the maximum is subtracted before exp
    got = host(ops.cross_entropy(big, torch.tensor([3, 0], dtype=torch.int32, device="cuda")))
    assert got[0] == 0.0 and got[1] == 1000.0


def test_cross_entropy_rejects_bad_arguments():
    from enzyme_ad.jax import ops, _native

    z = torch.zeros((4, 16), device="cuda")
    with pytest.raises(TypeError):
        ops.cross_entropy(z, torch.zeros(4, dtype=torch.int64, device="cuda"))
    with pytest.raises(ValueError):
        ops.cross_entropy(z, torch.zeros(3, dtype=torch.int32, device="cuda"))
    with pytest.raises(RuntimeError):
        ops.cross_entropy(z.cpu(), torch.zeros(4, dtype=torch.int32))
    lib = _native.lib()
    t = torch.zeros(4, dtype=torch.int32, device="cuda")
    out = torch.zeros(4, device="cuda")
    assert lib.emi_cross_entropy_fwd(None, z.data_ptr(), t.data_ptr(), out.data_ptr(), None, 4, 16, _native.EMI_F32) != 0
    assert b"null buffer" in lib.emi_last_error()
    assert lib.emi_cross_entropy_fwd(None, z.data_ptr(), t.data_ptr(), out.data_ptr(), out.data_ptr(), 4, 16, 10) != 0
    assert lib.emi_cross_entropy_bwd(None, z.data_ptr(), t.data_ptr(), out.data_ptr(), out.data_ptr(), z.data_ptr(), 4, 0,
                                     _native.EMI_F32) != 0


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_model_mean_loss_and_gradients(dt):
    """tokens -> embedding -> layers -> classifier -> mean cross-entropy, value and every weight gradient."""
    from enzyme_ad.jax import enzyme_jax_ir, vjp, llama

    cfg = dict(dim=64, hidden_dim=160, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=520, seq_len=24)
    w = L.make_weights(cfg, seed=21, norm_gain="uniform")
    rng = np.random.default_rng(5)
    B, S = 2, 24
    tokens = rng.integers(0, cfg["vocab_size"], size=(B, S)).astype(np.int32)
    targets = rng.integers(0, cfg["vocab_size"], size=(B, S)).astype(np.int32)
    names = sorted(w)
    dw, wr = {}, {}
    for k in names:
        dw[k], wr[k] = dev(w[k], dt)
    tok, tgt = torch.from_numpy(tokens).cuda(), torch.from_numpy(targets).cuda()

    @enzyme_jax_ir()
    def mean_loss(*ws):
        return llama.loss(tok, tgt, cfg, dict(zip(names, ws)))

    out, f_vjp = vjp(mean_loss, *[dw[k] for k in names])
    grads = f_vjp(torch.ones((), device="cuda"))
    logits, cache = L.model_fwd(tokens, wr, cfg, logits=True)
    ref_loss, _ = L.cross_entropy_fwd(logits, targets)
    ref = float(ref_loss.mean())
    assert abs(float(out) - ref) <= (1e-4 if dt == "f32" else 2e-2) * abs(ref)
    dlogits = L.cross_entropy_bwd(logits, targets, np.full((B, S), 1.0 / (B * S)))
    ref_grads = L.model_bwd(dlogits, wr, cfg, cache)[1]
    for k, g in zip(names, grads):
        check(g, ref_grads[k], dt, "d loss / d " + k)
    # forward mode through the same graph: d loss along a random direction = <gradient, direction>
    from enzyme_ad.jax import jvp
    tw = [dev(rng.standard_normal(w[k].shape) * 0.02, dt)[0] for k in names]
    _, tl = jvp(mean_loss, tuple(dw[k] for k in names), tuple(tw))
    parts = [float((g.double() * t.double()).sum()) for g, t in zip(grads, tw)]
    want, scale = sum(parts), sum(abs(p_) for p_ in parts)          # the parts cancel: bound the error by their size
    assert abs(float(tl) - want) <= (1e-3 if dt == "f32" else 5e-2) * scale, (float(tl), want, scale)


def _call(name, xla, args, rets):
    from enzyme_ad.jax import _native
    fn = getattr(_native.lib(), name)
    fn.restype, fn.argtypes = C.c_void_p, [C.POINTER(F.CallFrame)]
    cf = xla.frame(args, rets, {})
    return fn(C.byref(cf))


def _buf(xla, t):
    code = {torch.float32: F.F32, torch.bfloat16: F.BF16, torch.int32: F.S32}[t.dtype]
    return xla.buffer(code, list(t.shape), t.data_ptr())


def test_cross_entropy_ffi_handlers():
    from enzyme_ad.jax import _native

    lib = _native.lib()
    rng = np.random.default_rng(2)
    xla = F.FakeXla(stream=torch.cuda.current_stream().cuda_stream)
    z, _ = dev(rng.standard_normal((2, 3, 512)) * 2, "bf16")
    tz, _ = dev(rng.standard_normal((2, 3, 512)), "bf16")
    t = torch.from_numpy(rng.integers(0, 512, size=(2, 3)).astype(np.int32)).cuda()
    dl = torch.from_numpy(rng.standard_normal((2, 3)).astype(np.float32)).cuda()
    loss, lse, tl = (torch.empty((2, 3), device="cuda") for _ in range(3))
    dz = torch.empty_like(z)
    assert _call("emi_cross_entropy_fwd_ffi", xla, [_buf(xla, z), _buf(xla, t)], [_buf(xla, loss), _buf(xla, lse)]) is None
    assert _call("emi_cross_entropy_bwd_ffi", xla, [_buf(xla, b) for b in (z, t, lse, dl)], [_buf(xla, dz)]) is None
    assert _call("emi_cross_entropy_jvp_ffi", xla, [_buf(xla, b) for b in (z, t, lse, tz)], [_buf(xla, tl)]) is None
    torch.cuda.synchronize()
    st = torch.cuda.current_stream().cuda_stream
    loss2, lse2, tl2, dz2 = torch.empty_like(loss), torch.empty_like(lse), torch.empty_like(tl), torch.empty_like(dz)
    assert lib.emi_cross_entropy_fwd(st, z.data_ptr(), t.data_ptr(), loss2.data_ptr(), lse2.data_ptr(), 6, 512, _native.EMI_BF16) == 0
    assert lib.emi_cross_entropy_bwd(st, z.data_ptr(), t.data_ptr(), lse2.data_ptr(), dl.data_ptr(), dz2.data_ptr(), 6, 512, _native.EMI_BF16) == 0
    assert lib.emi_cross_entropy_jvp(st, z.data_ptr(), t.data_ptr(), lse2.data_ptr(), tz.data_ptr(), tl2.data_ptr(), 6, 512, _native.EMI_BF16) == 0
    assert torch.equal(loss, loss2) and torch.equal(lse, lse2) and torch.equal(tl, tl2) and torch.equal(dz, dz2)
    # shape and dtype errors come back as XLA_FFI errors, nothing is launched
    assert _call("emi_cross_entropy_fwd_ffi", xla, [_buf(xla, z), _buf(xla, dl)], [_buf(xla, loss), _buf(xla, lse)]) is not None
    assert _call("emi_cross_entropy_bwd_ffi", xla, [_buf(xla, b) for b in (z, t, lse, dl)], [_buf(xla, tl)]) is not None
    assert len(xla.errors) == 2 and "targets must be s32" in xla.errors[0][1]
