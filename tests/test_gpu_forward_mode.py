"""GPU parity of forward mode (`jvp`): the three nonlinear tangent kernels, the composed
layer / model against the oracle's `model_jvp`, the <J v, w> = <v, J^T w> identity between the
HIP forward and reverse paths, and the reference's own API known answers
(test/test.py:100-167)."""
import numpy as np
import pytest
import torch

from oracle import llama_ref as L
from gpu_util import dev, host, check

pytestmark = pytest.mark.gpu


def test_reference_add_one_known_answers():
    """f(x, y) = x + 1 + y: primal [12, 23, 34], tangent [50.1, 70.2, 110.3], both cotangents
    equal to the output cotangent [500, 700, 110]."""
    from enzyme_ad.jax import enzyme_jax_ir, jvp, vjp, ops

    @enzyme_jax_ir()
    def add_one(x, y):
        return ops.add(ops.add(x, torch.ones_like(x)), y)

    f = lambda a: torch.tensor(a, dtype=torch.float32, device="cuda")
    x, y = f([1.0, 2.0, 3.0]), f([10.0, 20.0, 30.0])
    primals, tangents = jvp(add_one, (x, y), (f([0.1, 0.2, 0.3]), f([50.0, 70.0, 110.0])))
    assert torch.equal(primals, f([12.0, 23.0, 34.0]))
    assert torch.equal(tangents, f([0.1, 0.2, 0.3]) + f([50.0, 70.0, 110.0]))
    np.testing.assert_allclose(host(tangents), [50.1, 70.2, 110.3], rtol=1e-6)
    primals, f_vjp = vjp(add_one, x, y)
    gx, gy = f_vjp(f([500.0, 700.0, 110.0]))
    assert torch.equal(primals, f([12.0, 23.0, 34.0]))
    assert torch.equal(gx, f([500.0, 700.0, 110.0])) and torch.equal(gy, f([500.0, 700.0, 110.0]))


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("rows,dim", [(5, 288), (64, 4096), (3, 100)])
def test_rmsnorm_and_swiglu_tangents(dt, rows, dim):
    from enzyme_ad.jax import ops, jvp
    rng = np.random.Generator(np.random.PCG64(rows + dim))
    x, xr = dev(rng.standard_normal((rows, dim)), dt)
    g, gr = dev(rng.uniform(0.5, 1.5, dim), dt)
    tx, txr = dev(rng.standard_normal((rows, dim)), dt)
    tg, tgr = dev(rng.standard_normal(dim), dt)
    y, ty = jvp(lambda a, b: ops.rmsnorm(a, b), (x, g), (tx, tg))
    check(y, L.rmsnorm_fwd(xr, gr), dt, "rmsnorm")
    check(ty, L.rmsnorm_jvp(xr, gr, txr, tgr), dt, "rmsnorm tangent")
    _, ty = jvp(lambda a, b: ops.rmsnorm(a, b), (x, g), (tx, None))
    check(ty, L.rmsnorm_jvp(xr, gr, txr, 0 * tgr), dt, "rmsnorm tangent, x only")
    _, ty = jvp(lambda a, b: ops.rmsnorm(a, b), (x, g), (None, tg))
    check(ty, L.rmsnorm_jvp(xr, gr, 0 * txr, tgr), dt, "rmsnorm tangent, gamma only")
    b, br = dev(rng.standard_normal((rows, dim)), dt)
    tb, tbr = dev(rng.standard_normal((rows, dim)), dt)
    o, to = jvp(lambda a, c: ops.swiglu(a, c), (x, b), (tx, tb))
    check(o, L.swiglu_fwd(xr, br), dt, "swiglu")
    check(to, L.swiglu_jvp(xr, br, txr, tbr), dt, "swiglu tangent")
    _, to = jvp(lambda a, c: ops.swiglu(a, c), (x, b), (None, tb))
    check(to, L.swiglu_jvp(xr, br, 0 * txr, tbr), dt, "swiglu tangent, b only")


@pytest.mark.parametrize("dt,B,h,S,d,causal", [("f32", 1, 6, 40, 48, True), ("bf16", 2, 2, 300, 128, True),
                                               ("bf16", 1, 3, 130, 64, False), ("f32", 1, 2, 70, 50, True)])
def test_attention_tangent(dt, B, h, S, d, causal):
    from enzyme_ad.jax import ops, jvp
    rng = np.random.Generator(np.random.PCG64(S + d))
    ts = [dev(rng.standard_normal((B, S, h * d)), dt) for _ in range(6)]
    (q, qr), (k, kr), (v, vr), (tq, tqr), (tk, tkr), (tv, tvr) = ts
    fn = lambda a, b, c: ops.attention(a, b, c, h, causal=causal)
    o, to = jvp(fn, (q, k, v), (tq, tk, tv))
    hd = lambda t: t.reshape(B, S, h, d).transpose(0, 2, 1, 3)
    un = lambda t: t.transpose(0, 2, 1, 3).reshape(B, S, h * d)
    check(o, un(L.attention_fwd(hd(qr), hd(kr), hd(vr), causal=causal)[0]), dt, "attention")
    check(to, un(L.attention_jvp(hd(qr), hd(kr), hd(vr), hd(tqr), hd(tkr), hd(tvr), causal=causal)), dt, "attention tangent")
    _, to = jvp(fn, (q, k, v), (None, None, tv))
    check(to, un(L.attention_jvp(hd(qr), hd(kr), hd(vr), 0 * hd(tqr), 0 * hd(tkr), hd(tvr), causal=causal)), dt, "tangent, v only")


@pytest.mark.parametrize("dt,std", [("f32", 0.05), ("bf16", 0.04)])
def test_model_forward_mode_and_adjoint_identity(dt, std):
    """Two layers: tangents of the input and of every weight against the oracle's model_jvp, and
    <J v, w> (HIP forward mode) = <v, J^T w> (HIP reverse mode) in float64 on the host."""
    from enzyme_ad.jax import enzyme_jax_ir, JaXPipeline, jvp, vjp, llama
    cfg = {"dim": 256, "hidden_dim": 512, "n_layers": 2, "n_heads": 2, "n_kv_heads": 2, "vocab_size": 8, "seq_len": 160}
    B, S = 2, 160
    rng = np.random.Generator(np.random.PCG64(31))
    w = L.make_weights(cfg, 31, std=std, embedding=False, norm_gain="uniform")
    wd, wr, twd, twr = {}, {}, {}, {}
    for kname, a in w.items():
        wd[kname], wr[kname] = dev(a, dt)
        twd[kname], twr[kname] = dev(rng.standard_normal(a.shape) * std, dt)
    x, xr = dev(rng.standard_normal((B, S, cfg["dim"])), dt)
    tx, txr = dev(rng.standard_normal((B, S, cfg["dim"])), dt)

    @enzyme_jax_ir(pipeline_options=JaXPipeline(), inner_jit=False)
    def fn(x, weights):
        return llama.forward(x, cfg, weights)

    y, ty = jvp(fn, (x, wd), (tx, twd))
    ry, rty = L.model_jvp(xr, wr, txr, twr, cfg)
    check(y, ry, dt, "model output")
    e = check(ty, rty, dt, "model tangent")
    wv, wvr = dev(rng.standard_normal(ry.shape), dt)
    _, f_vjp = vjp(fn, x, wd)
    gx, gw = f_vjp(wv)
    lhs = float(np.sum(host(ty) * wvr))
    rhs = float(np.sum(host(gx) * txr)) + sum(float(np.sum(host(gw[kname]) * twr[kname])) for kname in gw)
    print("forward mode: tangent max rel err %.2e; <Jv,w> = %.6g, <v,J^T w> = %.6g" % (e, lhs, rhs), flush=True)
    assert abs(lhs - rhs) <= (2e-3 if dt == "f32" else 3e-2) * max(abs(lhs), abs(rhs), 1.0)
