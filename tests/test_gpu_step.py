"""GPU parity of the single-token (decode) form, the literal shape of the reference's
test/llama.py: mat-vec kernels and their adjoints through emi_gemm, attention of one
query over a key/value cache, and the whole step forward + VJP against the CPU oracle
(`forward_step`, `forward_step_vjp`) on the same seeded inputs."""
import numpy as np
import pytest
import torch

from oracle import llama_ref as L
from gpu_util import dev, host, check

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("m,n,k", [(1, 288, 288), (1, 768, 288), (3, 520, 264), (8, 4096, 1024), (1, 11008, 4096),
                                   (1, 4096, 11008),      # few long rows: two wavefronts share a row of W
                                   (2, 1000, 20000),      # four wavefronts per row, two rows of x, a ragged last batch
                                   (5, 301, 9000)])       # four per row in fp32, rows that do not fill the last block
def test_skinny_gemm_forms(dt, m, n, k):
    """Y = X W^T (M <= 8 tokens), dX = dY W and dW = dY^T X with and without residual."""
    from enzyme_ad.jax import ops
    rng = np.random.Generator(np.random.PCG64(m * 1000 + n + k))
    x, xr = dev(rng.standard_normal((m, k)), dt)
    w, wr = dev(rng.standard_normal((n, k)) * 0.05, dt)
    r, rr = dev(rng.standard_normal((m, n)), dt)
    dy, dyr = dev(rng.standard_normal((m, n)), dt)
    rx, rxr = dev(rng.standard_normal((m, k)), dt)
    rw, rwr = dev(rng.standard_normal((n, k)), dt)
    check(ops.gemm(x, w, False, True), xr @ wr.T, dt, "y")
    check(ops.gemm(x, w, False, True, r), xr @ wr.T + rr, dt, "y + r")
    check(ops.gemm(dy, w, False, False), dyr @ wr, dt, "dx")                    # banded kernel (workspace)
    plain = torch.empty((m, k), dtype=dy.dtype, device="cuda")                  # same product without a workspace
    from enzyme_ad.jax import _native as N
    N.check(N.lib().emi_gemm(torch.cuda.current_stream().cuda_stream, dy.data_ptr(), w.data_ptr(), None, plain.data_ptr(),
                             m, k, n, n, k, k, k, 0, 0, ops._code(dy)))
    check(plain, dyr @ wr, dt, "dx without workspace")
    check(ops.gemm(dy, w, False, False, rx), dyr @ wr + rxr, dt, "dx + r")
    check(ops.gemm(dy, x, True, False), dyr.T @ xr, dt, "dw")
    check(ops.gemm(dy, x, True, False, rw), dyr.T @ xr + rwr, dt, "dw + r")


@pytest.mark.parametrize("dt,heads,d,s", [("f32", 6, 48, 2), ("f32", 6, 48, 301), ("bf16", 4, 128, 1000), ("bf16", 3, 64, 77),
                                            ("f32", 2, 50, 33), ("bf16", 2, 36, 5)])
def test_attention_step_forward_backward(dt, heads, d, s):
    from enzyme_ad.jax import ops
    D = heads * d
    rng = np.random.Generator(np.random.PCG64(s * 7 + d))
    q, qr = dev(rng.standard_normal(D), dt)
    kc, kcr = dev(rng.standard_normal((s, D)), dt)
    vc, vcr = dev(rng.standard_normal((s, D)), dt)
    do, dor = dev(rng.standard_normal(D), dt)
    with ops.Tape() as tape:
        o = ops.attention_step(q, kc, vc, heads)
    hd = lambda t: t.reshape(1, -1, heads, d).transpose(0, 2, 1, 3)
    ro, _ = L.attention_fwd(hd(qr), hd(kcr), hd(vcr), causal=False)
    check(o, ro.transpose(0, 2, 1, 3).reshape(D), dt, "o")
    dq, dk, dv = tape.backward([o], [do], [q, kc, vc])
    rdq, rdk, rdv = L.attention_bwd(hd(qr), hd(kcr), hd(vcr), hd(dor), causal=False)
    un = lambda t: t.transpose(0, 2, 1, 3).reshape(-1, D)
    check(dq, un(rdq)[0], dt, "dq")
    check(dk, un(rdk), dt, "dk")
    check(dv, un(rdv), dt, "dv")


def _step_case(cfg, pos, dt, seed, zero_cache, std, uniform=False):
    from enzyme_ad.jax import enzyme_jax_ir, JaXPipeline, vjp, llama
    rng = np.random.Generator(np.random.PCG64(seed))
    w = L.make_weights(cfg, seed, std=std, embedding=False, norm_gain="uniform")
    if uniform:
        w = {k: rng.uniform(0, 1, size=v.shape) for k, v in w.items()}
    wd, wr = {}, {}
    for k, a in w.items():
        wd[k], wr[k] = dev(a, dt)
    x, xr = dev(rng.uniform(0, 1, cfg["dim"]) if uniform else rng.standard_normal(cfg["dim"]), dt)
    shape = (cfg["n_layers"], pos, cfg["dim"])
    kc, kcr = dev(np.zeros(shape) if zero_cache else rng.standard_normal(shape), dt)
    vc, vcr = dev(np.zeros(shape) if zero_cache else rng.standard_normal(shape), dt)
    dy, dyr = dev(rng.standard_normal(cfg["dim"]), dt)

    @enzyme_jax_ir(pipeline_options=JaXPipeline(), inner_jit=False)
    def fn(x, weights, key_cache, value_cache):
        return llama.forward_step(x, cfg, weights, key_cache, value_cache)

    y, f_vjp = vjp(fn, x, wd, kc, vc)
    gx, gw, gkc, gvc = f_vjp(dy)
    ry, rdx, rgw, rdkc, rdvc = L.forward_step_vjp(xr, cfg, wr, kcr, vcr, dyr)
    np.testing.assert_allclose(ry, L.forward_step(xr, cfg, wr, kcr, vcr), rtol=1e-9, atol=1e-11)
    return (y, gx, gw, gkc, gvc), (ry, rdx, rgw, rdkc, rdvc)


@pytest.mark.parametrize("pos,zero_cache", [(1, True), (7, False)])
def test_step_form_stories15m_fp32(pos, zero_cache):
    """The reference's own case: dim 288, hidden 768, 6 layers, 6 heads, fp32, one token at
    position pos with a cache of pos rows (all zeros at pos = 1 in the shipped fixture,
    test/llama.py:246-254,299-301)."""
    cfg = {"dim": 288, "hidden_dim": 768, "n_layers": 6, "n_heads": 6, "n_kv_heads": 6, "vocab_size": 32000, "seq_len": 256}
    (y, gx, gw, gkc, gvc), (ry, rdx, rgw, rdkc, rdvc) = _step_case(cfg, pos, "f32", 21 + pos, zero_cache, std=0.05)
    errs = {"y": check(y, ry, "f32", "y"), "dx": check(gx, rdx, "f32", "dx"), "dkc": check(gkc, rdkc, "f32", "dkey_cache"),
            "dvc": check(gvc, rdvc, "f32", "dvalue_cache")}
    for k in rgw:
        errs[k] = check(gw[k], rgw[k], "f32", "grad " + k)
    print("step form max rel errors", {k: "%.2e" % v for k, v in errs.items()}, flush=True)


def test_step_form_reference_distributions():
    """uniform[0,1) weights and input as the fixture draws them (test/llama.py:266-301),
    compared with the reference's own rule allclose(atol = rtol = 1e-3) (:318-319)."""
    cfg = {"dim": 288, "hidden_dim": 768, "n_layers": 6, "n_heads": 6, "n_kv_heads": 6, "vocab_size": 32000, "seq_len": 256}
    (y, gx, gw, gkc, gvc), (ry, rdx, rgw, rdkc, rdvc) = _step_case(cfg, 1, "f32", 3, True, std=0.05, uniform=True)
    assert np.allclose(host(y), ry, atol=1e-3, rtol=1e-3)
    assert np.allclose(host(gx), rdx, atol=1e-3, rtol=1e-3)
    for k in rgw:
        assert np.allclose(host(gw[k]), rgw[k], atol=1e-3, rtol=1e-3), k


def test_step_form_bf16_llama_head_shape():
    """bf16, head_dim 128, through the vectorised mat-vec and step-attention kernels."""
    cfg = {"dim": 512, "hidden_dim": 1376, "n_layers": 2, "n_heads": 4, "n_kv_heads": 4, "vocab_size": 8, "seq_len": 512}
    (y, gx, gw, gkc, gvc), (ry, rdx, rgw, rdkc, rdvc) = _step_case(cfg, 300, "bf16", 9, False, std=0.04)
    check(y, ry, "bf16", "y")
    check(gx, rdx, "bf16", "dx")
    check(gkc, rdkc, "bf16", "dkey_cache")
    check(gvc, rdvc, "bf16", "dvalue_cache")
    for k in rgw:
        check(gw[k], rgw[k], "bf16", "grad " + k)


@pytest.mark.parametrize("dt,heads,d,s", [("f32", 6, 48, 2), ("f32", 6, 48, 301), ("bf16", 4, 128, 1000), ("bf16", 3, 64, 77),
                                            ("f32", 2, 50, 33), ("bf16", 2, 36, 5)])
def test_attention_step_tangent(dt, heads, d, s):
    """Forward mode of the step attention against the oracle's attention_jvp (one query, no
    mask), with all tangents and with single ones (null pointers are zero tangents)."""
    from enzyme_ad.jax import ops, jvp
    D = heads * d
    rng = np.random.Generator(np.random.PCG64(s * 11 + d))
    (q, qr), (tq, tqr) = (dev(rng.standard_normal(D), dt) for _ in range(2))
    (kc, kcr), (vc, vcr), (tk, tkr), (tv, tvr) = (dev(rng.standard_normal((s, D)), dt) for _ in range(4))
    hd = lambda t: t.reshape(1, -1, heads, d).transpose(0, 2, 1, 3)
    fn = lambda a, b, c: ops.attention_step(a, b, c, heads)
    for mask in ((1, 1, 1), (1, 0, 0), (0, 1, 0), (0, 0, 1)):
        tans = tuple(t if m else None for t, m in zip((tq, tk, tv), mask))
        o, to = jvp(fn, (q, kc, vc), tans)
        ref = L.attention_jvp(hd(qr), hd(kcr), hd(vcr), mask[0] * hd(tqr), mask[1] * hd(tkr), mask[2] * hd(tvr), causal=False)
        check(to, ref.transpose(0, 2, 1, 3).reshape(D), dt, "step tangent %s" % (mask,))


def test_step_form_forward_mode_adjoint_identity():
    """<J v, w> from forward mode of the whole step = <v, J^T w> from its reverse mode."""
    from enzyme_ad.jax import jvp, vjp, llama
    cfg = {"dim": 288, "hidden_dim": 768, "n_layers": 3, "n_heads": 6, "n_kv_heads": 6, "vocab_size": 32000, "seq_len": 256}
    pos = 9
    rng = np.random.Generator(np.random.PCG64(61))
    w = L.make_weights(cfg, 61, std=0.05, embedding=False, norm_gain="uniform")
    wd = {k: dev(a, "f32")[0] for k, a in w.items()}
    tw = {k: dev(rng.standard_normal(a.shape) * 0.05, "f32")[0] for k, a in w.items()}
    x, tx, dy = (dev(rng.standard_normal(cfg["dim"]), "f32")[0] for _ in range(3))
    shape = (cfg["n_layers"], pos, cfg["dim"])
    kc, vc, tkc, tvc = (dev(rng.standard_normal(shape), "f32")[0] for _ in range(4))
    fn = lambda x, w, kc, vc: llama.forward_step(x, cfg, w, kc, vc)
    y, ty = jvp(fn, (x, wd, kc, vc), (tx, tw, tkc, tvc))
    y2, f_vjp = vjp(fn, x, wd, kc, vc)
    gx, gw, gkc, gvc = f_vjp(dy)
    lhs = float(np.dot(host(ty), host(dy)))
    rhs = float(np.sum(host(gx) * host(tx)) + np.sum(host(gkc) * host(tkc)) + np.sum(host(gvc) * host(tvc)) +
                sum(np.sum(host(gw[k]) * host(tw[k])) for k in w))
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), abs(rhs)), (lhs, rhs)
