"""Pins oracle/llama_ref.py: (1) the batched/causal functions equal the literal
single-token step of test/llama.py replayed with a real KV cache; (2) the
closed-form adjoints equal the reference's per-op rules chained in trace order;
(3) central finite differences; (4) an independent torch.autograd restatement;
(5) closed-form special cases."""
import numpy as np
import pytest
import torch

from oracle import llama_ref as L

CFG = {"dim": 24, "hidden_dim": 40, "n_layers": 2, "n_heads": 3, "n_kv_heads": 3,
       "vocab_size": 50, "seq_len": 8}


def _weights(cfg, seed=0, uniform=False):
    w = L.make_weights(cfg, seed, std=0.3, dtype=np.float64)
    if uniform:   # the reference fixture draws uniform[0,1) (test/llama.py:266-291)
        rng = np.random.default_rng(seed)
        w = {k: rng.uniform(0, 1, size=v.shape) for k, v in w.items()}
    return w


@pytest.mark.parametrize("uniform", [False, True])
def test_batched_forward_equals_step_form_replayed(uniform):
    cfg, S = CFG, 6
    w = _weights(cfg, 3, uniform)
    rng = np.random.default_rng(5)
    x = rng.standard_normal((1, S, cfg["dim"]))
    kc = np.zeros((cfg["n_layers"], 0, cfg["dim"]))
    vc = np.zeros((cfg["n_layers"], 0, cfg["dim"]))
    outs = []
    for t in range(S):
        y, kc, vc = L.forward_step(x[0, t], cfg, w, kc, vc, return_caches=True)
        outs.append(y)
    got, _ = L.model_fwd(x, w, cfg, logits=False)
    np.testing.assert_allclose(got[0], np.stack(outs), rtol=1e-10, atol=1e-12)


def test_step_form_reference_fixture_shape():
    """The shipped fixture: pos = 1 with an all-zero cached row (llama.py:299-301):
    softmax weights are [1, e^s]/(1+e^s)."""
    cfg = CFG
    w = _weights(cfg, 1, uniform=True)
    x = np.random.default_rng(2).uniform(0, 1, cfg["dim"])
    kc = np.zeros((cfg["n_layers"], 1, cfg["dim"]))
    y = L.forward_step(x, cfg, w, kc, kc.copy())
    assert y.shape == (cfg["dim"],) and np.all(np.isfinite(y))


def test_rule_chained_adjoints_equal_closed_forms():
    rng = np.random.default_rng(7)
    x, g, dy = rng.standard_normal(16), rng.uniform(0.5, 1.5, 16), rng.standard_normal(16)
    dx_r, dg_r = L.rmsnorm_bwd_by_rules(x, g, dy)
    dx_c, dg_c = L.rmsnorm_bwd(x[None], g, dy[None])
    np.testing.assert_allclose(dx_c[0], dx_r, rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(dg_c, dg_r, rtol=1e-12, atol=1e-14)
    # softmax: rule chain (incl. the reduce-max path) vs P*(dP - sum(dP*P))
    s, dp = rng.standard_normal(9), rng.standard_normal(9)
    p = L.softmax(s)
    np.testing.assert_allclose(L.softmax_bwd_by_rules(s, dp), p * (dp - np.sum(dp * p)), rtol=1e-12, atol=1e-14)
    # ... also with a tie at the maximum (every arg-max gets the cotangent; it cancels)
    s[3] = s[5] = s.max() + 1.0
    p = L.softmax(s)
    np.testing.assert_allclose(L.softmax_bwd_by_rules(s, dp), p * (dp - np.sum(dp * p)), rtol=1e-12, atol=1e-13)
    a, b, dgv = rng.standard_normal(11), rng.standard_normal(11), rng.standard_normal(11)
    da_r, db_r = L.silu_mul_bwd_by_rules(a, b, dgv)
    da_c, db_c = L.swiglu_bwd(a, b, dgv)
    np.testing.assert_allclose(da_c, da_r, rtol=1e-12)
    np.testing.assert_allclose(db_c, db_r, rtol=1e-12)


def test_special_cases():
    # rmsnorm of a constant vector c: gamma * c / sqrt(c^2 + eps)
    c, g = 3.0, np.linspace(0.5, 1.5, 8)
    np.testing.assert_allclose(L.rmsnorm_fwd(np.full((1, 8), c), g), (g * c / np.sqrt(c * c + 1e-5))[None], rtol=1e-14)
    # rope: position 0 is the identity; pair norms preserved; inverse undoes
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 5, 3, 8))
    cos, sin = L.rope_angles(5, 8)
    y = L.rope_fwd(x, cos, sin)
    np.testing.assert_allclose(y[:, 0], x[:, 0], rtol=1e-14)
    np.testing.assert_allclose(y[..., 0::2] ** 2 + y[..., 1::2] ** 2, x[..., 0::2] ** 2 + x[..., 1::2] ** 2, rtol=1e-12)
    np.testing.assert_allclose(L.rope_fwd(y, cos, sin, inverse=True), x, rtol=1e-12, atol=1e-14)
    # first frequency is 1 rad per position, last is theta^-(d-2)/d
    assert np.isclose(cos[3, 0], np.cos(3.0)) and np.isclose(sin[4, 3], np.sin(4.0 * 10000 ** (-6 / 8)))
    # attention with S = 1: out = v; softmax rows sum to one => lse consistent
    q, k, v = (rng.standard_normal((1, 2, 1, 4)) for _ in range(3))
    o, lse = L.attention_fwd(q, k, v)
    np.testing.assert_allclose(o, v, rtol=1e-14)
    # causal: the first query only sees key 0
    q, k, v = (rng.standard_normal((1, 2, 6, 4)) for _ in range(3))
    o, lse = L.attention_fwd(q, k, v)
    np.testing.assert_allclose(o[:, :, 0], v[:, :, 0], rtol=1e-13)
    s = np.einsum("bhqd,bhkd->bhqk", q, k) / 2.0
    np.testing.assert_allclose(lse[0, 0, 2], np.log(np.sum(np.exp(s[0, 0, 2, :3]))), rtol=1e-13)


def _fd(f, x, dy, h=1e-6):
    g = np.zeros_like(x)
    it = np.nditer(x, flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        xp, xm = x.copy(), x.copy()
        xp[i] += h
        xm[i] -= h
        g[i] = np.sum((f(xp) - f(xm)) * dy) / (2 * h)
    return g


def test_layer_backward_matches_finite_differences():
    cfg = {"dim": 8, "hidden_dim": 12, "n_layers": 1, "n_heads": 2}
    rng = np.random.default_rng(11)
    lw = {k: rng.standard_normal(s) * 0.4 for k, s in
          [("rms_att_weight", (8,)), ("wq", (8, 8)), ("wk", (8, 8)), ("wv", (8, 8)), ("wo", (8, 8)),
           ("rms_ffn_weight", (8,)), ("w1", (12, 8)), ("w2", (8, 12)), ("w3", (12, 8))]}
    x = rng.standard_normal((2, 3, 8))
    dy = rng.standard_normal((2, 3, 8))
    y, cache = L.layer_fwd(x, lw, 2)
    dx, gw = L.layer_bwd(dy, lw, cache, 2)
    np.testing.assert_allclose(dx, _fd(lambda t: L.layer_fwd(t, lw, 2)[0], x, dy), rtol=2e-6, atol=2e-8)
    for name in lw:
        def f(wv, name=name):
            l2 = dict(lw)
            l2[name] = wv
            return L.layer_fwd(x, l2, 2)[0]
        np.testing.assert_allclose(gw[name], _fd(f, lw[name], dy), rtol=5e-6, atol=5e-8, err_msg=name)


# ---- independent torch restatement (written against test/llama.py, not the oracle)

def _torch_model(tokens, w, cfg, logits):
    from oracle import llama_torch
    return llama_torch.model(tokens, w, cfg, logits)


@pytest.mark.parametrize("logits", [False, True])
def test_model_forward_backward_matches_torch_autograd(logits):
    cfg = CFG
    w = _weights(cfg, 9)
    rng = np.random.default_rng(4)
    tokens = rng.integers(0, cfg["vocab_size"], size=(2, 7))
    out, fc = L.model_fwd(tokens, w, cfg, logits=logits)
    dout = rng.standard_normal(out.shape)
    _, gw = L.model_bwd(dout, w, cfg, fc)
    tw = {k: torch.tensor(v, dtype=torch.float64, requires_grad=True) for k, v in w.items()}
    tout = _torch_model(torch.tensor(tokens), tw, cfg, logits)
    np.testing.assert_allclose(out, tout.detach().numpy(), rtol=1e-9, atol=1e-11)
    tout.backward(torch.tensor(dout))
    for k in gw:
        if k == "wcls" and not logits:
            continue
        np.testing.assert_allclose(gw[k], tw[k].grad.numpy(), rtol=1e-8, atol=1e-10, err_msg=k)


def test_attention_backward_adjoint_identity():
    """<J v, w> = <v, J^T w> with J v from a forward-difference of the forward."""
    rng = np.random.default_rng(21)
    q, k, v, do = (rng.standard_normal((1, 2, 5, 4)) for _ in range(4))
    dq, dk, dv = L.attention_bwd(q, k, v, do)
    tq, tk, tv = (rng.standard_normal(q.shape) for _ in range(3))
    h = 1e-6
    jp = (L.attention_fwd(q + h * tq, k + h * tk, v + h * tv)[0] - L.attention_fwd(q - h * tq, k - h * tk, v - h * tv)[0]) / (2 * h)
    assert np.isclose(np.sum(jp * do), np.sum(tq * dq) + np.sum(tk * dk) + np.sum(tv * dv), rtol=1e-7)


@pytest.mark.parametrize("pos", [1, 4])
def test_step_vjp_matches_literal_step_and_finite_differences(pos):
    """`forward_step_vjp`: its forward value is the literal step's, and its cotangents are
    the central finite differences of the literal step (float64) with respect to x, one
    weight of every kind and both caches."""
    cfg = CFG
    w = _weights(cfg, 7)
    rng = np.random.default_rng(11 + pos)
    x = rng.standard_normal(cfg["dim"])
    kc = rng.standard_normal((cfg["n_layers"], pos, cfg["dim"])) if pos > 1 else np.zeros((cfg["n_layers"], pos, cfg["dim"]))
    vc = rng.standard_normal(kc.shape) if pos > 1 else np.zeros(kc.shape)
    dy = rng.standard_normal(cfg["dim"])
    y, dx, gw, dkc, dvc = L.forward_step_vjp(x, cfg, w, kc, vc, dy)
    np.testing.assert_allclose(y, L.forward_step(x, cfg, w, kc, vc), rtol=1e-11, atol=1e-12)

    def f(xx=x, ww=w, kk=kc, vv=vc):
        return float(np.dot(L.forward_step(xx, cfg, ww, kk, vv), dy))

    def fd(arr, idx, make, h=1e-6):
        a = arr.copy(); a[idx] += h; up = f(**make(a))
        a = arr.copy(); a[idx] -= h; dn = f(**make(a))
        return (up - dn) / (2 * h)

    picks = np.random.default_rng(3)
    for idx in [tuple(picks.integers(0, n) for n in x.shape) for _ in range(4)]:
        np.testing.assert_allclose(dx[idx], fd(x, idx, lambda a: dict(xx=a)), rtol=2e-5, atol=1e-7)
    for name in list(L.LAYER_KEYS) + ["rms_final_weight"]:
        for idx in [tuple(picks.integers(0, n) for n in w[name].shape) for _ in range(3)]:
            got = gw[name][idx]
            want = fd(w[name], idx, lambda a, name=name: dict(ww={**w, name: a}))
            np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-7, err_msg=name)
    for idx in [tuple(picks.integers(0, n) for n in kc.shape) for _ in range(4)]:
        np.testing.assert_allclose(dkc[idx], fd(kc, idx, lambda a: dict(kk=a)), rtol=2e-5, atol=1e-7)
        np.testing.assert_allclose(dvc[idx], fd(vc, idx, lambda a: dict(vv=a)), rtol=2e-5, atol=1e-7)


def test_forward_mode_matches_reverse_mode_and_finite_differences():
    """`model_jvp`: <J v, w> = <v, J^T w> against `model_bwd` for random tangents of the input
    and every weight, and J v = central finite difference of `model_fwd` along v (float64)."""
    cfg, B, S = CFG, 2, 5
    w = _weights(cfg, 13)
    rng = np.random.default_rng(17)
    x = rng.standard_normal((B, S, cfg["dim"]))
    tx = rng.standard_normal(x.shape)
    tw = {k: rng.standard_normal(np.shape(v)) for k, v in w.items()}
    wvec = rng.standard_normal(x.shape)                       # cotangent on the output
    y, ty = L.model_jvp(x, w, tx, tw, cfg)
    y2, fc = L.model_fwd(x, w, cfg)
    np.testing.assert_allclose(y, y2, rtol=1e-12, atol=1e-13)
    gx, gw = L.model_bwd(wvec, w, cfg, fc)
    lhs = float(np.sum(ty * wvec))
    rhs = float(np.sum(gx * tx)) + sum(float(np.sum(gw[k] * tw[k])) for k in gw)
    np.testing.assert_allclose(lhs, rhs, rtol=1e-9)
    h = 1e-6
    up, _ = L.model_fwd(x + h * tx, {k: w[k] + h * tw[k] for k in w}, cfg)
    dn, _ = L.model_fwd(x - h * tx, {k: w[k] - h * tw[k] for k in w}, cfg)
    np.testing.assert_allclose(ty, (up - dn) / (2 * h), rtol=2e-5, atol=1e-6)


def test_cross_entropy_oracle_is_pinned():
    """The loss on the logits has no call site in the reference (the classifier is commented out at
    test/llama.py:236), so the oracle's definition is pinned by what the mathematics fixes and by library
    routines: uniform logits give log V, a shifted row gives the same loss, gradient rows sum to zero, scipy's
    logsumexp, torch's float64 cross_entropy with autograd, central finite differences and the identity
    <J v, w> = <v, J^T w>."""
    from scipy.special import logsumexp

    rng = np.random.default_rng(11)
    T, V = 7, 53
    z = rng.normal(size=(T, V)) * 3.0
    t = rng.integers(0, V, size=(T,))
    loss, lse = L.cross_entropy_fwd(z, t)
    # closed forms
    u_loss, u_lse = L.cross_entropy_fwd(np.full((2, V), 1.75), np.array([0, V - 1]))
    np.testing.assert_allclose(u_loss, np.log(V), rtol=1e-14)
    np.testing.assert_allclose(u_lse, 1.75 + np.log(V), rtol=1e-14)
    np.testing.assert_allclose(L.cross_entropy_fwd(z + 100.0, t)[0], loss, rtol=1e-12)
    big = np.zeros((1, 4)); big[0, 2] = 1000.0                      # no overflow; the hot class costs nothing
    assert L.cross_entropy_fwd(big, np.array([2]))[0][0] == 0.0 and L.cross_entropy_fwd(big, np.array([0]))[0][0] == 1000.0
    # library routines
    np.testing.assert_allclose(lse, logsumexp(z, axis=-1), rtol=1e-14)
    zt = torch.tensor(z, dtype=torch.float64, requires_grad=True)
    lt = torch.nn.functional.cross_entropy(zt, torch.tensor(t), reduction="none")
    np.testing.assert_allclose(loss, lt.detach().numpy(), rtol=1e-13)
    dl = rng.normal(size=(T,))
    (gt,) = torch.autograd.grad(lt, zt, torch.tensor(dl))
    dz = L.cross_entropy_bwd(z, t, dl)
    np.testing.assert_allclose(dz, gt.numpy(), rtol=1e-12, atol=1e-15)
    np.testing.assert_allclose(L.cross_entropy_bwd(z, t, np.ones(T)).sum(axis=-1), 0.0, atol=1e-14)
    # finite differences and forward / reverse agreement
    tz = rng.normal(size=(T, V))
    h = 1e-6
    fd = (L.cross_entropy_fwd(z + h * tz, t)[0] - L.cross_entropy_fwd(z - h * tz, t)[0]) / (2 * h)
    tl = L.cross_entropy_jvp(z, t, tz)
    np.testing.assert_allclose(tl, fd, rtol=1e-7, atol=1e-9)
    np.testing.assert_allclose((tl * dl).sum(), (tz * dz).sum(), rtol=1e-12)
    # masked tokens
    tm = t.copy(); tm[[1, 4]] = [-1, V]
    lm, _ = L.cross_entropy_fwd(z, tm)
    assert lm[1] == 0.0 and lm[4] == 0.0 and np.array_equal(np.delete(lm, [1, 4]), np.delete(loss, [1, 4]))
    dm = L.cross_entropy_bwd(z, tm, dl)
    assert not dm[1].any() and not dm[4].any()
    assert not L.cross_entropy_jvp(z, tm, tz)[[1, 4]].any()
