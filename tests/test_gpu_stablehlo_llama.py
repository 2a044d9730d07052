"""The reference's llama step (test/llama.py:35-238) handed over as StableHLO text:
`hlo_call` parses it, matches its clusters to the fused kernels and runs it; value and
all gradients are compared with the CPU oracle on the same seeded inputs, with the clusters
fused and unfused, and forward mode is tied to reverse mode by <J v, w> = <v, J^T w>."""
import numpy as np
import pytest
import torch

from oracle import llama_ref as L
from gpu_util import check, dev, host
from enzyme_ad.jax.llama_text import WEIGHT_ORDER, llama_step_text

pytestmark = pytest.mark.gpu

STORIES = {"dim": 288, "hidden_dim": 768, "n_layers": 6, "n_heads": 6, "n_kv_heads": 6, "vocab_size": 32000, "seq_len": 256}


def _inputs(cfg, pos, dt, seed, zero_cache, std):
    rng = np.random.Generator(np.random.PCG64(seed))
    w = L.make_weights(cfg, seed, std=std, embedding=False, norm_gain="uniform")
    wd, wr = {}, {}
    for k in WEIGHT_ORDER:
        wd[k], wr[k] = dev(w[k], dt)
    x, xr = dev(rng.standard_normal(cfg["dim"]), dt)
    shape = (cfg["n_layers"], pos, cfg["dim"])
    kc, kcr = dev(np.zeros(shape) if zero_cache else rng.standard_normal(shape), dt)
    vc, vcr = dev(np.zeros(shape) if zero_cache else rng.standard_normal(shape), dt)
    dy, dyr = dev(rng.standard_normal(cfg["dim"]), dt)
    return (x, wd, kc, vc, dy), (xr, wr, kcr, vcr, dyr)


def _run(cfg, pos, dt, seed, zero_cache, std, fuse):
    from enzyme_ad.jax import stablehlo, vjp

    text, order = llama_step_text(cfg, pos, dt)
    exe = stablehlo.compile_text(text, fuse=fuse)
    (x, wd, kc, vc, dy), (xr, wr, kcr, vcr, dyr) = _inputs(cfg, pos, dt, seed, zero_cache, std)

    def fn(x, weights, key_cache, value_cache):
        return exe.run([x] + [weights[k] for k in WEIGHT_ORDER] + [key_cache, value_cache])[0]

    y, f_vjp = vjp(fn, x, wd, kc, vc)
    gx, gw, gkc, gvc = f_vjp(dy)
    ry, rdx, rgw, rdkc, rdvc = L.forward_step_vjp(xr, cfg, wr, kcr, vcr, dyr)
    errs = {"y": check(y, ry, dt, "y"), "dx": check(gx, rdx, dt, "dx"), "dkc": check(gkc, rdkc, dt, "dkey_cache"),
            "dvc": check(gvc, rdvc, dt, "dvalue_cache")}
    for k in WEIGHT_ORDER:
        errs[k] = check(gw[k], rgw[k], dt, "grad " + k)
    return exe, errs


@pytest.mark.parametrize("pos,zero_cache", [(1, True), (7, False)])
@pytest.mark.parametrize("fuse", [True, False])
def test_llama_step_text_stories15m_fp32(pos, zero_cache, fuse):
    exe, errs = _run(STORIES, pos, "f32", 40 + pos, zero_cache, 0.05, fuse)
    if fuse:
        L_ = STORIES["n_layers"]
        assert exe.fused == {"rmsnorm": 2 * L_ + 1, "swiglu": L_, "rope": 2 * L_, "softmax_dot": 6 * L_, "attention_step": L_}
    else:
        assert exe.fused == {}
    print("llama text fuse=%s max rel errors" % fuse, {k: "%.2e" % v for k, v in errs.items()}, flush=True)


def test_llama_step_text_bf16_llama_head_shape():
    cfg = {"dim": 512, "hidden_dim": 1376, "n_layers": 2, "n_heads": 4, "n_kv_heads": 4, "vocab_size": 8, "seq_len": 512}
    exe, errs = _run(cfg, 300, "bf16", 12, False, 0.04, True)
    assert exe.fused["attention_step"] == 2 and exe.fused["rmsnorm"] == 5


def test_llama_step_text_through_hlo_call_and_forward_mode():
    """hlo_call on the text; jvp (clusters without a tangent kernel stay unfused) against vjp."""
    from enzyme_ad.jax import hlo_call, jvp, vjp

    cfg = dict(STORIES, n_layers=2)
    text, order = llama_step_text(cfg, 3, "f32")
    (x, wd, kc, vc, dy), (xr, wr, kcr, vcr, dyr) = _inputs(cfg, 3, "f32", 77, False, 0.05)
    args = [x] + [wd[k] for k in WEIGHT_ORDER] + [kc, vc]
    fn = lambda *a: hlo_call(*a, source=text)[0]
    y = fn(*args)
    check(y, L.forward_step(xr, cfg, wr, kcr, vcr), "f32", "y")
    rng = np.random.Generator(np.random.PCG64(5))
    tans = [dev(rng.standard_normal(tuple(a.shape)) * (0.05 if a.dim() > 1 else 1.0), "f32")[0] for a in args]
    y2, ty = jvp(fn, tuple(args), tuple(tans))
    assert torch.equal(y2, y) or check(y2, host(y), "f32", "y under forward mode") < 1e-5
    _, f_vjp = vjp(fn, *args)
    grads = f_vjp(dy)
    lhs = float(np.dot(host(ty), host(dy)))
    rhs = sum(float(np.sum(host(g) * host(t))) for g, t in zip(grads, tans))
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), abs(rhs)), (lhs, rhs)


def test_optimized_module_runs_and_matches_the_fused_run():
    """optimize_module's text (clusters as custom calls to this library's FFI targets) through
    hlo_call: value and every gradient equal those of the matched graph bit for bit."""
    from enzyme_ad.jax import hlo_call, optimize_module, vjp

    cfg = dict(STORIES, n_layers=2)
    text, order = llama_step_text(cfg, 5, "f32")
    low = optimize_module(text)
    assert low.count("stablehlo.custom_call") == 2 * 6 + 1 and "stablehlo.exponential" not in low
    (x, wd, kc, vc, dy), (xr, wr, kcr, vcr, dyr) = _inputs(cfg, 5, "f32", 88, False, 0.05)
    args = [x] + [wd[k] for k in WEIGHT_ORDER] + [kc, vc]
    outs = []
    for src in (text, low):
        y, f_vjp = vjp(lambda *a: hlo_call(*a, source=src)[0], *args)
        outs.append((y, f_vjp(dy)))
    check(outs[1][0], L.forward_step(xr, cfg, wr, kcr, vcr), "f32", "y of the lowered module")
    assert torch.equal(outs[0][0], outs[1][0])
    for a, b in zip(outs[0][1], outs[1][1]):
        assert torch.equal(a, b)
