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
        assert exe.fused == {"rmsnorm": 2 * L_ + 1, "swiglu": L_, "rope": 2 * L_, "softmax_dot": 6 * L_, "attention_step": L_,
                             "linear": 7 * L_}
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
    assert low.count("stablehlo.custom_call") == 2 * (6 + 7) + 1 and "stablehlo.exponential" not in low
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


@pytest.mark.parametrize("dt,pos", [("f32", 1), ("f32", 7), ("bf16", 40)])
def test_reverse_module_of_the_llama_step(dt, pos):
    """The symbolic reverse-mode module (forward recomputation + adjoint custom calls, printed
    as StableHLO text) run through hlo_call: its 13 cotangents against the oracle's
    forward_step_vjp and against the tape's vjp of the same text."""
    from enzyme_ad.jax import hlo_call, stablehlo_ad, vjp

    cfg = dict(STORIES, n_layers=3)
    text, order = llama_step_text(cfg, pos, dt)
    rev = stablehlo_ad.reverse_module_text(text)
    (x, wd, kc, vc, dy), (xr, wr, kcr, vcr, dyr) = _inputs(cfg, pos, dt, 90 + pos, pos == 1, 0.05)
    args = [x] + [wd[k] for k in WEIGHT_ORDER] + [kc, vc]
    grads = hlo_call(*(args + [dy]), source=rev)
    assert len(grads) == len(args)
    ry, rdx, rgw, rdkc, rdvc = L.forward_step_vjp(xr, cfg, wr, kcr, vcr, dyr)
    want = [rdx] + [rgw[k] for k in WEIGHT_ORDER] + [rdkc, rdvc]
    for name, g, w in zip(order, grads, want):
        check(g, w, dt, "reverse module, cotangent of " + name)
    _, f_vjp = vjp(lambda *a: hlo_call(*a, source=text)[0], *args)
    for name, g, t in zip(order, grads, f_vjp(dy)):
        check(g, host(t), dt, "reverse module vs tape, " + name, factor=0.1 if dt == "f32" else 1.0)


def test_reverse_module_of_generic_operators_matches_the_tape():
    """A module of generic operators only (broadcasts, reductions, transposes, slices with
    strides, concatenation, a batched product, unary maps): symbolic reverse mode against the
    tape's reverse mode."""
    from enzyme_ad.jax import hlo_call, stablehlo_ad, vjp

    text = """
    func.func @main(%a: tensor<4x6xf32>, %b: tensor<6xf32>, %w: tensor<2x3x5xf32>) -> (tensor<4x6xf32>, tensor<2x4x5xf32>, tensor<f32>) {
      %bb = stablehlo.broadcast_in_dim %b, dims = [1] : (tensor<6xf32>) -> tensor<4x6xf32>
      %m = stablehlo.multiply %a, %bb : tensor<4x6xf32>
      %e = stablehlo.exponential %m : tensor<4x6xf32>
      %t = stablehlo.tanh %a : tensor<4x6xf32>
      %d = stablehlo.divide %e, %t : tensor<4x6xf32>
      %z = stablehlo.constant dense<0.000000e+00> : tensor<f32>
      %rs = stablehlo.reduce(%d init: %z) applies stablehlo.add across dimensions = [1] : (tensor<4x6xf32>, tensor<f32>) -> tensor<4xf32>
      %rb = stablehlo.broadcast_in_dim %rs, dims = [0] : (tensor<4xf32>) -> tensor<4x6xf32>
      %lg = stablehlo.logistic %rb : tensor<4x6xf32>
      %o1 = stablehlo.subtract %d, %lg : tensor<4x6xf32>
      %s0 = stablehlo.slice %a [0:4, 0:6:2] : (tensor<4x6xf32>) -> tensor<4x3xf32>
      %s1 = stablehlo.slice %m [0:4, 3:6] : (tensor<4x6xf32>) -> tensor<4x3xf32>
      %cc = stablehlo.concatenate %s0, %s1, dim = 0 : (tensor<4x3xf32>, tensor<4x3xf32>) -> tensor<8x3xf32>
      %c3 = stablehlo.reshape %cc : (tensor<8x3xf32>) -> tensor<2x4x3xf32>
      %o2 = stablehlo.dot_general %c3, %w, batching_dims = [0] x [0], contracting_dims = [2] x [1] : (tensor<2x4x3xf32>, tensor<2x3x5xf32>) -> tensor<2x4x5xf32>
      %tr = stablehlo.transpose %o2, dims = [2, 0, 1] : (tensor<2x4x5xf32>) -> tensor<5x2x4xf32>
      %sq = stablehlo.multiply %tr, %tr : tensor<5x2x4xf32>
      %o3 = stablehlo.reduce(%sq init: %z) applies stablehlo.add across dimensions = [0, 1, 2] : (tensor<5x2x4xf32>, tensor<f32>) -> tensor<f32>
      return %o1, %o2, %o3 : tensor<4x6xf32>, tensor<2x4x5xf32>, tensor<f32>
    }"""
    rng = np.random.Generator(np.random.PCG64(7))
    a = dev(rng.uniform(0.5, 1.5, (4, 6)), "f32")[0]
    b = dev(rng.standard_normal(6) * 0.3, "f32")[0]
    w = dev(rng.standard_normal((2, 3, 5)), "f32")[0]
    cts = (dev(rng.standard_normal((4, 6)), "f32")[0], dev(rng.standard_normal((2, 4, 5)), "f32")[0], dev(rng.standard_normal(()), "f32")[0].reshape(()))
    outs, f_vjp = vjp(lambda *xs: tuple(hlo_call(*xs, source=text)), a, b, w)
    tape = f_vjp(cts)
    rev = stablehlo_ad.reverse_module_text(text)
    sym = hlo_call(a, b, w, *cts, source=rev)
    for name, g, t in zip("abw", sym, tape):
        check(g, host(t), "f32", "symbolic vs tape, " + name, factor=0.1)


def test_forward_module_of_the_llama_step():
    """The symbolic forward-mode module (each argument followed by its tangent; results
    interleaved with their tangents) through hlo_call against the tape's jvp of the same text,
    with every argument active and with only the weights active."""
    from enzyme_ad.jax import hlo_call, jvp, stablehlo_ad

    cfg = dict(STORIES, n_layers=2)
    text, order = llama_step_text(cfg, 6, "f32")
    (x, wd, kc, vc, dy), _ = _inputs(cfg, 6, "f32", 71, False, 0.05)
    args = [x] + [wd[k] for k in WEIGHT_ORDER] + [kc, vc]
    rng = np.random.Generator(np.random.PCG64(8))
    tans = [dev(rng.standard_normal(tuple(a.shape)) * (0.05 if a.dim() > 1 else 1.0), "f32")[0] for a in args]
    fn = lambda *a: hlo_call(*a, source=text)[0]
    for active in ([True] * len(args), [False] + [True] * (len(args) - 3) + [False, False]):
        fwd = stablehlo_ad.forward_module_text(text, arg_active=active)
        flat = []
        for a, t, on in zip(args, tans, active):
            flat += [a, t] if on else [a]
        y, ty = hlo_call(*flat, source=fwd)
        y_ref, ty_ref = jvp(fn, tuple(args), tuple(t if on else None for t, on in zip(tans, active)))
        check(y, host(y_ref), "f32", "forward module, primal", factor=0.1)
        check(ty, host(ty_ref), "f32", "forward module, tangent", factor=0.1)
