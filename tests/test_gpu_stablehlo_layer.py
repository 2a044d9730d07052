"""One decoder layer over a batch of sequences handed over as StableHLO text (RMSNorm over the
last index, projections, pair rotation with constant tables, batched scores with a causal mask
from iotas, softmax, SwiGLU): matched to the fused kernels and operator by operator, value and
all ten gradients against the oracle's layer_fwd / layer_bwd."""
import numpy as np
import pytest
import torch

from oracle import llama_ref as L
from gpu_util import check, dev, host
from enzyme_ad.jax.llama_text import LAYER_ORDER, llama_layer_text

pytestmark = pytest.mark.gpu


def _case(cfg, B, S, dt, seed, fuse):
    from enzyme_ad.jax import stablehlo, vjp

    text, order = llama_layer_text(cfg, B, S, dt)
    exe = stablehlo.compile_text(text, fuse=fuse)
    rng = np.random.Generator(np.random.PCG64(seed))
    D, H = cfg["dim"], cfg["hidden_dim"]
    shapes = {"rms_att_weight": (D,), "wq": (D, D), "wk": (D, D), "wv": (D, D), "wo": (D, D), "rms_ffn_weight": (D,), "w1": (H, D),
              "w2": (D, H), "w3": (H, D)}
    lw, lwr = {}, {}
    for k in LAYER_ORDER:
        a = rng.uniform(0.5, 1.5, shapes[k]) if k.startswith("rms") else rng.standard_normal(shapes[k]) * 0.05
        lw[k], lwr[k] = dev(a, dt)
    x, xr = dev(rng.standard_normal((B, S, D)), dt)
    dy, dyr = dev(rng.standard_normal((B, S, D)), dt)
    y, f_vjp = vjp(lambda x, w: exe.run([x] + [w[k] for k in LAYER_ORDER])[0], x, lw)
    gx, gw = f_vjp(dy)
    ry, cache = L.layer_fwd(xr, lwr, cfg["n_heads"])
    rdx, rgw = L.layer_bwd(dyr, lwr, cache, cfg["n_heads"])
    errs = {"y": check(y, ry, dt, "y"), "dx": check(gx, rdx, dt, "dx")}
    for k in LAYER_ORDER:
        errs[k] = check(gw[k], rgw[k], dt, "grad " + k)
    return exe, errs


@pytest.mark.parametrize("fuse", [True, False])
def test_layer_text_fp32(fuse):
    cfg = {"dim": 128, "hidden_dim": 352, "n_heads": 2}
    exe, errs = _case(cfg, 2, 40, "f32", 5, fuse)
    if fuse:
        assert exe.fused == {"rmsnorm_rows": 2, "rope_rows": 2, "attention": 1, "swiglu": 1}
        names = sorted(o.name for o in exe.funcs["main"].ops)
        assert names == sorted(["dot_general"] * 7 + ["emi.rmsnorm_rows"] * 2 + ["emi.rope_rows"] * 2 + ["add"] * 2 +
                               ["emi.attention", "emi.swiglu", "return"])
    print("layer text fuse=%s max rel errors" % fuse, {k: "%.2e" % v for k, v in errs.items()}, flush=True)


def test_layer_text_bf16_head_dim_128_runs_the_mfma_kernels():
    cfg = {"dim": 512, "hidden_dim": 1376, "n_heads": 4}
    exe, errs = _case(cfg, 2, 300, "bf16", 6, True)
    assert exe.fused["attention"] == 1 and exe.fused["rope_rows"] == 2


def test_layer_text_forward_mode_adjoint_identity():
    from enzyme_ad.jax import hlo_call, jvp, vjp

    cfg = {"dim": 128, "hidden_dim": 352, "n_heads": 2}
    text, order = llama_layer_text(cfg, 1, 33, "f32")
    rng = np.random.Generator(np.random.PCG64(9))
    shapes = [(1, 33, 128), (128,), (128, 128), (128, 128), (128, 128), (128, 128), (128,), (352, 128), (128, 352), (352, 128)]
    args = [dev(rng.uniform(0.5, 1.5, s) if len(s) == 1 else rng.standard_normal(s) * (1.0 if len(s) == 3 else 0.05), "f32")[0] for s in shapes]
    tans = [dev(rng.standard_normal(s) * (1.0 if len(s) != 2 else 0.05), "f32")[0] for s in shapes]
    dy = dev(rng.standard_normal(shapes[0]), "f32")[0]
    fn = lambda *a: hlo_call(*a, source=text)[0]
    _, ty = jvp(fn, tuple(args), tuple(tans))
    _, f_vjp = vjp(fn, *args)
    grads = f_vjp(dy)
    lhs = float(np.sum(host(ty) * host(dy)))
    rhs = sum(float(np.sum(host(g) * host(t))) for g, t in zip(grads, tans))
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), abs(rhs)), (lhs, rhs)
