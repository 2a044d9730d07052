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
        assert exe.fused == {"rmsnorm_rows": 2, "rope_rows": 2, "attention": 1, "swiglu": 1, "linear": 7, "linear_group": 2}
        names = sorted(o.name for o in exe.funcs["main"].ops)                 # the hand-wired llama.layer, operator for operator
        assert names == sorted(["emi.linear"] * 2 + ["emi.linear_group"] * 2 + ["emi.rmsnorm_rows"] * 2 + ["emi.rope_rows"] * 2 +
                               ["emi.attention", "emi.swiglu", "return"])      # q, k, v and w1, w3 as grouped launches
    print("layer text fuse=%s max rel errors" % fuse, {k: "%.2e" % v for k, v in errs.items()}, flush=True)


def test_layer_text_bf16_head_dim_128_runs_the_mfma_kernels():
    cfg = {"dim": 512, "hidden_dim": 1376, "n_heads": 4}
    exe, errs = _case(cfg, 2, 300, "bf16", 6, True)
    assert exe.fused["attention"] == 1 and exe.fused["rope_rows"] == 2


def test_layer_text_at_a_size_the_fused_epilogues_serve():
    """4096 tokens x dim 3072 (24 heads x 128): the run list's `emi.attention_block` and `emi.ffn` take the kernels with
    RoPE and SwiGLU in their epilogues.  Value and every gradient against the hand-wired `llama.layer` on the same
    operands (the same kernels; the angle table comes from the module's constants instead of the device kernel)."""
    from enzyme_ad.jax import llama, stablehlo, vjp
    cfg = {"dim": 3072, "hidden_dim": 3072, "n_heads": 24}
    B, S, dt = 16, 256, "bf16"
    text, order = llama_layer_text(cfg, B, S, dt)
    exe = stablehlo.compile_text(text)
    assert sorted(o.name for o in exe.funcs["main"].run_ops) == sorted(["emi.rmsnorm_rows"] * 2 + ["emi.attention_block", "emi.linear",
                                                                        "emi.ffn", "return"])
    rng = np.random.Generator(np.random.PCG64(11))
    D, H = cfg["dim"], cfg["hidden_dim"]
    shapes = {"rms_att_weight": (D,), "wq": (D, D), "wk": (D, D), "wv": (D, D), "wo": (D, D), "rms_ffn_weight": (D,), "w1": (H, D),
              "w2": (D, H), "w3": (H, D)}
    lw = {k: dev(rng.uniform(0.5, 1.5, shapes[k]) if k.startswith("rms") else rng.standard_normal(shapes[k]) * 0.02, dt)[0]
          for k in LAYER_ORDER}
    x = dev(rng.standard_normal((B, S, D)), dt)[0]
    dy = dev(rng.standard_normal((B, S, D)), dt)[0]
    y, f_vjp = vjp(lambda x, w: exe.run([x] + [w[k] for k in LAYER_ORDER])[0], x, lw)
    gx, gw = f_vjp(dy)
    y0, f0 = vjp(lambda x, w: llama.layer(x, w, cfg["n_heads"]), x, lw)
    gx0, gw0 = f0(dy)
    # the two tables differ in the last bit of an fp32 entry here and there, which flips bf16 roundings: agreement to
    # about one bf16 unit of the largest element is what identical kernels give
    check(y, host(y0), dt, "y")
    check(gx, host(gx0), dt, "dx")
    for k in LAYER_ORDER:
        check(gw[k], host(gw0[k]), dt, "grad " + k)


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


def test_layer_text_lowered_and_symbolic_programs():
    """optimize_module's three programs for the batched layer (clusters as emi_rmsnorm_fwd / emi_gemm_rope /
    emi_attn_fwd / emi_gemm_swiglu_fwd custom calls; the reverse program with emi_attn_bwd_rope, emi_gemm_swiglu_bwd
    & co.; the forward program with emi_attn_jvp & co.) through hlo_call against the tape."""
    from enzyme_ad.jax import hlo_call, jvp, optimize_module, stablehlo_ad, vjp
    from enzyme_ad.jax import primitives as P

    cfg = {"dim": 256, "hidden_dim": 704, "n_heads": 2}
    for dt, tol in (("f32", 1e-5), ("bf16", 2e-2)):
        text, order = llama_layer_text(cfg, 2, 70, dt)
        rng = np.random.Generator(np.random.PCG64(3))
        shapes = [(2, 70, 256), (256,), (256, 256), (256, 256), (256, 256), (256, 256), (256,), (704, 256), (256, 704), (704, 256)]
        args = [dev(rng.uniform(0.5, 1.5, s) if len(s) == 1 else rng.standard_normal(s) * (1.0 if len(s) == 3 else 0.05), dt)[0] for s in shapes]
        tans = [dev(rng.standard_normal(s) * (1.0 if len(s) != 2 else 0.05), dt)[0] for s in shapes]
        dy = dev(rng.standard_normal(shapes[0]), dt)[0]
        fn = lambda *a: hlo_call(*a, source=text)[0]
        y, f_vjp = vjp(fn, *args)
        grads = f_vjp(dy)
        low = optimize_module(text)
        assert low.count("stablehlo.custom_call") == 10 and low.count("@emi_gemm_rope") == 2 and low.count("@emi_gemm_swiglu_fwd") == 1
        assert "stablehlo.exponential" not in low and "stablehlo.dot_general" not in low
        y_low = hlo_call(*args, source=low)[0]
        assert torch.equal(y_low, y)
        fwd_pipe = P.forward_mode_pipeline(P.JaXPipeline(), [True] * len(args), 1)
        rev = optimize_module(text, P.reverse_mode_pipeline(fwd_pipe, [True]).pass_pipeline())
        assert rev.count("@emi_attn_bwd_rope") == 1 and rev.count("@emi_gemm_swiglu_bwd") == 1 and rev.count("@emi_rmsnorm_bwd") == 2
        assert "@emi_rope" not in rev and "@emi_swiglu_bwd" not in rev
        sym = hlo_call(*(args + [dy]), source=rev)
        for name, g, t in zip(order, sym, grads):
            e = float((g.float() - t.float()).abs().max() / t.float().abs().max())
            assert e <= tol, "reverse program, %s: %.3e" % (name, e)
        fwd = optimize_module(text, fwd_pipe.pass_pipeline())
        assert fwd.count("@emi_attn_jvp") == 1
        flat = [v for a, t in zip(args, tans) for v in (a, t)]
        y_f, ty_f = hlo_call(*flat, source=fwd)
        _, ty = jvp(fn, tuple(args), tuple(tans))
        e = float((ty_f.float() - ty.float()).abs().max() / ty.float().abs().max())
        assert torch.equal(y_f, y) and e <= tol, "forward program: %.3e" % e
