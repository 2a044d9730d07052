"""GPU parity of the composed path: decoder layer and whole model, forward and
VJP through `enzyme_jax_ir` + `vjp`, against the CPU oracle (same seeded
inputs).  Mirrors the reference's test/llama.py fixture: primal, then
gradients for a given output cotangent (`splatvjp_noprim`, test/test_utils.py
:508-514), compared leaf by leaf (`recursive_check`, :522-550)."""
import numpy as np
import pytest
import torch

from oracle import llama_ref as L
from gpu_util import dev, host, check, rel_err

pytestmark = pytest.mark.gpu


def _to_dev_tree(w, dt):
    d, r = {}, {}
    for k, a in w.items():
        d[k], r[k] = dev(a, dt)
    return d, r


def _run_model(cfg, B, S, dt, seed, logits, tokens_in=True, std=0.02, norm_gain="normal"):
    from enzyme_ad.jax import enzyme_jax_ir, JaXPipeline, vjp
    from enzyme_ad.jax import llama
    w = L.make_weights(cfg, seed, std=std, norm_gain=norm_gain)
    wd, wr = _to_dev_tree(w, dt)
    rng = np.random.Generator(np.random.PCG64(seed + 1000))
    if tokens_in:
        tok = rng.integers(0, cfg["vocab_size"], size=(B, S))
        xin, xin_ref = torch.from_numpy(tok.astype(np.int32)).cuda(), tok
    else:
        xin, xin_ref = dev(rng.standard_normal((B, S, cfg["dim"])), dt)

    @enzyme_jax_ir(pipeline_options=JaXPipeline(), inner_jit=False)
    def fn(x, weights):
        return llama.forward(x, cfg, weights, logits=logits)

    out = fn(xin, wd)                                      # primal
    ref, fc = L.model_fwd(xin_ref, wr, cfg, logits=logits)
    e_out = check(out, ref, dt, "model output")
    dout, dout_ref = dev(rng.standard_normal(ref.shape), dt)
    out2, f_vjp = vjp(fn, xin, wd)
    assert torch.equal(out2, out)                          # deterministic kernels
    gx, gw = f_vjp(dout)
    rgx, rgw = L.model_bwd(dout_ref, wr, cfg, fc)
    errs = {"out": e_out}
    if not tokens_in:
        errs["dx"] = check(gx, rgx, dt, "dx")
    for k in rgw:
        errs[k] = check(gw[k], rgw[k], dt, "grad " + k)
    print("max rel errors", {k: "%.2e" % v for k, v in errs.items()}, flush=True)
    return errs


def test_c1_stories15m_fp32_tokens_logits():
    """Configuration C1: dim 288, hidden 768, 6 layers, 6 heads of 48, vocab 32000,
    seq 256, batch 1, fp32, weights N(0, 0.02), cotangent N(0,1) on the logits."""
    cfg = {"dim": 288, "hidden_dim": 768, "n_layers": 6, "n_heads": 6, "n_kv_heads": 6,
           "vocab_size": 32000, "seq_len": 256}
    _run_model(cfg, 1, 256, "f32", seed=1, logits=True)


def test_reference_fixture_shape_fp32_uniform_weights():
    """The reference fixture's distributions (uniform[0,1) weights, no logits, output =
    final RMSNorm; test/llama.py:266-291) on a short batched sequence."""
    cfg = {"dim": 288, "hidden_dim": 768, "n_layers": 2, "n_heads": 6, "n_kv_heads": 6,
           "vocab_size": 64, "seq_len": 16}
    from enzyme_ad.jax import vjp, llama
    rng = np.random.default_rng(0)
    w = {k: rng.uniform(0, 1, size=v.shape) for k, v in L.make_weights(cfg, 0, embedding=False).items()}
    wd, wr = _to_dev_tree(w, "f32")
    x, xr = dev(rng.uniform(0, 1, size=(1, 16, 288)), "f32")
    dy, dyr = dev(rng.uniform(0, 1, size=(1, 16, 288)), "f32")
    out, f_vjp = vjp(lambda a, b: llama.forward(a, cfg, b), x, wd)
    ref, fc = L.model_fwd(xr, wr, cfg)
    check(out, ref, "f32", "fixture output")
    gx, gw = f_vjp(dy)
    rgx, rgw = L.model_bwd(dyr, wr, cfg, fc)
    # All-positive weights make this problem badly conditioned in fp32 (dx ~ 1e-6 after
    # cancellation); the reference compares it with allclose(atol=1e-3, rtol=1e-3)
    # (test/llama.py:318-319, test/test_utils.py:522-550) and so does this test.
    assert np.allclose(host(gx), rgx, atol=1e-3, rtol=1e-3)
    print("fixture dx max rel err %.2e" % rel_err(host(gx), rgx), flush=True)
    for k in rgw:
        if k != "wcls":
            assert np.allclose(host(gw[k]), rgw[k], atol=1e-3, rtol=1e-3), k
            print("fixture grad %s max rel err %.2e" % (k, rel_err(host(gw[k]), rgw[k])), flush=True)


def test_small_llama_bf16_mfma_paths():
    """bf16, head_dim 128 and 64 through the MFMA attention and GEMM kernels."""
    for nh in (2, 4):
        cfg = {"dim": 256, "hidden_dim": 512, "n_layers": 2, "n_heads": nh, "n_kv_heads": nh,
               "vocab_size": 512, "seq_len": 256}
        _run_model(cfg, 2, 256, "bf16", seed=4 + nh, logits=True, norm_gain="uniform")


def test_layer_bf16_llama7b_head_shape():
    """One layer with 7B head geometry (head_dim 128) at reduced width; activations N(0,1)."""
    cfg = {"dim": 512, "hidden_dim": 1376, "n_layers": 1, "n_heads": 4, "n_kv_heads": 4,
           "vocab_size": 8, "seq_len": 384}
    _run_model(cfg, 2, 384, "bf16", seed=5, logits=False, tokens_in=False, norm_gain="uniform")
