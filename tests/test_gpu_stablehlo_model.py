"""The whole model as StableHLO text (`llama_text.llama_model_text`: tokens -> gather -> L layers sliced out of stacked
weights -> final RMSNorm -> wcls -> mean softmax cross-entropy, in the one-hot and the take_along_axis spelling)
through `hlo_call`: every cluster is matched (sibling projections as grouped launches, the loss onto the
cross-entropy kernels), value and every weight gradient equal the oracle's, and the printed primal and reverse
modules run through the library's XLA-FFI handlers."""
import numpy as np
import pytest
import torch

from oracle import llama_ref as L
from gpu_util import dev, host, check, TOL
from enzyme_ad.jax.llama_text import MODEL_ORDER, llama_model_text

pytestmark = pytest.mark.gpu

C1 = dict(dim=288, hidden_dim=768, n_layers=6, n_heads=6, n_kv_heads=6, vocab_size=32000)          # stories15M, fp32
C4_REDUCED = dict(dim=768, hidden_dim=2048, n_layers=2, n_heads=12, n_kv_heads=12, vocab_size=32000)  # stories110M width, 2 layers


def _weights(cfg, dt, seed):
    w = L.make_weights(cfg, seed, std=0.02, norm_gain="uniform")
    wd, wr = {}, {}
    for k in MODEL_ORDER:
        wd[k], wr[k] = dev(w[k], dt)
    return wd, wr


def _tokens(cfg, B, S, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    tok, tgt = rng.integers(0, cfg["vocab_size"], size=(B, S)), rng.integers(0, cfg["vocab_size"], size=(B, S))
    return tok, tgt, torch.from_numpy(tok.astype(np.int32)).cuda(), torch.from_numpy(tgt.astype(np.int32)).cuda()


@pytest.mark.parametrize("cfg,B,S,dt", [(C1, 1, 256, "f32"), (C4_REDUCED, 2, 128, "bf16")])
@pytest.mark.parametrize("loss", ["onehot", "gather"])
def test_model_text_loss_and_every_gradient(cfg, B, S, dt, loss):
    from enzyme_ad.jax import hlo_call, stablehlo, vjp
    text, order = llama_model_text(cfg, B, S, dt, loss)
    exe = stablehlo.compile_text(text)
    Lc = cfg["n_layers"]
    assert exe.fused == {"swiglu": Lc, "rmsnorm_rows": 2 * Lc + 1, "rope_rows": 2 * Lc, "attention": Lc, "cross_entropy": 1,
                         "linear": 7 * Lc + 1, "linear_group": 2 * Lc}
    run_names = [o.name for o in exe.funcs["main"].run_ops]
    assert run_names.count("emi.select") == 9 * Lc and "slice" not in run_names and "dot_general" not in run_names
    wd, wr = _weights(cfg, dt, 11)
    tok, tgt, tokd, tgtd = _tokens(cfg, B, S, 12)
    fn = lambda w: hlo_call(tokd, *[w[k] for k in MODEL_ORDER], tgtd, source=text)[0]
    out, f_vjp = vjp(fn, wd)
    logits, fcache = L.model_fwd(tok, wr, cfg, logits=True)
    rows, _ = L.cross_entropy_fwd(logits.reshape(B * S, -1), tgt.reshape(-1))
    want = float(rows.mean())
    assert abs(float(out) - want) <= TOL[dt] * abs(want), (float(out), want)
    (gw,) = f_vjp(torch.ones((), device="cuda", dtype=out.dtype))
    dlogits = L.cross_entropy_bwd(logits.reshape(B * S, -1), tgt.reshape(-1), np.full(B * S, 1.0 / (B * S))).reshape(logits.shape)
    _, rgw = L.model_bwd(dlogits, wr, cfg, fcache)
    for k in MODEL_ORDER:
        e = check(gw[k], rgw[k], dt, "d loss / d " + k)
        print("model text (%s, %s): d%s max relative error %.3e" % (dt, loss, k, e), flush=True)


def test_model_text_logits_and_printed_modules_through_the_ffi_handlers():
    """Logits form at a reduced size: value and gradients against the oracle, then the printed primal and reverse
    modules (the sub-blocks of a layer on the targets with RoPE and SwiGLU in GEMM epilogues, the lookup as `stablehlo.gather`, its adjoint as
    `emi_embedding_bwd`) with every custom call
    served by the library's FFI handler, against `hlo_call` on the same text."""
    from enzyme_ad.jax import hlo_call, optimize_module, primitives as P, vjp
    from test_gpu_ffi_module import _ffi_executable, _close
    cfg = dict(dim=256, hidden_dim=704, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=1000)
    B, S, dt = 2, 70, "bf16"
    text, order = llama_model_text(cfg, B, S, dt, None)
    wd, wr = _weights(cfg, dt, 21)
    tok, _, tokd, _ = _tokens(cfg, B, S, 22)
    args = [tokd] + [wd[k] for k in MODEL_ORDER]
    fn = lambda w: hlo_call(tokd, *[w[k] for k in MODEL_ORDER], source=text)[0]
    out, f_vjp = vjp(fn, wd)
    ref, fcache = L.model_fwd(tok, wr, cfg, logits=True)
    check(out, ref, dt, "logits")
    dout, doutr = dev(np.random.Generator(np.random.PCG64(23)).standard_normal(ref.shape), dt)
    (gw,) = f_vjp(dout)
    _, rgw = L.model_bwd(doutr, wr, cfg, fcache)
    for k in MODEL_ORDER:
        check(gw[k], rgw[k], dt, "d" + k)
    low = optimize_module(text)
    assert low.count("@emi_gemm_rope") == 2 * cfg["n_layers"] and low.count("@emi_gemm_swiglu_fwd") == cfg["n_layers"]
    assert low.count('"stablehlo.gather"') == 1
    assert "stablehlo.dot_general" not in low and "stablehlo.exponential" not in low
    active = [False] + [True] * len(MODEL_ORDER)
    fwd_pipe = P.forward_mode_pipeline(P.JaXPipeline(), active, 1)
    rev = optimize_module(text, P.reverse_mode_pipeline(fwd_pipe, [True]).pass_pipeline())
    assert rev.count("@emi_attn_bwd_rope") == cfg["n_layers"] and rev.count("@emi_gemm_swiglu_bwd") == cfg["n_layers"]
    assert rev.count("@emi_embedding_bwd") == 1 and "@emi_rope" not in rev
    for name, prog, ins in (("primal", low, args), ("reverse", rev, args + [dout])):
        exe, calls = _ffi_executable(prog)
        got = exe.run(ins)
        torch.cuda.synchronize()
        want = hlo_call(*ins, source=prog)
        assert len(calls) == prog.count("stablehlo.custom_call") and "emi_gemm_rope" in calls and "emi_gemm_swiglu_fwd" in calls, name
        for a, b in zip(got, want):
            assert torch.equal(a, b) if name == "primal" else _close(a, b, 2e-2), name
    # the reverse program's gradients are the tape's
    sym = hlo_call(*(args + [dout]), source=rev)
    for k, g in zip(MODEL_ORDER, sym):
        assert _close(g, gw[k], 2e-2), "reverse program, d" + k
