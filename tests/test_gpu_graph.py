"""HIP-graph capture of the reference's step (forward + reverse mode): every replay is checked
against the eager result on fresh inputs, with eager work and synchronisations between
replays."""
import numpy as np
import pytest
import torch

from oracle import llama_ref as L
from gpu_util import dev, host

pytestmark = pytest.mark.gpu

CFG = {"dim": 288, "hidden_dim": 768, "n_layers": 6, "n_heads": 6, "n_kv_heads": 6, "vocab_size": 32000, "seq_len": 256}


def _inputs(seed, pos):
    rng = np.random.Generator(np.random.PCG64(seed))
    w = L.make_weights(CFG, seed, std=0.05, embedding=False, norm_gain="uniform")
    wd = {k: dev(a, "f32")[0] for k, a in w.items()}
    x, dy = (dev(rng.standard_normal(CFG["dim"]), "f32")[0] for _ in range(2))
    kc, vc = (dev(rng.standard_normal((CFG["n_layers"], pos, CFG["dim"])), "f32")[0] for _ in range(2))
    return x, wd, kc, vc, dy


def _flat(out):
    y, (gx, gw, gkc, gvc) = out
    return [y, gx, gkc, gvc] + [gw[k] for k in sorted(gw)]


def test_captured_step_replays_match_eager():
    from enzyme_ad.jax import llama, vjp
    from enzyme_ad.jax.graph import capture

    def step(x, w, kc, vc, dy):
        y, f_vjp = vjp(lambda a, b, c, d: llama.forward_step(a, CFG, b, c, d), x, w, kc, vc)
        return y, f_vjp(dy)

    g = capture(step, *_inputs(1, 5))
    for seed in (2, 3, 4, 5):
        args = _inputs(seed, 5)
        eager = [t.clone() for t in _flat(step(*args))]
        torch.cuda.synchronize()
        junk = torch.randn(1 << 20, device="cuda").sin_()            # unrelated eager work between replays
        got = _flat(g(*args))
        torch.cuda.synchronize()
        for a, b in zip(got, eager):
            assert torch.equal(a, b)
        del junk
    assert g.replays == 4
    with pytest.raises(ValueError):
        g(*_inputs(6, 6))                                            # another cache length: shapes are fixed at capture


def test_captured_text_step_replays_match_eager():
    """The same through the StableHLO text front end (parsed-module constants are uploaded in
    the eager run before capture)."""
    from enzyme_ad.jax import hlo_call, vjp
    from enzyme_ad.jax.graph import capture
    from enzyme_ad.jax.llama_text import WEIGHT_ORDER, llama_step_text

    cfg = dict(CFG, n_layers=2)
    text, order = llama_step_text(cfg, 5)

    def step(dy, *args):
        y, f_vjp = vjp(lambda *a: hlo_call(*a, source=text)[0], *args)
        return (y,) + tuple(f_vjp(dy))

    def inputs(seed):
        x, wd, kc, vc, dy = _inputs(seed, 5)
        return [dy, x] + [wd[k][:2].contiguous() for k in WEIGHT_ORDER[:-1]] + [wd["rms_final_weight"], kc[:2].contiguous(), vc[:2].contiguous()]

    g = capture(step, *inputs(1))
    for seed in (7, 8, 9):
        args = inputs(seed)
        eager = [t.clone() for t in step(*args)]
        torch.cuda.synchronize()
        got = g(*args)
        torch.cuda.synchronize()
        for a, b in zip(got, eager):
            assert torch.equal(a, b)
