"""GPU checks at the full sizes of the benchmark configurations, where the CPU oracle
cannot redo the whole computation in seconds: oracle comparisons on the parts it can redo
(sampled rows, sampled queries, causal prefixes of a sequence) and size-independent
properties for the rest (rows of P sum to one, RoPE round trip, exact linearity of the
reverse pass in its cotangent, causality, and <J v, w> = <v, J^T w> between the forward-mode
and reverse-mode kernels)."""
import numpy as np
import pytest
import torch

from oracle import llama_ref as L
from gpu_util import dev, host, check, rel_err, TDTYPE

pytestmark = pytest.mark.gpu


def _randn(shape, dt, seed, scale=1.0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, device="cuda", generator=g) * scale).to(TDTYPE[dt])


def _dot(a, b):
    return float((a.double() * b.double()).sum().item())


@pytest.mark.parametrize("dt", ["bf16", "f32"])
def test_c2_rmsnorm_rope_full_size(dt):
    """x [16, 2048, 4096]: sampled rows against the oracle, dgamma against a float64 column sum,
    RoPE round trip and pair-norm preservation over the whole tensor."""
    from enzyme_ad.jax import ops
    B, S, D, h = 16, 2048, 4096, 32
    x, dy = _randn((B, S, D), dt, 2), _randn((B, S, D), dt, 3)
    gam = (torch.rand(D, device="cuda", generator=torch.Generator(device="cuda").manual_seed(4)) + 0.5).to(TDTYPE[dt])
    with ops.Tape() as tape:
        y = ops.rmsnorm(x, gam)
    dx, dg = tape.backward([y], [dy], [x, gam])
    rows = [0, 1, 2047, 2048, 12345, B * S - 1]
    xs, dys = host(x.reshape(-1, D)[rows]), host(dy.reshape(-1, D)[rows])
    gr = host(gam)
    check(y.reshape(-1, D)[rows], L.rmsnorm_fwd(xs, gr), dt, "rmsnorm rows")
    check(dx.reshape(-1, D)[rows], L.rmsnorm_bwd(xs, gr, dys)[0], dt, "rmsnorm dx rows")
    x64, dy64 = x.reshape(-1, D).double(), dy.reshape(-1, D).double()
    r = torch.rsqrt((x64 * x64).mean(dim=1, keepdim=True) + 1e-5)
    check(dg, (dy64 * x64 * r).sum(dim=0).cpu().numpy(), dt, "dgamma over 32768 rows")
    with ops.Tape() as tape:
        z = ops.rope(x, h)
    back = ops.rope(z, h, inverse=True)
    assert rel_err(host(back[:, ::97]), host(x[:, ::97])) <= (2e-2 if dt == "bf16" else 1e-5)
    pos = [0, 1, 777, 2047]
    cos, sin = L.rope_angles(S, D // h)
    ref = L.rope_fwd(host(x[3, pos]).reshape(1, len(pos), h, D // h), cos[pos], sin[pos])
    check(z[3, pos], ref.reshape(len(pos), D), dt, "rope rows")
    (dxr,) = tape.backward([z], [dy], [x])
    check(dxr[5, pos], L.rope_bwd(host(dy[5, pos]).reshape(1, len(pos), h, D // h), cos[pos], sin[pos]).reshape(len(pos), D), dt, "rope adjoint rows")


def test_c3_attention_full_size():
    """Q, K, V [8, 32, 2048, 128] bf16 causal: sampled queries (output, lse, dQ) against the oracle,
    V = 1 gives O = 1 (rows of P sum to one), and the adjoint identity with the tangent kernel for
    dK, dV at full size."""
    from enzyme_ad.jax import ops, jvp
    B, h, S, d = 8, 32, 2048, 128
    q, k, v, do = (_randn((B, h, S, d), "bf16", 10 + i) for i in range(4))
    with ops.Tape() as tape:
        o = ops.attention(q, k, v, h, layout="bhsd")
    dq, dk, dv = tape.backward([o], [do], [q, k, v])
    for (b, hh, qi) in [(0, 0, 0), (1, 5, 31), (2, 7, 64), (3, 31, 1000), (7, 16, 2047), (5, 9, 1283)]:
        sl = lambda t, n=qi + 1: host(t[b, hh, :n])[None, None]
        ro, _ = L.attention_fwd(sl(q)[:, :, -1:], sl(k), sl(v), causal=False)
        check(o[b, hh, qi], ro[0, 0, 0], "bf16", "o at query %d" % qi)
        rdq, _, _ = L.attention_bwd(sl(q)[:, :, -1:], sl(k), sl(v), sl(do)[:, :, -1:], causal=False)
        check(dq[b, hh, qi], rdq[0, 0, 0], "bf16", "dq at query %d" % qi)
    ones = torch.ones_like(v)
    o1 = ops.attention(q, k, ones, h, layout="bhsd")
    assert float((o1.float() - 1).abs().max()) <= 2 ** -7          # one bf16 ulp at 1: the rows of P sum to one
    tq, tk, tv = (_randn((B, h, S, d), "bf16", 20 + i) for i in range(3))
    _, to = jvp(lambda a, b_, c: ops.attention(a, b_, c, h, layout="bhsd"), (q, k, v), (tq, tk, tv))
    lhs, rhs = _dot(to, do), _dot(dq, tq) + _dot(dk, tk) + _dot(dv, tv)
    print("C3 attention <J v, w> = %.6g, <v, J^T w> = %.6g" % (lhs, rhs), flush=True)
    assert abs(lhs - rhs) <= 2e-2 * max(abs(lhs), abs(rhs))


def _layer_weights(D, H, dt, seed):
    shapes = [("rms_att_weight", (D,)), ("wq", (D, D)), ("wk", (D, D)), ("wv", (D, D)), ("wo", (D, D)),
              ("rms_ffn_weight", (D,)), ("w1", (H, D)), ("w2", (D, H)), ("w3", (H, D))]
    w = {}
    for i, (name, shp) in enumerate(shapes):
        if name.startswith("rms"):
            w[name] = (torch.rand(shp, device="cuda", generator=torch.Generator(device="cuda").manual_seed(seed + i)) + 0.5).to(TDTYPE[dt])
        else:
            w[name] = _randn(shp, dt, seed + i, 0.02)
    return w


def test_c5_llama7b_layer_full_size():
    """One 7B-shaped layer at batch 4 x seq 4096 in bf16: the first 48 tokens of a sequence only see
    each other, so the oracle redoes them (forward); the reverse pass is exactly linear in its
    cotangent (powers of two), the output before position t does not change when later tokens do,
    and forward and reverse mode satisfy <J v, w> = <v, J^T w> over all ten inputs."""
    from enzyme_ad.jax import enzyme_jax_ir, JaXPipeline, vjp, jvp, llama
    D, H, nh, B, S = 4096, 11008, 32, 4, 4096
    lw = _layer_weights(D, H, "bf16", 50)
    x, dy = _randn((B, S, D), "bf16", 60), _randn((B, S, D), "bf16", 61)

    @enzyme_jax_ir(pipeline_options=JaXPipeline(), inner_jit=False)
    def fn(x, lw):
        return llama.layer(x, lw, nh)

    y, f_vjp = vjp(fn, x, lw)
    gx, gw = f_vjp(dy)
    P = 48
    lwr = {k_: host(v_) for k_, v_ in lw.items()}
    for b in (0, 3):
        ry, _ = L.layer_fwd(host(x[b:b + 1, :P]), lwr, nh)
        check(y[b, :P], ry[0], "bf16", "layer output, first %d tokens of sequence %d" % (P, b))
    gx4, gw4 = f_vjp(dy * 4)
    assert torch.equal(gx4, gx * 4) and all(torch.equal(gw4[k_], gw[k_] * 4) for k_ in gw)
    x2 = x.clone()
    x2[:, 3000:] = _randn((B, S - 3000, D), "bf16", 62)
    y2 = fn(x2, lw)
    # Bit for bit up to the last 256-query block that lies wholly before the change; inside the block that
    # straddles it the running-maximum updates of a wavefront are shared by its 32 queries, so earlier
    # queries may round differently (never see other values).
    assert torch.equal(y2[:, :2816], y[:, :2816]) and not torch.equal(y2[:, 3000:], y[:, 3000:])
    assert rel_err(host(y2[:, 2816:3000]), host(y[:, 2816:3000])) <= 2e-2
    tx = _randn((B, S, D), "bf16", 63)
    tlw = {k_: _randn(v_.shape, "bf16", 70 + i, 0.02) for i, (k_, v_) in enumerate(lw.items())}
    _, ty = jvp(fn, (x, lw), (tx, tlw))
    lhs = _dot(ty, dy)
    rhs = _dot(gx, tx) + sum(_dot(gw[k_], tlw[k_]) for k_ in gw)
    print("C5 layer <J v, w> = %.6g, <v, J^T w> = %.6g" % (lhs, rhs), flush=True)
    assert abs(lhs - rhs) <= 3e-2 * max(abs(lhs), abs(rhs))


def test_c4_stories110m_full_size():
    """dim 768, hidden 2048, 12 layers, 12 heads of 64, vocab 32000, seq 1024, batch 8, bf16, tokens in
    and logits out: the first 40 positions of a sequence against the oracle (logits), exact
    linearity of the reverse pass in the logits cotangent, and the adjoint identity between forward
    and reverse mode over every weight."""
    from enzyme_ad.jax import enzyme_jax_ir, JaXPipeline, vjp, jvp, llama
    cfg = {"dim": 768, "hidden_dim": 2048, "n_layers": 12, "n_heads": 12, "n_kv_heads": 12, "vocab_size": 32000, "seq_len": 1024}
    B, S = 8, 1024
    w = L.make_weights(cfg, 4, std=0.02, norm_gain="uniform")
    wd, wr = {}, {}
    for k_, a in w.items():
        wd[k_], wr[k_] = dev(a, "bf16")
    rng = np.random.Generator(np.random.PCG64(1004))
    tok = rng.integers(0, cfg["vocab_size"], size=(B, S))
    tokd = torch.from_numpy(tok.astype(np.int32)).cuda()

    @enzyme_jax_ir(pipeline_options=JaXPipeline(), inner_jit=False)
    def fn(weights):
        return llama.forward(tokd, cfg, weights, logits=True)

    out, f_vjp = vjp(fn, wd)
    P = 40
    ref, _ = L.model_fwd(tok[2:3, :P], wr, cfg, logits=True)
    check(out[2, :P], ref[0], "bf16", "logits of the first %d positions" % P)
    dout = _randn(tuple(out.shape), "bf16", 90)
    (gw,) = f_vjp(dout)
    (gw2,) = f_vjp(dout * 2)
    # bit for bit, except the embedding table: its scatter-add uses fp32 atomics, whose order is not fixed
    assert all(torch.equal(gw2[k_], gw[k_] * 2) for k_ in gw if k_ != "token_embedding_table")
    assert rel_err(host(gw2["token_embedding_table"]), 2 * host(gw["token_embedding_table"])) <= 2 ** -7
    tw = {k_: _randn(v_.shape, "bf16", 100 + i, 0.02) for i, (k_, v_) in enumerate(wd.items())}
    _, tout = jvp(fn, (wd,), (tw,))
    lhs = _dot(tout, dout)
    rhs = sum(_dot(gw[k_], tw[k_]) for k_ in gw)
    print("C4 model <J v, w> = %.6g, <v, J^T w> = %.6g" % (lhs, rhs), flush=True)
    assert abs(lhs - rhs) <= 3e-2 * max(abs(lhs), abs(rhs))


@pytest.mark.parametrize("dt", ["bf16", "f32"])
def test_c4_logits_cross_entropy_full_size(dt):
    """Logits [8 x 1024, 32000] of the 110M configuration: sampled tokens against the oracle (loss, adjoint row,
    tangent), and over the whole tensor: every gradient row sums to zero and is linear in its loss cotangent, a
    constant shift of a row leaves its loss unchanged, and <J v, w> = <v, J^T w> between the tangent and adjoint
    kernels."""
    from enzyme_ad.jax import ops, jvp, vjp

    T, V = 8 * 1024, 32000
    z = _randn((8, 1024, V), dt, 41, 3.0)
    tz = _randn((8, 1024, V), dt, 42)
    g = torch.Generator(device="cuda").manual_seed(43)
    tgt = torch.randint(0, V, (8, 1024), device="cuda", generator=g, dtype=torch.int32)
    dl = torch.randn((8, 1024), device="cuda", generator=g)
    fn = lambda logits: ops.cross_entropy(logits, tgt)
    loss, tl = jvp(fn, (z,), (tz,))
    _, f_vjp = vjp(fn, z)
    (dz,) = f_vjp(dl)
    rows = [(0, 0), (3, 517), (7, 1023)]
    for b, s_ in rows:
        zr, tzr, t1 = host(z[b, s_]), host(tz[b, s_]), int(tgt[b, s_])
        ref_loss, _ = L.cross_entropy_fwd(zr[None], np.array([t1]))
        assert abs(float(loss[b, s_]) - ref_loss[0]) <= 1e-5 * max(1.0, abs(ref_loss[0]))
        check(dz[b, s_], L.cross_entropy_bwd(zr[None], np.array([t1]), np.array([float(dl[b, s_])]))[0], dt, "dlogits row")
        ref_tl = L.cross_entropy_jvp(zr[None], np.array([t1]), tzr[None])[0]
        assert abs(float(tl[b, s_]) - ref_tl) <= 1e-4 * max(1.0, abs(ref_tl))
    # rows of softmax - onehot sum to zero (up to the rounding of 32000 stored elements)
    row_sum = dz.float().sum(dim=-1)
    bound = (2e-2 if dt == "bf16" else 1e-4) * dl.abs().clamp_min(1e-3)
    assert bool((row_sum.abs() <= bound).all()), float((row_sum.abs() / bound).max())
    # exact linearity in the cotangent under a power-of-two scale
    (dz4,) = f_vjp(dl * 4.0)
    assert torch.equal(dz4, dz * 4.0)
    # a shifted row has the same loss (fp32 logits; in bf16 the shift would round the logits)
    if dt == "f32":
        shifted = ops.cross_entropy(z[:1] + 8.0, tgt[:1])
        assert float((shifted - loss[:1]).abs().max()) <= 2e-5
    lhs, rhs = _dot(tl, dl), _dot(tz, dz)
    assert abs(lhs - rhs) <= (2e-2 if dt == "bf16" else 1e-4) * max(abs(lhs), abs(rhs), 1.0), (lhs, rhs)
