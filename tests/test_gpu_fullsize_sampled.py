"""Element-wise oracle checks at the benchmark shapes.

The GEMM kernel for large problems is only selected at the benchmark sizes, where redoing the whole product on the
host is out of reach; a single output entry, however, is one K-term dot product.  These tests compare at least one
entry of every 256 x 256 output tile (and points on all four edges) with a float64 host dot product of the stored
operands, for every GEMM launch of the 7B-layer step and for the split-K / long-contraction launches of the 110M
model.  Attention is checked one whole (batch, head) at a time against the oracle (output, log-sum-exp, dQ, dK, dV
for every row), and the layer's reverse pass at full size is compared gradient by gradient with the oracle by giving
it a cotangent that is non-zero only on a causal prefix of each sequence, which the oracle can redo."""
import numpy as np
import pytest
import torch

from oracle import llama_ref as L
from gpu_util import host, check, check_rows, rel_err, TDTYPE

pytestmark = pytest.mark.gpu


def _randn(shape, dt, seed, scale=1.0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, device="cuda", generator=g) * scale).to(TDTYPE[dt])


def _sample_points(M, N, tile, rng):
    """One random entry per tile x tile output block, the four corners and 48 points on each edge."""
    ii, jj = [], []
    for i0 in range(0, M, tile):
        for j0 in range(0, N, tile):
            ii.append(i0 + int(rng.integers(0, min(tile, M - i0))))
            jj.append(j0 + int(rng.integers(0, min(tile, N - j0))))
    for i in (0, M - 1):
        for j in [0, N - 1] + list(rng.integers(0, N, 48)):
            ii.append(i)
            jj.append(int(j))
    for j in (0, N - 1):
        for i in rng.integers(0, M, 48):
            ii.append(int(i))
            jj.append(j)
    return np.array(ii), np.array(jj)


def _check_gemm_samples(a, b, c, trans_a, trans_b, residual, tile, seed, what):
    """c = op(a) . op(b) [+ residual] at sampled entries against float64 dot products of the stored operands."""
    M, N = c.shape
    rng = np.random.Generator(np.random.PCG64(seed))
    ii, jj = _sample_points(M, N, tile, rng)
    ti, tj = torch.from_numpy(ii).cuda(), torch.from_numpy(jj).cuda()
    ref = np.empty(len(ii))
    step = 1024                                       # bounds the gathered operands to a few hundred MB
    for s in range(0, len(ii), step):
        si, sj = ti[s:s + step], tj[s:s + step]
        ar = (a.index_select(1, si).t() if trans_a else a.index_select(0, si)).double()     # [n, K]
        br = (b.index_select(0, sj) if trans_b else b.index_select(1, sj).t()).double()     # [n, K]
        ref[s:s + step] = (ar * br).sum(dim=1).cpu().numpy()
    if residual is not None:
        ref = ref + host(residual[ti, tj])
    got = host(c[ti, tj])
    assert np.all(np.isfinite(got)), what
    scale = float(np.sqrt(np.mean(ref * ref)))
    # the contract: max-norm relative error; and entry by entry: one bf16 rounding of the fp32 sum
    e = float(np.max(np.abs(got - ref))) / float(np.max(np.abs(ref)))
    assert e <= 2e-2, "%s: max rel err %.3e" % (what, e)
    bad = np.abs(got - ref) > 2.0 ** -8 * np.abs(ref) + 1e-3 * scale
    assert not bad.any(), "%s: %d of %d sampled entries off by more than a bf16 rounding, first at (%d, %d): %g vs %g" % (
        what, int(bad.sum()), len(ref), ii[bad][0], jj[bad][0], got[bad][0], ref[bad][0])
    return e


C5 = dict(dim=4096, hidden_dim=11008, batch=4, seq=4096)


def _c5_launches():
    D, H, T = C5["dim"], C5["hidden_dim"], C5["batch"] * C5["seq"]
    out = []
    for name, (n_out, k_in) in zip(("wq", "wk", "wv", "wo", "w1", "w3", "w2"), [(D, D)] * 4 + [(H, D)] * 2 + [(D, H)]):
        out.append((name + ":Y", T, n_out, k_in))
        out.append((name + ":dX", T, k_in, n_out))
        out.append((name + ":dW", n_out, k_in, T))
    return out


@pytest.mark.parametrize("idx", range(21))
def test_c5_gemm_launch_sampled(idx):
    """Each of the 21 GEMM launches of one forward + reverse step of the 7B layer (batch 4 x seq 4096), in the
    layout the step uses: Y = X W^T (NT; wo and w2 with the residual operand), dX = dY (W^T)^T (NT on the transposed
    weight; the second and third of a fan-in with the residual operand), dW = dY^T X (TN, K = 16384 tokens)."""
    from enzyme_ad.jax import ops
    role, M, N, K = _c5_launches()[idx]
    name, kind = role.split(":")
    seed = 1000 + 10 * idx
    if kind == "dW":
        a = _randn((K, M), "bf16", seed)               # dY  [T, out], N(0, 1)
        b = _randn((K, N), "bf16", seed + 1)           # X   [T, in],  N(0, 1)
        c = ops.gemm(a, b, True, False)
        _check_gemm_samples(a, b, c, True, False, None, 256, seed + 2, role)
        return
    a = _randn((M, K), "bf16", seed)                   # activations N(0, 1)
    b = _randn((N, K), "bf16", seed + 1, 0.02)         # weight N(0, 0.02), [out, in] (or its transpose for dX)
    with_res = name in ("wo", "w2") if kind == "Y" else name in ("wk", "wv", "w3")
    r = _randn((M, N), "bf16", seed + 3) if with_res else None
    c = ops.gemm(a, b, False, True, r)
    _check_gemm_samples(a, b, c, False, True, r, 256, seed + 2, role + (" +R" if with_res else ""))


@pytest.mark.parametrize("shape", [
    # (trans_a, trans_b, M, N, K): the 110M model's weight gradients over 8192 tokens (split-K), its classifier
    # (vocabulary 32000) and the classifier's dX with its 32000-long contraction
    (True, False, 768, 768, 8192), (True, False, 2048, 768, 8192), (True, False, 768, 2048, 8192),
    (True, False, 32000, 768, 8192), (False, True, 8192, 32000, 768), (False, True, 8192, 768, 32000),
    (False, True, 8192, 2048, 768), (False, True, 8192, 768, 2048),
])
def test_c4_gemm_shapes_sampled(shape):
    from enzyme_ad.jax import ops
    ta, tb, M, N, K = shape
    seed = 3000 + (M * 7 + N * 3 + K) % 997
    a = _randn((K, M) if ta else (M, K), "bf16", seed)
    b = _randn((N, K) if tb else (K, N), "bf16", seed + 1, 1.0 if ta else 0.02)
    r = _randn((M, N), "bf16", seed + 3) if (M, N) == (8192, 768) else None
    c = ops.gemm(a, b, ta, tb, r)
    _check_gemm_samples(a, b, c, ta, tb, r, 128, seed + 2, "gemm %s" % (shape,))


@pytest.mark.parametrize("cfg", [
    # (B, h, S, d, layout, heads checked): C3 and the attention of C5
    (8, 32, 2048, 128, "bhsd", [(0, 0), (5, 17), (7, 31)]),
    (4, 32, 4096, 128, "bshd", [(0, 0), (3, 31)]),
    # the attention of C4 (stories110M: 12 heads of 64, seq 1024, batch 8) at its own grid
    (8, 12, 1024, 64, "bshd", [(0, 0), (7, 11)]),
])
def test_attention_whole_heads_full_size(cfg):
    """Every row of o, lse, dQ, dK and dV of a few (batch, head) pairs against the oracle, with the kernels running
    the full-size problem (their block-to-work mapping depends on the grid)."""
    from enzyme_ad.jax import ops
    B, h, S, d, layout, picks = cfg
    shape = (B, h, S, d) if layout == "bhsd" else (B, S, h * d)
    q, k, v, do = (_randn(shape, "bf16", 200 + i) for i in range(4))
    with ops.Tape() as tape:
        o, lse = ops.attention(q, k, v, h, layout=layout, return_lse=True)
    dq, dk, dv = tape.backward([o], [do], [q, k, v])
    pick = (lambda t, b, hh: t[b, hh]) if layout == "bhsd" else (lambda t, b, hh: t.reshape(B, S, h, d)[b, :, hh])
    for (b, hh) in picks:
        qs, ks, vs, dos = (host(pick(t, b, hh))[None, None] for t in (q, k, v, do))
        ro, rlse = L.attention_fwd(qs, ks, vs)
        assert float(np.max(np.abs(host(lse[b, hh]) - rlse[0, 0]))) <= 1e-3, "lse of (batch %d, head %d)" % (b, hh)
        rdq, rdk, rdv = L.attention_bwd(qs, ks, vs, dos)
        for name, got, ref in (("o", o, ro), ("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
            g = host(pick(got, b, hh))
            check(g, ref[0, 0], "bf16", "%s of (batch %d, head %d)" % (name, b, hh))
            # Beyond the contract's per-tensor bound: every row against its own maximum.  Outputs hold 2e-2 row by
            # row.  Gradient rows are held to 4x that: where a query sees few keys, dS = P (dP - delta) cancels to a
            # small difference while delta = rowsum(dO . O) carries the rounding of the stored bf16 O (|error| about
            # 2^-9 |dO| |O| sqrt(d)), so a row's own error is not bounded by one bf16 rounding of its largest entry
            # (measured worst rows: dq 2.3e-2 at query 1 of a head, dk / dv below 1e-2); a misplaced or missing row
            # would be off by ~100 %.
            worst = check_rows(g, ref[0, 0], "bf16", "%s rows of (batch %d, head %d)" % (name, b, hh),
                               factor=1.0 if name == "o" else 4.0)
            print("attention %s (batch %d, head %d) of %s: worst row-relative error %.3e" % (name, b, hh, cfg[:4], worst), flush=True)


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


def test_c5_layer_every_gradient_from_prefix_cotangent():
    """The 7B-shaped layer at batch 4 x seq 4096 with a cotangent that is non-zero on the first 40 tokens of every
    sequence only.  By causality the reverse pass then depends on those tokens alone, so the oracle can redo it: dx on
    the prefixes (and exact zeros after them) and all nine weight gradients, while the kernels run their full-size
    launches (the dW GEMMs contract over all 16384 tokens)."""
    from enzyme_ad.jax import enzyme_jax_ir, JaXPipeline, vjp, llama
    D, H, nh, B, S, P = 4096, 11008, 32, 4, 4096, 40
    lw = _layer_weights(D, H, "bf16", 50)
    x, dy = _randn((B, S, D), "bf16", 60), _randn((B, S, D), "bf16", 61)
    dy[:, P:] = 0

    @enzyme_jax_ir(pipeline_options=JaXPipeline(), inner_jit=False)
    def fn(x, lw):
        return llama.layer(x, lw, nh)

    y, f_vjp = vjp(fn, x, lw)
    gx, gw = f_vjp(dy)
    assert float(gx[:, P:].float().abs().max()) == 0.0
    lwr = {k_: host(v_) for k_, v_ in lw.items()}
    ry, cache = L.layer_fwd(host(x[:, :P]), lwr, nh)
    rgx, rgw = L.layer_bwd(host(dy[:, :P]), lwr, cache, nh)
    check(y[:, :P], ry, "bf16", "layer output on the prefixes")
    check(gx[:, :P], rgx, "bf16", "dx on the prefixes")
    check_rows(host(gx[:, :P]).reshape(-1, D), rgx.reshape(-1, D), "bf16", "dx rows on the prefixes")
    for k_ in rgw:
        check(gw[k_], rgw[k_], "bf16", "d" + k_)
        if rgw[k_].ndim == 2:
            check_rows(host(gw[k_]), rgw[k_], "bf16", "rows of d" + k_)


def test_c5_width_short_sequence_every_gradient():
    """Full width (dim 4096, hidden 11008, 32 heads), one sequence of 256 tokens: output, dx and all nine weight
    gradients over every element against the oracle."""
    from enzyme_ad.jax import enzyme_jax_ir, JaXPipeline, vjp, llama
    D, H, nh, B, S = 4096, 11008, 32, 1, 256
    lw = _layer_weights(D, H, "bf16", 150)
    x, dy = _randn((B, S, D), "bf16", 160), _randn((B, S, D), "bf16", 161)

    @enzyme_jax_ir(pipeline_options=JaXPipeline(), inner_jit=False)
    def fn(x, lw):
        return llama.layer(x, lw, nh)

    y, f_vjp = vjp(fn, x, lw)
    gx, gw = f_vjp(dy)
    lwr = {k_: host(v_) for k_, v_ in lw.items()}
    ry, cache = L.layer_fwd(host(x), lwr, nh)
    rgx, rgw = L.layer_bwd(host(dy), lwr, cache, nh)
    check(y, ry, "bf16", "layer output")
    check(gx, rgx, "bf16", "dx")
    check_rows(host(gx).reshape(-1, D), rgx.reshape(-1, D), "bf16", "dx rows")
    for k_ in rgw:
        check(gw[k_], rgw[k_], "bf16", "d" + k_)
        if rgw[k_].ndim == 2:
            check_rows(host(gw[k_]), rgw[k_], "bf16", "rows of d" + k_)


def test_c4_model_every_gradient_from_prefix_cotangent():
    """The 110M configuration at its own size (12 layers, dim 768, hidden 2048, 12 heads of 64, vocabulary 32000,
    batch 8 x seq 1024, bf16, tokens in, logits out) with a logits cotangent that is non-zero on the first 32
    positions of every sequence only.  By causality the reverse pass depends on those positions alone, so the oracle
    redoes it whole: the logits on the prefixes and every weight gradient (per layer, `wcls`, the final gain, the
    embedding table) at the contract's bound, while the kernels run their full-size launches (the deferred weight
    gradients contract over all 8192 tokens, the head_dim-64 attention kernels run the 8 x 12 x 1024 grid)."""
    from enzyme_ad.jax import enzyme_jax_ir, JaXPipeline, vjp, llama
    from gpu_util import dev
    cfg = {"dim": 768, "hidden_dim": 2048, "n_layers": 12, "n_heads": 12, "n_kv_heads": 12, "vocab_size": 32000, "seq_len": 1024}
    B, S, P = 8, 1024, 32
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
    dout = _randn(tuple(out.shape), "bf16", 91)
    dout[:, P:] = 0
    (gw,) = f_vjp(dout)
    ref, fcache = L.model_fwd(tok[:, :P], wr, cfg, logits=True)
    check(out[:, :P], ref, "bf16", "logits on the prefixes")
    _, rgw = L.model_bwd(host(dout[:, :P]), wr, cfg, fcache)
    assert set(rgw) == set(gw)
    for k_ in sorted(rgw):
        e = check(gw[k_], rgw[k_], "bf16", "d" + k_)
        print("C4 prefix cotangent: d%s max relative error %.3e" % (k_, e), flush=True)
        if rgw[k_].ndim == 3:
            # per layer, for the record (beyond the contract, which bounds each gradient tensor as a whole): twelve
            # layers of bf16 activations separate the last layer's cotangent from the first layer's weights, and a
            # layer's own maximum can be far below the stack's (measured worst: dwk[6] 2.6e-2 of that layer's maximum)
            per = [rel_err(host(gw[k_][l]), rgw[k_][l]) for l in range(cfg["n_layers"])]
            print("    per layer: worst %.3e (layer %d)" % (max(per), int(np.argmax(per))), flush=True)
            assert max(per) <= 4e-2
