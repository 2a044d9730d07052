"""Tape rules whose cotangent fan-in or tangent propagation needs its own case: transpose in both modes, a stacked
weight that is used whole and sliced, concatenate along an inner index with an operand that has a second use."""
import numpy as np
import pytest
import torch

from gpu_util import host

pytestmark = pytest.mark.gpu


def _randn(shape, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.randn(shape, device="cuda", generator=g)


def test_transpose_forward_and_reverse_mode():
    """Transpose rule (HLODerivatives.td:1334-1339): the tangent is transposed, the cotangent is transposed back;
    <J v, w> = <v, J^T w> bit for bit (pure data movement)."""
    from enzyme_ad.jax import ops, jvp, vjp
    a, ta, w = _randn((48, 80), 1), _randn((48, 80), 2), _randn((80, 48), 3)
    out, tout = jvp(ops.transpose, (a,), (ta,))
    assert torch.equal(out, a.t().contiguous()) and torch.equal(tout, ta.t().contiguous())
    _, f_vjp = vjp(ops.transpose, a)
    (ga,) = f_vjp(w)
    assert torch.equal(ga, w.t().contiguous())


def test_stacked_weight_used_whole_and_sliced():
    """`select` places its cotangent in a zero tensor (Slice rule, StableHLOAutoDiffOpInterfaceImpl.cpp:1586-1620);
    when the stacked weight is also consumed whole, the fan-in must be summed without writing into a buffer another
    rule (or the caller) still holds."""
    from enzyme_ad.jax import ops, vjp
    w = _randn((3, 16, 32), 4)
    x = _randn((8, 32), 5)

    def fn(w):
        y0 = ops.matmul_nt(x, ops.select(w, 0))
        y2 = ops.matmul_nt(x, ops.select(w, 2))
        return ops.add(y0, y2), ops.add(w, w)

    (s, ww), f_vjp = vjp(fn, w)
    cs, cw = _randn((8, 16), 6), _randn((3, 16, 32), 7)
    cw_before = cw.clone()
    (gw,) = f_vjp((cs, cw))
    ref = 2 * host(cw)
    ref[0] += host(cs).T @ host(x)
    ref[2] += host(cs).T @ host(x)
    assert np.max(np.abs(host(gw) - ref)) <= 1e-4 * np.max(np.abs(ref))
    assert torch.equal(cw, cw_before), "the caller's cotangent was written in place"


def test_concatenate_inner_dim_with_operand_fan_in():
    """Concatenate rule (StableHLOAutoDiffOpInterfaceImpl.cpp:2015-2059): slices of the cotangent along dim 1 are not
    contiguous; an operand with a second use has them added to another cotangent."""
    from enzyme_ad.jax import ops, hlo_ops, vjp
    a, b = _randn((6, 10), 8), _randn((6, 22), 9)

    def fn(a, b):
        return hlo_ops.concatenate([a, b], 1), ops.add(a, a)

    (y, a2), f_vjp = vjp(fn, a, b)
    cy, ca = _randn((6, 32), 10), _randn((6, 10), 11)
    ga, gb = f_vjp((cy, ca))
    assert ga.is_contiguous() and gb.is_contiguous()
    assert np.max(np.abs(host(ga) - (host(cy)[:, :10] + 2 * host(ca)))) <= 1e-5
    assert torch.equal(gb, cy[:, 10:].contiguous())


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_stacked_weight_gradients_written_in_place_and_deferred(dt):
    """A stacked weight that is only ever sliced, one select per layer: the weight-gradient products are written
    straight into the slices of one buffer and run grouped at the end of the backward pass.  Layers that are never
    selected keep a zero gradient; the RMSNorm gain of a stacked gain tensor takes the same route."""
    from enzyme_ad.jax import ops, vjp
    L, T, D, H = 4, 136, 64, 96
    w = (_randn((L, H, D), 20) * 0.1).to(dt)
    gam = (_randn((L, D), 21) * 0.1 + 1).to(dt)
    x = _randn((T, D), 22).to(dt)

    def fn(w, gam):
        ys = []
        for l in (0, 1, 3):                                  # layer 2 is never used
            ys.append(ops.matmul_nt(ops.rmsnorm(x, ops.select(gam, l)), ops.select(w, l)))
        return ops.add(ops.add(ys[0], ys[1]), ys[2])

    out, f_vjp = vjp(fn, w, gam)
    c = _randn((T, H), 23).to(dt)
    gw, gg = f_vjp(c)
    w64, g64, x64, c64 = (t.double().requires_grad_(t is not x and t is not c) for t in (w, gam, x, c))
    ref = 0
    for l in (0, 1, 3):
        xn = x64 * torch.rsqrt((x64 * x64).mean(-1, keepdim=True) + 1e-5) * g64[l]
        ref = ref + xn @ w64[l].T
    ref.backward(c64)
    tol = 1e-4 if dt == torch.float32 else 3e-2
    assert float((gw.double() - w64.grad).abs().max()) <= tol * float(w64.grad.abs().max())
    assert float((gg.double() - g64.grad).abs().max()) <= tol * float(g64.grad.abs().max())
    assert not gw[2].any() and not gg[2].any()
    # twice in a row: the buffers of the first call are not reused
    gw2, _ = f_vjp(c)
    assert torch.equal(gw, gw2) and gw2.data_ptr() != gw.data_ptr()


def test_stacked_weight_slice_selected_twice_or_used_twice():
    """The cases the in-place route must stay away from: one slice selected by two select calls, and one selected
    slice feeding two products (its cotangent is a sum that the select rule stores)."""
    from enzyme_ad.jax import ops, vjp
    w = _randn((2, 24, 40), 30)
    x1, x2 = _randn((16, 40), 31), _randn((16, 40), 32)

    def twice_selected(w):
        return ops.add(ops.matmul_nt(x1, ops.select(w, 1)), ops.matmul_nt(x2, ops.select(w, 1)))

    def twice_used(w):
        s = ops.select(w, 1)
        return ops.add(ops.matmul_nt(x1, s), ops.matmul_nt(x2, s))

    c = _randn((16, 24), 33)
    ref = np.zeros((2, 24, 40))
    ref[1] = host(c).T @ host(x1) + host(c).T @ host(x2)
    for fn in (twice_selected, twice_used):
        _, f_vjp = vjp(fn, w)
        (gw,) = f_vjp(c)
        assert np.max(np.abs(host(gw) - ref)) <= 1e-4 * np.max(np.abs(ref)), fn.__name__


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_pair_shares_a_launch_and_matches_two_ropes(dtype):
    """rope_pair on operands that lie side by side (as the grouped projection returns them) and on operands that do
    not: outputs and both cotangents equal those of two separate rope calls, bit for bit."""
    from enzyme_ad.jax import ops
    B, S, H, d = 2, 37, 3, 16
    buf = _randn((2, B, S, H * d), 11).to(dtype)
    cot = _randn((2, B, S, H * d), 12).to(dtype)
    for side_by_side in (True, False):
        q, k = (buf[0], buf[1]) if side_by_side else (buf[0].clone(), buf[1].clone())
        cq, ck = (cot[0], cot[1]) if side_by_side else (cot[0].clone(), cot[1].clone())
        with ops.Tape() as tape:
            yq, yk = ops.rope_pair(q, k, H)
        gq, gk = tape.backward([yq, yk], [cq, ck], [q, k])
        with ops.Tape() as tape2:
            rq, rk = ops.rope(q, H), ops.rope(k, H)
        hq, hk = tape2.backward([rq, rk], [cq, ck], [q, k])
        for a, b in ((yq, rq), (yk, rk), (gq, hq), (gk, hk)):
            assert torch.equal(a, b)
    # a cotangent on one of the two results only
    q, k = buf[0], buf[1]
    with ops.Tape() as tape:
        yq, yk = ops.rope_pair(q, k, H)
    gq, gk = tape.backward([yk], [cot[1]], [q, k])
    with ops.Tape() as tape2:
        rk = ops.rope(k, H)
    (hk,) = tape2.backward([rk], [cot[1]], [k])
    assert gq is None or not bool(gq.any())
    assert torch.equal(gk, hk)


def test_stack_produced_on_the_tape_takes_the_general_slice_rule():
    """A stacked weight that an operator on the tape produced (bf16 copy of fp32 master weights) is sliced and
    multiplied: its producer's rule runs before any deferred product could have filled an in-place buffer, so such a
    stack must take the general Slice rule.  Also `w[-1]` and `w[L-1]` are one slice (its two cotangents add)."""
    from enzyme_ad.jax import ops, hlo_ops as H, vjp
    L_, T, D, Hd = 3, 72, 64, 96
    w32 = _randn((L_, Hd, D), 40) * 0.1
    x = _randn((T, D), 41).to(torch.bfloat16)

    def fn(w32):
        w = H.convert(w32, torch.bfloat16)
        y0 = ops.matmul_nt(x, ops.select(w, 0))
        y2 = ops.matmul_nt(x, ops.select(w, 2))
        y2b = ops.matmul_nt(x, ops.select(w, -1))
        return y0, y2, y2b

    ys, f_vjp = vjp(fn, w32)
    cs = [_randn((T, Hd), 42 + i).to(torch.bfloat16) for i in range(3)]
    (g,) = f_vjp(tuple(cs))
    assert g.dtype == torch.float32
    xr = host(x)
    ref = np.zeros((L_, Hd, D))
    ref[0] = host(cs[0]).T @ xr
    ref[2] = host(cs[1]).T @ xr + host(cs[2]).T @ xr
    assert float(g[1].abs().max()) == 0.0
    assert np.max(np.abs(host(g) - ref)) <= 2e-2 * np.max(np.abs(ref))


def _small_model(seed):
    cfg = {"dim": 64, "hidden_dim": 96, "n_layers": 2, "n_heads": 2, "n_kv_heads": 2, "vocab_size": 50, "seq_len": 48}
    g = torch.Generator(device="cuda").manual_seed(seed)
    r = lambda *s: torch.randn(s, device="cuda", generator=g) * 0.1
    Lc, D, Hd = cfg["n_layers"], cfg["dim"], cfg["hidden_dim"]
    w = {"rms_att_weight": r(Lc, D) + 1, "rms_ffn_weight": r(Lc, D) + 1, "rms_final_weight": r(D) + 1,
         "wq": r(Lc, D, D), "wk": r(Lc, D, D), "wv": r(Lc, D, D), "wo": r(Lc, D, D),
         "w1": r(Lc, Hd, D), "w3": r(Lc, Hd, D), "w2": r(Lc, D, Hd)}
    x = torch.randn((2, 48, D), device="cuda", generator=g)
    dy = torch.randn((2, 48, D), device="cuda", generator=g)
    return cfg, w, x, dy


def test_reverse_passes_on_two_threads_match_the_serial_run():
    """The active tape and everything a reverse pass shares between its rules (in-place gradient buffers of stacked
    weights, deferred weight-gradient products, weight transposes) are per thread and per pass: two threads that each
    differentiate their own model on their own stream, many times over, get the bits of the serial run (handlers run
    on executor threads in the reference, enzyme_call.cc:173,263)."""
    import threading
    from enzyme_ad.jax import vjp, llama

    def run(seed):
        cfg, w, x, dy = _small_model(seed)
        y, f_vjp = vjp(lambda x, w: llama.forward(x, cfg, w), x, w)
        gx, gw = f_vjp(dy)
        return [y, gx] + [gw[k] for k in sorted(gw)]

    serial = {seed: [t.clone() for t in run(seed)] for seed in (1, 2)}
    torch.cuda.synchronize()
    results, errors = {}, []

    def worker(seed):
        try:
            stream = torch.cuda.Stream()                       # default priority
            with torch.cuda.stream(stream):
                for _ in range(6):
                    out = run(seed)
                stream.synchronize()
            results[seed] = out
        except Exception as e:                                 # surfaced in the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(seed,)) for seed in (1, 2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for seed in (1, 2):
        for a, b in zip(results[seed], serial[seed]):
            assert torch.equal(a, b)


def test_vjp_inside_a_rule_of_another_reverse_pass():
    """A reverse pass started while another one is running (a rule that itself differentiates a function) has its own
    buffers: the outer pass's in-place stacked gradients and deferred products are untouched by it."""
    from enzyme_ad.jax import ops, vjp, llama
    cfg, w, x, dy = _small_model(3)
    cfg2, w2, x2, dy2 = _small_model(4)
    y, f_vjp = vjp(lambda x, w: llama.forward(x, cfg, w), x, w)
    gx_ref, gw_ref = f_vjp(dy)
    y2, f_vjp2 = vjp(lambda x, w: llama.forward(x, cfg2, w), x2, w2)
    gx2_ref, gw2_ref = f_vjp2(dy2)
    inner = {}

    def fn(x, w):
        h = llama.forward(x, cfg, w)
        out = ops.add(h, h)

        def rule(c, acc):
            # runs in the middle of the outer pass, before the layers' rules
            _, g = vjp(lambda x, w: llama.forward(x, cfg2, w), x2, w2)
            inner["g"] = g(dy2)
            return (ops._accumulate(acc[0], c), ops._accumulate(acc[1], c))

        ops.Tape._active.nodes[-1] = (ops.Tape._active.nodes[-1][0], out, rule)
        return out

    out, f = vjp(fn, x, w)
    gx, gw = f(dy)
    gx_in, gw_in = inner["g"]
    assert torch.equal(gx_in, gx2_ref) and all(torch.equal(gw_in[k], gw2_ref[k]) for k in gw2_ref)
    assert torch.equal(gx, gx_ref * 2) and all(torch.equal(gw[k], gw_ref[k] * 2) for k in gw_ref)
