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
