"""GPU parity of the StableHLO text front end: the generic tensor kernels against numpy, the
reference's `hlo_call` fixture (test/testffi.py:6-49) against its closed-form answers, and the
differentiation rules of the generic operators against the known-answer vectors of the
reference's lit tests (tests/golden/diffrules.json), each driven through StableHLO text."""
import json
import os

import numpy as np
import pytest
import torch

from gpu_util import TDTYPE, dev, host

pytestmark = pytest.mark.gpu

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "diffrules.json")))


def f32(a):
    return torch.tensor(np.asarray(a, dtype=np.float32), device="cuda")


def ulp_close(got, want, dt):
    got, want = host(got), np.asarray(want, dtype=np.float64)
    tol = 2e-6 if dt == "f32" else 8e-3                    # one bf16 ulp is 2^-8 relative
    np.testing.assert_allclose(got, want, rtol=tol, atol=tol * 1e-3)


# ---------------------------------------------------------------------------
# kernels
# ---------------------------------------------------------------------------

NP_BINARY = {"add": np.add, "subtract": np.subtract, "multiply": np.multiply, "divide": np.divide,
             "maximum": np.maximum, "minimum": np.minimum, "ge": lambda a, b: (a >= b).astype(np.float64),
             "eq": lambda a, b: (a == b).astype(np.float64), "nmul": lambda a, b: -(a * b), "power": np.power,
             "d_sqrt": lambda a, b: np.where(b == 0, 0.0, a / (2 * np.where(b == 0, 1.0, b))),
             "d_rsqrt": lambda a, b: -0.5 * a * b ** 3, "d_logistic": lambda a, b: a * b * (1 - b),
             "d_tanh": lambda a, b: a * (1 - b * b), "d_sin": lambda a, b: a * np.cos(b),
             "d_cos": lambda a, b: -a * np.sin(b), "d_pow_a": lambda a, b: b * np.power(a, b - 1),
             "d_pow_b": lambda a, b: np.power(a, b) * np.log(a), "d_abs": lambda a, b: np.where(b >= 0, a, -a),
             "d_log1p": lambda a, b: a / (b + 1), "d_expm1": lambda a, b: a * np.exp(b),
             "d_cbrt": lambda a, b: a / (3 * b * b), "atan2": np.arctan2}
NP_UNARY = {"negate": np.negative, "exponential": np.exp, "log": np.log, "sqrt": np.sqrt,
            "rsqrt": lambda x: 1 / np.sqrt(x), "logistic": lambda x: 1 / (1 + np.exp(-x)), "tanh": np.tanh,
            "sine": np.sin, "cosine": np.cos, "abs": np.abs, "copy": lambda x: x, "log_plus_one": np.log1p,
            "exponential_minus_one": np.expm1, "cbrt": np.cbrt}
POSITIVE = {"log", "sqrt", "rsqrt", "power", "d_pow_a", "d_pow_b", "log_plus_one", "d_log1p", "d_cbrt"}


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("n", [1, 7, 1000, 4099])
def test_elementwise_maps_match_numpy(dt, n):
    from enzyme_ad.jax import hlo_ops as H

    rng = np.random.default_rng(n)
    for name, fn in NP_BINARY.items():
        a = rng.uniform(0.5, 2.0, n) if name in POSITIVE else rng.normal(size=n)
        b = rng.uniform(0.5, 2.0, n) if name in POSITIVE else rng.normal(size=n)
        if name in ("ge", "eq", "maximum") and n > 2:
            b[::3] = a[::3]                                             # ties
        ta, ra = dev(a, dt)
        tb, rb = dev(b, dt)
        ulp_close(H._bin(name, ta, tb), fn(ra, rb), dt)
        s, rs = torch.tensor(1.25, dtype=TDTYPE[dt], device="cuda"), 1.25    # rank-0 operand, either side
        ulp_close(H._bin(name, ta, s), fn(ra, rs), dt)
        ulp_close(H._bin(name, s, tb), fn(rs, rb), dt)
    for name, fn in NP_UNARY.items():
        x = rng.uniform(0.5, 2.0, n) if name in POSITIVE else rng.normal(size=n)
        tx, rx = dev(x, dt)
        ulp_close(H._un(name, tx), fn(rx), dt)
    tx, rx = dev(rng.normal(size=n), "f32")
    back = H._convert(H._convert(tx, torch.bfloat16), torch.float32)
    assert torch.equal(back, tx.to(torch.bfloat16).float())


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("n", [1, 9, 4099, 70001])
def test_compare_and_select_match_numpy(dt, n):
    from enzyme_ad.jax import hlo_ops as H

    rng = np.random.default_rng(n + 1)
    a, b = rng.normal(size=n), rng.normal(size=n)
    b[::3] = a[::3]
    (ta, ra), (tb, rb) = dev(a, dt), dev(b, dt)
    s = torch.tensor(0.25, dtype=TDTYPE[dt], device="cuda")
    fns = {"EQ": np.equal, "NE": np.not_equal, "GE": np.greater_equal, "GT": np.greater, "LE": np.less_equal, "LT": np.less}
    for d, fn in fns.items():
        m = H._compare(d, ta, tb)
        assert m.dtype == torch.bool and np.array_equal(m.cpu().numpy(), fn(ra, rb)), d
        assert np.array_equal(H._compare(d, ta, s).cpu().numpy(), fn(ra, 0.25)), d
        assert np.array_equal(H._compare(d, s, tb).cpu().numpy(), fn(0.25, rb)), d
    m = H._compare("GT", ta, tb)
    assert np.array_equal(host(H._select(m, ta, tb)), np.where(ra > rb, ra, rb))
    assert np.array_equal(host(H._select(m, s, tb)), np.where(ra > rb, 0.25, rb))
    assert np.array_equal(host(H._select(m, ta, s)), np.where(ra > rb, ra, 0.25))
    one = torch.tensor(True, device="cuda")
    assert np.array_equal(host(H._select(one, ta, tb)), ra)
    inf = torch.full_like(ta, float("inf"))
    assert np.array_equal(host(H._select(m, ta, inf)), np.where(ra > rb, ra, np.inf))         # no 0 * inf


def test_elementwise_maps_on_unaligned_views():
    from enzyme_ad.jax import hlo_ops as H

    base, ref = dev(np.arange(64, dtype=np.float32), "f32")
    a, b = base[1:34], base[3:36]                                        # 4-byte aligned only
    assert np.array_equal(host(H._bin("add", a, b)), ref[1:34] + ref[3:36])
    assert np.array_equal(host(H._un("negate", a)), -ref[1:34])


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_strided_copy_forms_match_numpy(dt):
    from enzyme_ad.jax import hlo_ops as H

    rng = np.random.default_rng(3)
    x, rx = dev(rng.normal(size=(6, 8, 16)), dt)
    for perm in ([0, 1, 2], [2, 1, 0], [1, 0, 2], [0, 2, 1], [2, 0, 1]):
        assert np.array_equal(host(H._permute(x, perm)), rx.transpose(perm))
    v, rv = dev(rng.normal(size=(8,)), dt)
    assert np.array_equal(host(H._broadcast(v, (6, 8, 16), [1])), np.broadcast_to(rv[None, :, None], (6, 8, 16)))
    r, rr = dev(rng.normal(size=(6, 1, 16)), dt)
    assert np.array_equal(host(H._broadcast(r, (6, 8, 16), [0, 1, 2])), np.broadcast_to(rr, (6, 8, 16)))
    s = torch.tensor(2.5, dtype=TDTYPE[dt], device="cuda")
    assert np.array_equal(host(H._broadcast(s, (5, 3), [])), np.full((5, 3), 2.5))
    assert np.array_equal(host(H._slice(x, [1, 0, 3], [6, 8, 16], [2, 3, 1])), rx[1:6:2, 0:8:3, 3:16])
    assert np.array_equal(host(H._slice(x, [0, 0, 0], [6, 8, 8], [1, 1, 1])), rx[:, :, :8])
    y, ry = dev(rng.normal(size=(6, 3, 16)), dt)
    assert np.array_equal(host(H._concat([x, y], 1)), np.concatenate([rx, ry], 1))
    z, rz = dev(rng.normal(size=(6, 8, 5)), dt)
    assert np.array_equal(host(H._concat([x, z, x], 2)), np.concatenate([rx, rz, rx], 2))
    box = H._scatter_box(H._slice(x, [1, 0, 3], [6, 8, 16], [2, 3, 1]), [6, 8, 16], [1, 0, 3], [2, 3, 1])
    want = np.zeros_like(rx)
    want[1:6:2, 0:8:3, 3:16] = rx[1:6:2, 0:8:3, 3:16]
    assert np.array_equal(host(box), want)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("shape,dims", [((37, 5000), [1]), ((37, 5000), [0]), ((4, 33, 7), [1]), ((4, 33, 7), [0, 2]),
                                        ((2, 3, 4), [0, 1, 2]), ((300, 64), [1]), ((1, 100003), [1]),
                                        # column sums split into bands of rows: a partial strip of columns, a strip of one
                                        # wavefront, several outer slices, more strips than one
                                        ((4096, 1000), [0]), ((3000, 96), [0]), ((2, 700, 520), [1]), ((1500, 5000), [0])])
def test_reduce_matches_numpy(dt, shape, dims):
    from enzyme_ad.jax import hlo_ops as H

    x, rx = dev(np.random.default_rng(5).normal(size=shape), dt)
    tol = 1e-5 if dt == "f32" else 8e-3
    got = host(H._reduce("add", x, dims))
    want = rx.sum(axis=tuple(dims))
    assert np.max(np.abs(got - want)) <= tol * max(1.0, np.max(np.abs(want)))
    assert np.array_equal(host(H._reduce("maximum", x, dims)), rx.max(axis=tuple(dims)))


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_dot_general_forms_match_numpy(dt):
    from enzyme_ad.jax import hlo_ops as H

    rng = np.random.default_rng(11)
    tol = 1e-5 if dt == "f32" else 1.5e-2
    cases = [
        ((2, 3), (4, 2), [], [], [0], [1], "ki,jk->ij"),
        ((5, 7, 9), (5, 9, 4), [0], [0], [2], [1], "bmk,bkn->bmn"),
        ((288, 288), (288,), [], [], [1], [0], "ok,k->o"),
        ((144, 2, 2), (144, 2), [0], [0], [2], [1], "ijk,ik->ij"),
        ((9, 48), (9,), [], [], [0], [0], "ij,i->j"),
        ((3, 4, 5, 6), (6, 3, 5, 2), [0], [1], [2, 3], [2, 0], "bmxy,ybxn->bmn"),
    ]
    for sa, sb, ba, bb, ca, cb, spec in cases:
        a, ra = dev(rng.normal(size=sa), dt)
        b, rb = dev(rng.normal(size=sb), dt)
        want = np.einsum(spec, ra, rb)
        got = host(H._dot_general(a, b, ba, bb, ca, cb))
        assert got.shape == want.shape, spec
        assert np.max(np.abs(got - want)) <= tol * np.max(np.abs(want)), spec


# ---------------------------------------------------------------------------
# hlo_call
# ---------------------------------------------------------------------------

HLO_FFI = """
module {
func.func @main(%arg0: tensor<2x2xf32>, %arg1: tensor<f32>) -> (tensor<f32>, tensor<2x2xf32>) {
%cst = stablehlo.constant dense<0.000000e+00> : tensor<f32>
%0 = stablehlo.transpose %arg0, dims = [1, 0] : (tensor<2x2xf32>) -> tensor<2x2xf32>
%1 = stablehlo.reduce(%0 init: %cst) applies stablehlo.add across dimensions = [0, 1] : (tensor<2x2xf32>, tensor<f32>) -> tensor<f32>
%2 = stablehlo.broadcast_in_dim %arg1, dims = [] : (tensor<f32>) -> tensor<2x2xf32>
%3 = stablehlo.multiply %0, %2 : tensor<2x2xf32>
%4 = stablehlo.transpose %3, dims = [1, 0] : (tensor<2x2xf32>) -> tensor<2x2xf32>
return %1, %4 : tensor<f32>, tensor<2x2xf32>
}
}
"""


def test_reference_hlo_call_fixture():
    """test/testffi.py: a = sum(mat), b = mat * scalar on ones(2, 2) and 2.7, with the
    fixture's tangents (5.0, 3.1) and cotangents (3.4, 7.0)."""
    from enzyme_ad.jax import hlo_call, jvp, vjp

    def do_something(mat, scalar):
        a, b = hlo_call(mat, scalar, source=HLO_FFI)
        return a, b

    mat, scalar = f32(np.ones((2, 2))), f32(2.7)
    a, b = do_something(mat, scalar)
    assert a.shape == () and float(a) == 4.0
    np.testing.assert_allclose(host(b), np.full((2, 2), 2.7), rtol=1e-7)
    (a, b), (ta, tb) = jvp(do_something, (mat, scalar), (f32(np.full((2, 2), 5.0)), f32(3.1)))
    assert float(ta) == 20.0
    np.testing.assert_allclose(host(tb), np.full((2, 2), 5.0 * 2.7 + 3.1), rtol=1e-6)
    _, f_vjp = vjp(do_something, mat, scalar)
    gm, gs = f_vjp((f32(3.4), f32(np.full((2, 2), 7.0))))
    np.testing.assert_allclose(host(gm), np.full((2, 2), 3.4 + 7.0 * 2.7), rtol=1e-6)
    np.testing.assert_allclose(float(gs), 28.0, rtol=1e-6)


def test_hlo_call_rejects_wrong_arguments():
    from enzyme_ad.jax import hlo_call

    with pytest.raises(ValueError):
        hlo_call(f32(np.ones((2, 3))), f32(2.7), source=HLO_FFI)
    with pytest.raises(AssertionError):
        hlo_call(f32(np.ones((2, 2))), source=HLO_FFI)
    with pytest.raises(AssertionError):
        hlo_call(f32(1.0), source="func.func @f(%a: tensor<f32>) -> tensor<f32> {\n return %a : tensor<f32>\n}")
    with pytest.raises(NotImplementedError):
        hlo_call(f32(1.0), source="func.func @main(%a: tensor<f32>) -> tensor<f32> {\n %b = stablehlo.erf_inv %a : tensor<f32>\n"
                                  " return %b : tensor<f32>\n}")


ELEMENTWISE = [k for k, v in GOLDEN.items() if isinstance(v, dict) and "grads" in v and "perm" not in v]


@pytest.mark.parametrize("name", ELEMENTWISE)
def test_rule_matches_reference_vector_through_text(name):
    """The lit tests' operands, results and reverse-mode cotangents (all-ones result cotangent),
    with the operator written as one line of StableHLO text."""
    from enzyme_ad.jax import hlo_call, jvp, vjp

    g = GOLDEN[name]
    n = len(g["args"][0])
    ty = "tensor<%dxf32>" % n
    names = ["%a", "%b"][:len(g["args"])]
    text = "func.func @main(%s) -> %s {\n  %%r = stablehlo.%s %s : %s\n  return %%r : %s\n}\n" % (
        ", ".join("%s: %s" % (v, ty) for v in names), ty, name, ", ".join(names), ty, ty)
    args = [f32(a) for a in g["args"]]
    fn = lambda *xs: hlo_call(*xs, source=text)[0]
    out, f_vjp = vjp(fn, *args)
    np.testing.assert_allclose(host(out), g["out"], rtol=2e-6, atol=1e-7)
    grads = f_vjp(f32(np.ones(n)))
    for got, want in zip(grads, g["grads"]):
        np.testing.assert_allclose(host(got), want, rtol=3e-6, atol=1e-7)
    # the symbolic programs (what optimize_module prints for the reference's AD pipelines)
    if True:
        from enzyme_ad.jax import stablehlo_ad
        sym = hlo_call(*args, f32(np.ones(n)), source=stablehlo_ad.reverse_module_text(text))
        for got, want in zip(sym, g["grads"]):
            np.testing.assert_allclose(host(got), want, rtol=3e-6, atol=1e-7)
        fwd = stablehlo_ad.forward_module_text(text)
        flat = [v for a in args for v in (a, f32(np.ones(n)))]
        out2, tan2 = hlo_call(*flat, source=fwd)
        np.testing.assert_allclose(host(out2), g["out"], rtol=2e-6, atol=1e-7)
        np.testing.assert_allclose(host(tan2), np.sum(np.asarray(g["grads"]), axis=0), rtol=3e-6, atol=1e-7)
    # forward mode against the same Jacobian: unit tangent on each operand in turn
    for i, want in enumerate(g["grads"]):
        tans = [f32(np.ones(n)) if j == i else None for j in range(len(args))]
        _, t = jvp(fn, tuple(args), tuple(tans))
        np.testing.assert_allclose(host(t), want, rtol=3e-6, atol=1e-7)


def test_clamp_rule_through_text():
    """clamp.mlir:14-34: scalar bounds, the operand's cotangent vanishes outside them (reverse and forward mode)."""
    from enzyme_ad.jax import hlo_call, jvp, vjp, stablehlo_ad

    g = GOLDEN["clamp_operand"]
    text = ("func.func @main(%x: tensor<10xf32>) -> tensor<10xf32> {\n"
            "  %lo = stablehlo.constant dense<1.000000e+00> : tensor<f32>\n"
            "  %hi = stablehlo.constant dense<2.000000e+00> : tensor<f32>\n"
            "  %r = stablehlo.clamp %lo, %x, %hi : (tensor<f32>, tensor<10xf32>, tensor<f32>) -> tensor<10xf32>\n"
            "  return %r : tensor<10xf32>\n}\n")
    x, one = f32(g["operand"]), f32(np.ones(10))
    fn = lambda a: hlo_call(a, source=text)[0]
    out, f_vjp = vjp(fn, x)
    assert np.array_equal(host(out), np.asarray(g["out"]))
    assert np.array_equal(host(f_vjp(one)[0]), np.asarray(g["grad_operand"]))
    _, t = jvp(fn, (x,), (one,))
    assert np.array_equal(host(t), np.asarray(g["grad_operand"]))
    (sym,) = hlo_call(x, one, source=stablehlo_ad.reverse_module_text(text))
    assert np.array_equal(host(sym), np.asarray(g["grad_operand"]))
    out2, tan2 = hlo_call(x, one, source=stablehlo_ad.forward_module_text(text))
    assert np.array_equal(host(out2), np.asarray(g["out"])) and np.array_equal(host(tan2), np.asarray(g["grad_operand"]))


def test_transpose_and_dot_general_rules_through_text():
    from enzyme_ad.jax import hlo_call, vjp

    g = GOLDEN["transpose"]
    text = ("func.func @main(%a: tensor<2x3xf32>) -> tensor<3x2xf32> {\n"
            "  %r = stablehlo.transpose %a, dims = [1, 0] : (tensor<2x3xf32>) -> tensor<3x2xf32>\n"
            "  return %r : tensor<3x2xf32>\n}\n")
    out, f_vjp = vjp(lambda a: hlo_call(a, source=text)[0], f32(g["args"][0]))
    assert np.array_equal(host(out), np.asarray(g["out"]))
    assert np.array_equal(host(f_vjp(f32(g["dret"]))[0]), np.asarray(g["grads"][0]))
    # dot_general.mlir:4-37: c[3,4] = a[2,3] (dim 0) . b[4,2] (dim 1), quoted-generic spelling
    text = ('func.func @main(%a : tensor<2x3xf32>, %b : tensor<4x2xf32>) -> tensor<3x4xf32> {\n'
            '  %c = "stablehlo.dot_general"(%a, %b) {\n'
            '    dot_dimension_numbers = #stablehlo.dot<\n'
            '      lhs_batching_dimensions = [], rhs_batching_dimensions = [],\n'
            '      lhs_contracting_dimensions = [0], rhs_contracting_dimensions = [1]>,\n'
            '    precision_config = [#stablehlo<precision DEFAULT>, #stablehlo<precision DEFAULT>]\n'
            '  } : (tensor<2x3xf32>, tensor<4x2xf32>) -> tensor<3x4xf32>\n'
            '  func.return %c : tensor<3x4xf32>\n}\n')
    rng = np.random.default_rng(0)
    a, b, c = rng.normal(size=(2, 3)), rng.normal(size=(4, 2)), rng.normal(size=(3, 4))
    out, f_vjp = vjp(lambda x, y: hlo_call(x, y, source=text)[0], f32(a), f32(b))
    np.testing.assert_allclose(host(out), np.einsum("ki,jk->ij", a, b), rtol=1e-5, atol=1e-6)
    da, db = f_vjp(f32(c))
    np.testing.assert_allclose(host(da), np.einsum("ij,jk->ki", c, b), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(host(db), np.einsum("ij,ki->jk", c, a), rtol=1e-5, atol=1e-6)


def test_reduce_max_and_broadcast_rules_through_text():
    """Reduce-maximum sends the cotangent to every maximal element, undivided
    (StableHLOAutoDiffOpInterfaceImpl.cpp:1881-1916); broadcast_in_dim sums it back (:1474)."""
    from enzyme_ad.jax import hlo_call, vjp

    text = ("func.func @main(%x: tensor<2x4xf32>, %v: tensor<4xf32>) -> (tensor<2xf32>, tensor<2x4xf32>) {\n"
            "  %m = stablehlo.constant dense<0xFF800000> : tensor<f32>\n"
            "  %r = stablehlo.reduce(%x init: %m) applies stablehlo.maximum across dimensions = [1] : "
            "(tensor<2x4xf32>, tensor<f32>) -> tensor<2xf32>\n"
            "  %b = stablehlo.broadcast_in_dim %v, dims = [1] : (tensor<4xf32>) -> tensor<2x4xf32>\n"
            "  return %r, %b : tensor<2xf32>, tensor<2x4xf32>\n}\n")
    x = f32([[1.0, 3.0, 3.0, -1.0], [0.5, 0.25, -2.0, 0.125]])
    (r, b), f_vjp = vjp(lambda x, v: tuple(hlo_call(x, v, source=text)), x, f32([1.0, 2.0, 3.0, 4.0]))
    assert np.array_equal(host(r), [3.0, 0.5])
    gx, gv = f_vjp((f32([10.0, 20.0]), f32(np.arange(8).reshape(2, 4))))
    assert np.array_equal(host(gx), [[0, 10.0, 10.0, 0], [20.0, 0, 0, 0]])
    assert np.array_equal(host(gv), [4.0, 6.0, 8.0, 10.0])


def test_compare_select_and_reduce_max_through_text_in_all_three_modes():
    """relu-like select on a compare, and a softmax spelled out (reduce-max, exp, reduce-add):
    tape reverse mode, symbolic reverse module and symbolic forward module agree."""
    from enzyme_ad.jax import hlo_call, jvp, stablehlo_ad, vjp

    text = """
    func.func @main(%x: tensor<3x5xf32>, %y: tensor<3x5xf32>) -> (tensor<3x5xf32>, tensor<3x5xf32>) {
      %z = stablehlo.constant dense<0.000000e+00> : tensor<3x5xf32>
      %p = stablehlo.compare GT, %x, %z, FLOAT : (tensor<3x5xf32>, tensor<3x5xf32>) -> tensor<3x5xi1>
      %r = stablehlo.select %p, %x, %y : tensor<3x5xi1>, tensor<3x5xf32>
      %ninf = stablehlo.constant dense<0xFF800000> : tensor<f32>
      %zero = stablehlo.constant dense<0.000000e+00> : tensor<f32>
      %mx = stablehlo.reduce(%r init: %ninf) applies stablehlo.maximum across dimensions = [1] : (tensor<3x5xf32>, tensor<f32>) -> tensor<3xf32>
      %mb = stablehlo.broadcast_in_dim %mx, dims = [0] : (tensor<3xf32>) -> tensor<3x5xf32>
      %e = stablehlo.exponential %r : tensor<3x5xf32>
      %sh = stablehlo.subtract %r, %mb : tensor<3x5xf32>
      %e2 = stablehlo.exponential %sh : tensor<3x5xf32>
      %sm = stablehlo.reduce(%e2 init: %zero) applies stablehlo.add across dimensions = [1] : (tensor<3x5xf32>, tensor<f32>) -> tensor<3xf32>
      %sb = stablehlo.broadcast_in_dim %sm, dims = [0] : (tensor<3xf32>) -> tensor<3x5xf32>
      %soft = stablehlo.divide %e2, %sb : tensor<3x5xf32>
      %mm = stablehlo.maximum %soft, %y : tensor<3x5xf32>
      return %mm, %mb : tensor<3x5xf32>, tensor<3x5xf32>
    }"""
    rng = np.random.default_rng(4)
    x, y = f32(rng.normal(size=(3, 5))), f32(rng.normal(size=(3, 5)) * 0.3)
    c1, c2 = f32(rng.normal(size=(3, 5))), f32(rng.normal(size=(3, 5)))
    tx, ty = f32(rng.normal(size=(3, 5))), f32(rng.normal(size=(3, 5)))
    fn = lambda a, b: tuple(hlo_call(a, b, source=text))
    outs, f_vjp = vjp(fn, x, y)
    r = np.where(host(x) > 0, host(x), host(y))
    e = np.exp(r - r.max(1, keepdims=True))
    np.testing.assert_allclose(host(outs[0]), np.maximum(e / e.sum(1, keepdims=True), host(y)), rtol=1e-6)
    tape = f_vjp((c1, c2))
    sym = hlo_call(x, y, c1, c2, source=stablehlo_ad.reverse_module_text(text))
    for g, t in zip(sym, tape):
        np.testing.assert_allclose(host(g), host(t), rtol=1e-5, atol=1e-6)
    _, tans = jvp(fn, (x, y), (tx, ty))
    fo = hlo_call(x, tx, y, ty, source=stablehlo_ad.forward_module_text(text))
    np.testing.assert_allclose(host(fo[1]), host(tans[0]), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(host(fo[3]), host(tans[1]), rtol=1e-5, atol=1e-6)
    # adjoint identity between the two symbolic programs
    lhs = float(np.sum(host(fo[1]) * host(c1)) + np.sum(host(fo[3]) * host(c2)))
    rhs = float(np.sum(host(sym[0]) * host(tx)) + np.sum(host(sym[1]) * host(ty)))
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), abs(rhs), 1.0)


def test_calls_between_functions_run_and_differentiate():
    """A private function called twice (what nested jit leaves in a traced module): tape modes
    run through the call, the symbolic programs inline it."""
    from enzyme_ad.jax import hlo_call, jvp, stablehlo_ad, vjp

    text = """module @jit_f {
      func.func public @main(%x: tensor<4xf32>, %y: tensor<4xf32>) -> (tensor<4xf32> {jax.result_info = ""}) {
        %0 = call @scale(%x, %y) : (tensor<4xf32>, tensor<4xf32>) -> tensor<4xf32>
        %1 = call @scale(%0, %x) : (tensor<4xf32>, tensor<4xf32>) -> tensor<4xf32>
        return %1 : tensor<4xf32>
      }
      func.func private @scale(%a: tensor<4xf32>, %b: tensor<4xf32>) -> tensor<4xf32> {
        %e = stablehlo.exponential %b : tensor<4xf32>
        %r = stablehlo.multiply %a, %e : tensor<4xf32>
        return %r : tensor<4xf32>
      }
    }"""
    x, y, c, tx, ty = (f32(v) for v in ([0.1, 0.2, -0.3, 0.4], [1.0, -1.0, 0.5, 0.0], [1.0, 2.0, 3.0, 4.0], [0.5, 0.5, 0.5, 0.5], [1.0, 0.0, -1.0, 2.0]))
    fn = lambda a, b: hlo_call(a, b, source=text)[0]
    out, f_vjp = vjp(fn, x, y)
    xr, yr = host(x), host(y)
    np.testing.assert_allclose(host(out), xr * np.exp(yr) * np.exp(xr), rtol=1e-6)
    gx, gy = f_vjp(c)
    np.testing.assert_allclose(host(gx), host(c) * np.exp(yr) * np.exp(xr) * (1 + xr), rtol=1e-5)
    np.testing.assert_allclose(host(gy), host(c) * host(out), rtol=1e-5)
    sym = hlo_call(x, y, c, source=stablehlo_ad.reverse_module_text(text))
    np.testing.assert_allclose(host(sym[0]), host(gx), rtol=1e-6)
    np.testing.assert_allclose(host(sym[1]), host(gy), rtol=1e-6)
    _, t = jvp(fn, (x, y), (tx, ty))
    fo = hlo_call(x, tx, y, ty, source=stablehlo_ad.forward_module_text(text))
    np.testing.assert_allclose(host(fo[1]), host(t), rtol=1e-6)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_gather_row_lookup_through_text_in_all_three_modes(dt):
    """The reference's gather.mlir input (an embedding lookup table[indices], indices [45, 1]) run from its text:
    value against numpy indexing, reverse mode against the oracle's scatter-add (repeated indices accumulate), the
    symbolic reverse and forward programs through hlo_call against the tape."""
    from enzyme_ad.jax import hlo_call, jvp, stablehlo_ad, vjp
    from oracle import ad_rules as R
    fixture = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "lit_primal_functions.json")))
    (fn_text,) = fixture["gather.mlir"]
    ty = "f32" if dt == "f32" else "bf16"
    text = "module {\n" + fn_text.replace("f32", ty) + "\n}"
    rng = np.random.default_rng(17)
    table, tr = dev(rng.standard_normal((64, 3)), dt)
    ttab, ttr = dev(rng.standard_normal((64, 3)), dt)
    c, cr = dev(rng.standard_normal((45, 3)), dt)
    idx_np = rng.integers(0, 64, size=(45, 1)).astype(np.int32)
    idx_np[7] = idx_np[3]                                   # a repeated row
    idx = torch.from_numpy(idx_np).cuda()
    fn = lambda t: hlo_call(t, idx, source=text)[0]
    out, f_vjp = vjp(fn, table)
    assert np.array_equal(host(out), R.gather_rows(tr, idx_np))
    (g,) = f_vjp(c)
    (rg,) = R.vjp_gather_rows(tr, idx_np, cr)
    assert np.max(np.abs(host(g) - rg)) <= (1e-6 if dt == "f32" else 2e-2) * np.max(np.abs(rg))
    _, t = jvp(fn, (table,), (ttab,))
    assert np.array_equal(host(t), R.gather_rows(ttr, idx_np))
    rev = hlo_call(table, idx, c, source=stablehlo_ad.reverse_module_text(text, arg_active=[True, False]))
    assert np.max(np.abs(host(rev[0]) - rg)) <= (1e-6 if dt == "f32" else 2e-2) * np.max(np.abs(rg))
    fwd = hlo_call(table, ttab, idx, source=stablehlo_ad.forward_module_text(text, arg_active=[True, False]))
    assert np.array_equal(host(fwd[0]), host(out)) and np.array_equal(host(fwd[1]), host(t))


@pytest.mark.parametrize("dt,rows,V,select_form", [("f32", (64,), 1000, False), ("f32", (3, 21), 517, True), ("bf16", (40,), 4096, False)])
def test_traced_cross_entropy_through_text_in_all_three_modes(dt, rows, V, select_form):
    """A traced mean softmax cross-entropy (log_softmax, one-hot from run-time integer targets, sum, mean) run from
    its text: the cluster is matched onto the cross-entropy kernels; value, gradient and tangent against the
    oracle (logsumexp(z) - z[target], (softmax - onehot) / n, targets outside [0, V) contributing nothing), and the
    symbolic reverse and forward programs through hlo_call against the same figures."""
    from enzyme_ad.jax import hlo_call, jvp, stablehlo, stablehlo_ad, vjp
    from oracle import llama_ref as L
    from test_stablehlo_frontend import traced_cross_entropy_text
    text = traced_cross_entropy_text(rows, V, dt=dt, select_form=select_form)
    assert stablehlo.Executable(text).fused == {"cross_entropy": 1}
    n = int(np.prod(rows))
    rng = np.random.default_rng(23)
    z, zr = dev(3.0 * rng.standard_normal(rows + (V,)), dt)
    tz, tzr = dev(rng.standard_normal(rows + (V,)), dt)
    tgt_np = rng.integers(0, V, size=rows).astype(np.int32)
    tgt_np.reshape(-1)[1] = -1                       # masked rows: no class matches
    tgt_np.reshape(-1)[5] = V
    tgt = torch.from_numpy(tgt_np).cuda()
    loss_rows, _ = L.cross_entropy_fwd(zr.reshape(n, V), tgt_np.reshape(n))
    want = float(np.sum(loss_rows) / n)
    tol = 1e-5 if dt == "f32" else 2e-2
    fn = lambda a: hlo_call(a, tgt, source=text)[0]
    out, f_vjp = vjp(fn, z)
    assert abs(float(host(out)) - want) <= tol * abs(want)
    one = torch.ones((), device="cuda", dtype=torch.float32 if dt == "f32" else torch.bfloat16)
    (g,) = f_vjp(one)
    rg = L.cross_entropy_bwd(zr.reshape(n, V), tgt_np.reshape(n), np.full(n, 1.0 / n)).reshape(rows + (V,))
    assert np.max(np.abs(host(g) - rg)) <= (2e-6 if dt == "f32" else 2e-2) * np.max(np.abs(rg))
    assert not host(g).reshape(n, V)[1].any() and not host(g).reshape(n, V)[5].any()
    _, t = jvp(fn, (z,), (tz,))
    rt = float(np.sum(L.cross_entropy_jvp(zr.reshape(n, V), tgt_np.reshape(n), tzr.reshape(n, V))) / n)
    assert abs(float(host(t)) - rt) <= (1e-4 if dt == "f32" else 3e-2) * max(abs(rt), 0.05)
    rev = hlo_call(z, tgt, one, source=stablehlo_ad.reverse_module_text(text))
    assert np.max(np.abs(host(rev[0]) - rg)) <= (2e-6 if dt == "f32" else 2e-2) * np.max(np.abs(rg))
    fwd = hlo_call(z, tz, tgt, source=stablehlo_ad.forward_module_text(text))
    assert abs(float(host(fwd[0])) - want) <= tol * abs(want)
    assert abs(float(host(fwd[1])) - rt) <= (1e-4 if dt == "f32" else 3e-2) * max(abs(rt), 0.05)
