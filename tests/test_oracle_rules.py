"""Pins oracle/ad_rules.py against the known-answer vectors the reference keeps
in test/lit_tests/diffrules/stablehlo/*.mlir (tests/golden/diffrules.json)."""
import json
import os

import numpy as np
import pytest

from oracle import ad_rules as R

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "diffrules.json")))

FWD = {
    "multiply": lambda a, b: a * b, "divide": lambda a, b: a / b, "add": lambda a, b: a + b,
    "subtract": lambda a, b: a - b, "negate": lambda a: -a, "exponential": np.exp,
    "sqrt": np.sqrt, "rsqrt": lambda a: 1 / np.sqrt(a), "logistic": R.logistic,
    "maximum": np.maximum, "power": np.power, "cosine": np.cos, "sine": np.sin,
    "minimum": np.minimum, "abs": np.abs, "log": np.log, "log_plus_one": np.log1p, "exponential_minus_one": np.expm1,
    "cbrt": np.cbrt, "tanh": np.tanh, "atan2": np.arctan2,
}


@pytest.mark.parametrize("name", sorted(FWD))
def test_elementwise_rule_matches_reference_vector(name):
    g = GOLD[name]
    args = [np.array(a, dtype=np.float64) for a in g["args"]]
    out = FWD[name](*args)
    np.testing.assert_allclose(out, g["out"], rtol=2e-7, atol=1e-7)
    d = np.ones_like(out)
    grads = getattr(R, "vjp_" + name)(*args, d)
    assert len(grads) == len(g["grads"])
    for got, want in zip(grads, g["grads"]):
        np.testing.assert_allclose(got, want, rtol=2e-7, atol=1e-7)


def test_transpose_rule_matches_reference_vector():
    g = GOLD["transpose"]
    x = np.array(g["args"][0])
    np.testing.assert_array_equal(np.transpose(x, g["perm"]), g["out"])
    (dx,) = R.vjp_transpose(x, g["perm"], np.array(g["dret"]))
    np.testing.assert_array_equal(dx, g["grads"][0])


def test_dot_general_rule_has_reference_ir_form():
    """dot_general.mlir:25-37: da = transpose(dc . b), db = dc^T-contract a.
    Evaluate the IR form literally with einsum and compare with the NT rule the
    oracle uses after renaming operands (c = a^T b^T  <=>  Y = X W^T with
    X = a^T, W = b)."""
    rng = np.random.default_rng(0)
    a = rng.standard_normal((2, 3))
    b = rng.standard_normal((4, 2))
    dc = rng.standard_normal((3, 4))
    da_ir = np.einsum("ij,jk->ik", dc, b).T          # %1 then transpose [1,0]
    db_ir = np.einsum("ij,ki->jk", dc, a)            # contract dc dim0 with a dim1
    dX, dW = R.vjp_matmul_nt(a.T, b, dc)
    np.testing.assert_allclose(dX.T, da_ir, rtol=1e-14)
    np.testing.assert_allclose(dW, db_ir, rtol=1e-14)
    # adjoint identity against numpy matmul
    v = rng.standard_normal(a.shape)
    jv = (v.T) @ b.T
    assert np.isclose(np.sum(jv * dc), np.sum(v * da_ir))


def test_sqrt_zero_guard_and_max_ties():
    (g,) = R.vjp_sqrt(np.array([0.0]), np.array([3.0]))
    assert g[0] == 0.0
    da, db = R.vjp_maximum(np.array([1.5]), np.array([1.5]), np.array([1.0]))
    assert da[0] == 1.0 and db[0] == 0.0


def test_reduce_and_broadcast_rules_are_adjoint():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, 5))
    w = rng.standard_normal(3)
    (dx,) = R.vjp_reduce_add(x, 1, w)
    v = rng.standard_normal((3, 5))
    assert np.isclose(np.sum(np.sum(v, axis=1) * w), np.sum(v * dx))
    (dm,) = R.vjp_reduce_max(np.array([[1.0, 3.0, 3.0]]), 1, np.array([2.0]))
    np.testing.assert_array_equal(dm, [[0.0, 2.0, 2.0]])     # every arg-max, undivided
    xb = rng.standard_normal((5,))
    d = rng.standard_normal((3, 5))
    (g,) = R.vjp_broadcast_in_dim(xb, (3, 5), (1,), d)
    np.testing.assert_allclose(g, d.sum(0))
    parts = R.vjp_concatenate([np.zeros((2, 4)), np.zeros((1, 4))], 0, np.arange(12.0).reshape(3, 4))
    assert parts[0].shape == (2, 4) and parts[1][0, 0] == 8.0
    (gs,) = R.vjp_slice(np.zeros((4,)), (1,), (3,), np.array([5.0, 6.0]))
    np.testing.assert_array_equal(gs, [0, 5, 6, 0])


def test_clamp_rule_matches_reference_vector():
    g = GOLD["clamp_operand"]
    x = np.array(g["operand"])
    np.testing.assert_array_equal(np.clip(x, g["min"], g["max"]), g["out"])
    (dx,) = R.vjp_clamp_operand(g["min"], x, g["max"], np.ones_like(x))
    np.testing.assert_array_equal(dx, g["grad_operand"])


def test_select_rule_has_reference_ir_form():
    """select.mlir REVERSE check lines, evaluated by hand on a vector: the cotangent d goes to
    on_true where pred holds and to on_false elsewhere (`select %pred, %d, %zero` /
    `select %pred, %zero, %d`); the predicate is inactive (HLODerivatives.td:1297-1304)."""
    pred = np.array([True, False, True, False])
    a = np.array([1.0, 2.0, 3.0, 4.0])
    b = np.array([-1.0, -2.0, -3.0, -4.0])
    d = np.array([3.0, 5.0, 7.0, 11.0])
    da, db = R.vjp_select(pred, a, b, d)
    np.testing.assert_array_equal(da, [3.0, 0.0, 7.0, 0.0])
    np.testing.assert_array_equal(db, [0.0, 5.0, 0.0, 11.0])
    # the two cotangents partition d, and J^T is the transpose of the forward's linear map
    np.testing.assert_array_equal(da + db, d)
    rng = np.random.default_rng(2)
    va, vb = rng.standard_normal(4), rng.standard_normal(4)
    assert np.isclose(np.sum(np.where(pred, va, vb) * d), np.sum(va * da) + np.sum(vb * db))
    # FORWARD check lines: the tangent is select(pred, ta, tb)
    eps = 1e-6
    fd = (np.where(pred, a + eps * va, b + eps * vb) - np.where(pred, a - eps * va, b - eps * vb)) / (2 * eps)
    np.testing.assert_allclose(np.sum(fd * d), np.sum(va * da) + np.sum(vb * db), rtol=1e-9)


def test_reshape_rule_is_row_major_inverse():
    """HLODerivatives.td:1271: the cotangent is reshaped to the operand's type. Element k of the
    flattened cotangent must land on element k of the flattened operand (row-major both ways)."""
    x = np.zeros((2, 3))
    d = np.array([[0.0, 1.0], [2.0, 3.0], [4.0, 5.0]])            # cotangent of reshape(x, (3, 2))
    (dx,) = R.vjp_reshape(x, d)
    np.testing.assert_array_equal(dx, [[0.0, 1.0, 2.0], [3.0, 4.0, 5.0]])
    rng = np.random.default_rng(3)
    v = rng.standard_normal((2, 3, 4))
    w = rng.standard_normal((6, 4))
    (g,) = R.vjp_reshape(v, w)
    assert g.shape == v.shape
    assert np.isclose(np.sum(np.reshape(v, (6, 4)) * w), np.sum(v * g))
    # a transposing "reshape" (the plausible mistake) fails the index check above: (2,3)->(3,2) via .T
    assert not np.array_equal(d.T, dx)


def test_convert_rule_returns_operand_type():
    """HLODerivatives.td:1290-1295: `Convert (TypeOf $x), (DiffeRet)`: the cotangent takes the operand's
    element type, with that type's rounding (a float64 cotangent of a float32 operand loses its low bits;
    float16 likewise)."""
    x32 = np.array([1.0, 2.0], dtype=np.float32)
    d64 = np.array([1.0 + 2.0 ** -30, 3.0], dtype=np.float64)
    (g,) = R.vjp_convert(x32, d64)
    assert g.dtype == np.float32
    np.testing.assert_array_equal(g, np.array([1.0, 3.0], dtype=np.float32))
    x16 = np.array([1.0], dtype=np.float16)
    (g16,) = R.vjp_convert(x16, np.array([1.0 + 2.0 ** -12], dtype=np.float32))
    assert g16.dtype == np.float16 and g16[0] == np.float16(1.0)
    # widening is exact, so <convert(v), w> = <v, convert^T(w)> holds bit for bit for representable values
    v = np.array([0.5, -1.25], dtype=np.float32)
    w = np.array([2.0, 4.0], dtype=np.float64)
    (gt,) = R.vjp_convert(v, w)
    assert float(np.sum(v.astype(np.float64) * w)) == float(np.sum(v * gt))


def test_gather_rows_rule_scatter_adds_repeated_indices():
    """gather.mlir REVERSE check lines: the cotangent rows are scatter-added into a zero table, so an index that
    occurs twice receives the sum of both rows and rows nobody looked up stay zero."""
    table = np.arange(12.0).reshape(4, 3)
    idx = np.array([[2], [0], [2]])
    np.testing.assert_array_equal(R.gather_rows(table, idx), table[[2, 0, 2]])
    d = np.array([[1.0, 2.0, 3.0], [10.0, 20.0, 30.0], [100.0, 200.0, 300.0]])
    (g,) = R.vjp_gather_rows(table, idx, d)
    np.testing.assert_array_equal(g, [[10.0, 20.0, 30.0], [0.0, 0.0, 0.0], [101.0, 202.0, 303.0], [0.0, 0.0, 0.0]])
    rng = np.random.default_rng(5)
    v = rng.standard_normal(table.shape)
    assert np.isclose(np.sum(R.gather_rows(v, idx) * d), np.sum(v * g))     # <J v, w> = <v, J^T w>
    # out of range: the lookup clamps, the scatter drops
    np.testing.assert_array_equal(R.gather_rows(table, np.array([[7]])), table[[3]])
    np.testing.assert_array_equal(R.vjp_gather_rows(table, np.array([[7]]), np.ones((1, 3)))[0], np.zeros((4, 3)))
