"""CPU oracle, part 1: the per-operation reverse-mode rules of the reference.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this
module; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do.

Each function restates one rule of the reference's StableHLO derivative table
(src/enzyme_ad/jax/Implementations/HLODerivatives.td, cited per function) or of
its C++ adjoint classes (Implementations/StableHLOAutoDiffOpInterfaceImpl.cpp)
in numpy.  A rule `vjp_<op>(primal operands..., dret)` returns the cotangent
of every operand.  The rules are pinned by the known-answer vectors the
reference keeps in test/lit_tests/diffrules/stablehlo/*.mlir (committed as data
in tests/golden/diffrules.json and checked by tests/test_oracle_rules.py).

Pinning status:
  add, subtract, multiply, divide, negate, exponential, sqrt, rsqrt, logistic,
  maximum, power, cosine, sine, transpose ... pinned by the lit vectors.
  dot_general ... pinned by the IR form in dot_general.mlir (operand order and
      transposition) plus the <Jv,w> = <v,J^T w> identity against numpy matmul.
  reduce(add), broadcast_in_dim, concatenate, slice ... pinned by the adjoint
      identity and hand-worked index cases (tests/test_oracle_rules.py).
  select ... pinned by the REVERSE / FORWARD check lines of select.mlir
      evaluated by hand on a vector, plus the adjoint identity.
  reshape ... pinned by a hand-worked row-major index case + adjoint identity.
  convert ... pinned by the result element type and its rounding.
  gather (row lookup) ... pinned by a hand-worked case with a repeated index and the
      adjoint identity against numpy indexing; its IR forms by gather.mlir's check lines.
  reduce(max) ... no numeric vector in the reference; pinned by the closed form
      stated in the C++ (cotangent to every element equal to the max) and by
      the softmax shift-invariance test (its contribution cancels).
"""
import numpy as np


def _checked_mul(d, x):
    # HLODerivatives.td:127-132 (CheckedMul): under strong-zero mode a zero
    # cotangent stays zero even when x is inf/nan; otherwise a plain product.
    return d * x


def _checked_div(d, x):
    # HLODerivatives.td:134-139 (CheckedDiv)
    return d / x


def vjp_add(x, y, d):
    """HLODerivatives.td:964-970 AddOp: both operands receive the cotangent."""
    return d, d


def vjp_subtract(x, y, d):
    """HLODerivatives.td:1312-1318 SubtractOp."""
    return d, -d


def vjp_negate(x, d):
    """HLODerivatives.td:1228 NegOp."""
    return (-d,)


def vjp_multiply(x, y, d):
    """HLODerivatives.td:1221-1226 MulOp."""
    return _checked_mul(d, y), _checked_mul(d, x)


def vjp_divide(x, y, d):
    """HLODerivatives.td:1133-1139 DivOp: dx = d/y, dy = -(d/y)*(x/y)."""
    q = _checked_div(d, y)
    return q, -_checked_mul(q, x / y)


def vjp_exponential(x, d):
    """HLODerivatives.td:1182 ExpOp."""
    return (_checked_mul(d, np.exp(x)),)


def vjp_sqrt(x, d):
    """HLODerivatives.td:1320-1324 SqrtOp: zero where x == 0."""
    x = np.asarray(x)
    with np.errstate(divide="ignore", invalid="ignore"):
        g = d / (2.0 * np.sqrt(x))
    return (np.where(x == 0, np.zeros_like(g), g),)


def vjp_rsqrt(x, d):
    """HLODerivatives.td:1283-1288 RsqrtOp: d / (-2 * x * sqrt(x))."""
    return (_checked_div(d, -2.0 * (x * np.sqrt(x))),)


def logistic(x):
    return 1.0 / (1.0 + np.exp(-x))


def vjp_logistic(x, d):
    """HLODerivatives.td:1203 LogisticOp: d * s * (1 - s)."""
    s = logistic(x)
    return (_checked_mul(d, _checked_mul(s, 1.0 - s)),)


def vjp_maximum(x, y, d):
    """HLODerivatives.td:1205-1211 MaxOp: ties go to the first operand."""
    lt = x < y
    z = np.zeros_like(d)
    return np.where(lt, z, d), np.where(lt, d, z)


def vjp_power(x, y, d):
    """HLODerivatives.td:1237-1242 PowOp."""
    return (_checked_mul(d, y * np.power(x, y - 1.0)),
            _checked_mul(d, np.power(x, y) * np.log(x)))


def vjp_minimum(x, y, d):
    """HLODerivatives.td:1213-1219 MinOp: y < x sends the cotangent to y, ties go to the first operand."""
    lt = y < x
    z = np.zeros_like(d)
    return np.where(lt, z, d), np.where(lt, d, z)


def vjp_abs(x, d):
    """HLODerivatives.td:1244 AbsOp, real operands: select(x >= 0, d, -d) (abs.mlir:21-27)."""
    return (np.where(x >= 0, d, -d),)


def vjp_log(x, d):
    """HLODerivatives.td:1199 LogOp."""
    return (_checked_div(d, x),)


def vjp_log_plus_one(x, d):
    """HLODerivatives.td:1201 Log1pOp."""
    return (_checked_div(d, x + 1.0),)


def vjp_exponential_minus_one(x, d):
    """HLODerivatives.td:1184 Expm1Op."""
    return (_checked_mul(d, np.exp(x)),)


def vjp_cbrt(x, d):
    """HLODerivatives.td:1085-1087 CbrtOp: d / (3 cbrt(x)^2), real for negative x too."""
    c = np.cbrt(x)
    return (_checked_div(d, 3.0 * (c * c)),)


def vjp_tanh(x, d):
    """HLODerivatives.td:1326-1330 TanhOp."""
    t = np.tanh(x)
    return (_checked_mul(d, 1.0 - t * t),)


def vjp_atan2(y, x, d):
    """HLODerivatives.td:972-978 Atan2Op (operands in the order y, x)."""
    den = x * x + y * y
    return _checked_mul(d, x / den), _checked_mul(d, -y / den)


def vjp_clamp_operand(lo, x, hi, d):
    """HLODerivatives.td:1050-1066 ClampOp, cotangent of the clamped operand: none outside [lo, hi]."""
    return (np.where((x < lo) | (x > hi), 0.0, d),)


def vjp_cosine(x, d):
    """HLODerivatives.td:1129 CosineOp."""
    return (_checked_mul(d, -np.sin(x)),)


def vjp_sine(x, d):
    """HLODerivatives.td:1308 SineOp."""
    return (_checked_mul(d, np.cos(x)),)


def vjp_transpose(x, perm, d):
    """HLODerivatives.td:1334-1339 TransposeOp: inverse permutation."""
    inv = np.argsort(np.asarray(perm))
    return (np.transpose(d, inv),)


def vjp_reshape(x, d):
    """HLODerivatives.td:1271 ReshapeOp."""
    return (np.reshape(d, np.shape(x)),)


def vjp_convert(x, d):
    """HLODerivatives.td:1290-1295 ConvertOp: cotangent converted back to the
    operand's element type."""
    return (np.asarray(d).astype(np.asarray(x).dtype),)


def vjp_select(cond, a, b, d):
    """HLODerivatives.td:1297-1304 SelectOp."""
    z = np.zeros_like(d)
    return np.where(cond, d, z), np.where(cond, z, d)


def gather_rows(table, indices):
    """stablehlo.gather in the form an embedding lookup traces to (gather.mlir:4-7): indices [..., 1] select whole
    rows of table [V, D]; out-of-range indices are clamped (the gather semantics)."""
    idx = np.clip(np.asarray(indices)[..., 0], 0, table.shape[0] - 1)
    return table[idx]


def vjp_gather_rows(table, indices, d):
    """HLODerivatives.td:1022-1046 GatherOp: scatter-add of the cotangent rows into a zero tensor shaped like the
    operand (REVERSE check lines of gather.mlir: `stablehlo.scatter` with an add region on a zero constant, repeated
    indices accumulate); the indices are inactive.  Updates whose index falls outside the operand are dropped (the
    scatter semantics)."""
    idx = np.asarray(indices)[..., 0].reshape(-1)
    g = np.zeros_like(table)
    rows = np.asarray(d).reshape(-1, table.shape[1])
    live = (idx >= 0) & (idx < table.shape[0])
    np.add.at(g, idx[live], rows[live])
    return (g,)


def vjp_matmul_nt(x, w, d):
    """DotGeneralOp rule, HLODerivatives.td:1166-1178, specialised to
    Y[T,out] = X[T,in] . W[out,in]^T (contracting dim 1 of both operands).

    The rule contracts the result cotangent with the *other* operand and
    transposes into the operand's own layout (IR form pinned by
    test/lit_tests/diffrules/stablehlo/dot_general.mlir:25-37):
        dX = dY . W      (contract `out`)
        dW = dY^T . X    (contract `T`)
    """
    return d @ w, d.T @ x


def vjp_reduce_add(x, axis, d):
    """StableHLOAutoDiffOpInterfaceImpl.cpp:1865-1879: broadcast the cotangent
    back over the reduced dimensions."""
    return (np.broadcast_to(np.expand_dims(d, axis), np.shape(x)).copy(),)


def vjp_reduce_max(x, axis, d):
    """StableHLOAutoDiffOpInterfaceImpl.cpp:1881-1916: every element equal to
    the maximum receives the full cotangent (no division by the tie count)."""
    m = np.max(x, axis=axis, keepdims=True)
    db = np.broadcast_to(np.expand_dims(d, axis), np.shape(x))
    return (np.where(x == m, db, np.zeros_like(db)),)


def vjp_broadcast_in_dim(x, out_shape, bdims, d):
    """StableHLOAutoDiffOpInterfaceImpl.cpp:1474-1573: sum the cotangent over
    the dimensions that were created or expanded by the broadcast."""
    x = np.asarray(x)
    red = [i for i in range(len(out_shape)) if i not in bdims]
    g = np.sum(d, axis=tuple(red)) if red else np.asarray(d)
    # dims that were size-1 in x and expanded
    for ax, n in enumerate(x.shape):
        if n == 1 and g.shape[ax] != 1:
            g = np.sum(g, axis=ax, keepdims=True)
    return (g,)


def vjp_concatenate(xs, axis, d):
    """StableHLOAutoDiffOpInterfaceImpl.cpp:2015-2059: slice the cotangent."""
    out, off = [], 0
    for x in xs:
        n = np.shape(x)[axis]
        idx = [slice(None)] * np.ndim(d)
        idx[axis] = slice(off, off + n)
        out.append(d[tuple(idx)])
        off += n
    return tuple(out)


def vjp_slice(x, start, limit, d):
    """StableHLOAutoDiffOpInterfaceImpl.cpp:1586-1620: pad the cotangent with
    zeros back to the operand's shape (unit strides)."""
    g = np.zeros(np.shape(x), dtype=np.asarray(d).dtype)
    g[tuple(slice(s, l) for s, l in zip(start, limit))] = d
    return (g,)
