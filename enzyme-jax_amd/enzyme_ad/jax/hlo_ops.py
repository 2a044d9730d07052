"""Generic StableHLO operators on the device, with their forward- and reverse-mode rules.

These are the operators of a module that reaches the library as text (`hlo_call`,
src/enzyme_ad/jax/primitives.py:1052-1108) and that the cluster matcher leaves unfused:
elementwise maps, convert, broadcast_in_dim, reduce (add / maximum), transpose,
dot_general, slice, concatenate.  Each one runs a kernel of csrc/tensor_ops.hip (or the
GEMM) through the C ABI and records the reference's rule for it on the active tape
(Implementations/HLODerivatives.td: Add :964, Div :1133, DotGeneral :1166, Exp :1182,
Max :1205, Mul :1221, Neg :1228, Reshape :1271, Rsqrt :1283, Convert :1290, Sub :1312,
Sqrt :1320, Transpose :1334; StableHLOAutoDiffOpInterfaceImpl.cpp: BroadcastInDim :1474,
Slice :1586, Reduce :1833-1916, Concatenate :2015).  The rules themselves are computed with
the same kernels, outside the tape.
"""
import ctypes

import torch

from . import _native as N
from .ops import Tape, _accumulate, _code, _p, _quiet, _set_tan, _stream, _tan

BINARY = {"add": 0, "subtract": 1, "multiply": 2, "divide": 3, "maximum": 4, "minimum": 5, "ge": 6, "eq": 7,
          "nmul": 8, "power": 9, "d_sqrt": 10, "d_rsqrt": 11, "d_logistic": 12, "d_tanh": 13, "d_sin": 14,
          "d_cos": 15, "d_pow_a": 16, "d_pow_b": 17, "d_abs": 18, "d_log1p": 19, "d_expm1": 20, "d_cbrt": 21, "atan2": 22}
UNARY = {"negate": 32, "exponential": 33, "log": 34, "sqrt": 35, "rsqrt": 36, "logistic": 37, "tanh": 38,
         "sine": 39, "cosine": 40, "abs": 41, "copy": 42, "log_plus_one": 43, "exponential_minus_one": 44, "cbrt": 45}
REDUCE = {"add": 0, "maximum": 4}


def _prod(xs):
    r = 1
    for x in xs:
        r *= int(x)
    return r


def _need_cuda(*ts):
    for t in ts:
        if not t.is_cuda:
            raise RuntimeError("operand is not in device memory: the HIP path has no CPU fallback")


def _i64(xs):
    return (ctypes.c_int64 * max(len(xs), 1))(*[int(x) for x in xs])


def _contiguous_strides(shape):
    st, acc = [], 1
    for d in reversed(shape):
        st.append(acc)
        acc *= int(d)
    return list(reversed(st))


# ---------------------------------------------------------------------------
# kernels without tape (used by the operators below and by their rules)
# ---------------------------------------------------------------------------

def _copy_box(src, dims, in_strides, in_off, dst, out_strides, out_off):
    _need_cuda(src, dst)
    if src.element_size() != dst.element_size():
        raise TypeError("strided copy between element sizes %d and %d" % (src.element_size(), dst.element_size()))
    N.check(N.lib().emi_strided_copy(_stream(), _p(src), _p(dst), len(dims), _i64(dims), _i64(in_strides), int(in_off),
                                     _i64(out_strides), int(out_off), src.element_size()))


def _contig(t):
    if t.is_contiguous():
        return t
    out = torch.empty(t.shape, dtype=t.dtype, device=t.device)
    _copy_box(t, list(t.shape), list(t.stride()), 0, out, _contiguous_strides(t.shape), 0)
    return out


def _bin(name, a, b):
    """Elementwise op(a, b); a rank-0 operand is broadcast by the kernel."""
    _need_cuda(a, b)
    if a.dtype != b.dtype:
        raise TypeError("%s: mixed dtypes %s and %s" % (name, a.dtype, b.dtype))
    a, b = _contig(a), _contig(b)
    sa = a.dim() == 0 and b.dim() > 0
    sb = b.dim() == 0 and a.dim() > 0
    if not (sa or sb) and a.shape != b.shape:
        raise ValueError("%s: shapes %s and %s" % (name, tuple(a.shape), tuple(b.shape)))
    y = torch.empty(b.shape if sa else a.shape, dtype=a.dtype, device=a.device)
    N.check(N.lib().emi_map_binary(_stream(), BINARY[name], _p(a), _p(b), _p(y), y.numel(), int(sa), int(sb), _code(a)))
    return y


def _un(name, x):
    _need_cuda(x)
    x = _contig(x)
    y = torch.empty_like(x)
    N.check(N.lib().emi_map_unary(_stream(), UNARY[name], _p(x), _p(y), x.numel(), _code(x)))
    return y


def _convert(x, dtype):
    _need_cuda(x)
    x = _contig(x)
    y = torch.empty(x.shape, dtype=dtype, device=x.device)
    N.check(N.lib().emi_convert(_stream(), _p(x), _p(y), x.numel(), _code(x), _code(y)))
    return y


COMPARE = {"EQ": 0, "NE": 1, "GE": 2, "GT": 3, "LE": 4, "LT": 5}


def _compare(direction, a, b):
    """i1 tensor (torch.bool, one byte per element) of direction(a, b); rank-0 operands broadcast."""
    _need_cuda(a, b)
    if a.dtype != b.dtype:
        raise TypeError("compare: mixed dtypes %s and %s" % (a.dtype, b.dtype))
    a, b = _contig(a), _contig(b)
    sa = a.dim() == 0 and b.dim() > 0
    sb = b.dim() == 0 and a.dim() > 0
    if not (sa or sb) and a.shape != b.shape:
        raise ValueError("compare: shapes %s and %s" % (tuple(a.shape), tuple(b.shape)))
    m = torch.empty(b.shape if sa else a.shape, dtype=torch.bool, device=a.device)
    N.check(N.lib().emi_compare(_stream(), COMPARE[direction], _p(a), _p(b), _p(m), m.numel(), int(sa), int(sb), _code(a)))
    return m


def _select(m, a, b):
    _need_cuda(m, a, b)
    if m.dtype != torch.bool or a.dtype != b.dtype:
        raise TypeError("select: predicate %s, values %s and %s" % (m.dtype, a.dtype, b.dtype))
    m, a, b = _contig(m), _contig(a), _contig(b)
    shape = max((tuple(t.shape) for t in (m, a, b)), key=len)
    flags = []
    for t in (m, a, b):
        if tuple(t.shape) == shape:
            flags.append(0)
        elif t.dim() == 0:
            flags.append(1)
        else:
            raise ValueError("select: shapes %s, %s, %s" % (tuple(m.shape), tuple(a.shape), tuple(b.shape)))
    y = torch.empty(shape, dtype=a.dtype, device=a.device)
    N.check(N.lib().emi_select(_stream(), _p(m), _p(a), _p(b), _p(y), y.numel(), flags[0], flags[1], flags[2], _code(a)))
    return y


def _permute(x, perm):
    out = torch.empty([x.shape[p] for p in perm], dtype=x.dtype, device=x.device)
    _copy_box(x, list(out.shape), [x.stride(p) for p in perm], 0, out, _contiguous_strides(out.shape), 0)
    return out


def _broadcast(x, shape, dims):
    shape = [int(s) for s in shape]
    if len(dims) != x.dim():
        raise ValueError("broadcast_in_dim: %d dims for a rank-%d operand" % (len(dims), x.dim()))
    strides = [0] * len(shape)
    for i, d in enumerate(dims):
        if x.shape[i] != shape[d] and x.shape[i] != 1:
            raise ValueError("broadcast_in_dim: operand dim %d (%d) does not fit result dim %d (%d)" %
                             (i, x.shape[i], d, shape[d]))
        strides[d] = x.stride(i) if x.shape[i] == shape[d] else 0
    out = torch.empty(shape, dtype=x.dtype, device=x.device)
    _copy_box(x, shape, strides, 0, out, _contiguous_strides(shape), 0)
    return out


def _slice(x, start, limit, stride):
    if all(st == 1 for st in stride):
        v = x                                   # unit strides: a view, no kernel; consumers that
        for d, (s, l) in enumerate(zip(start, limit)):     # need contiguous memory copy it then
            if s != 0 or l != x.shape[d]:
                v = v.narrow(d, s, max(0, l - s))
        return v
    shape = [max(0, -(-(l - s) // st)) for s, l, st in zip(start, limit, stride)]
    out = torch.empty(shape, dtype=x.dtype, device=x.device)
    off = sum(s * xs for s, xs in zip(start, x.stride()))
    _copy_box(x, shape, [xs * st for xs, st in zip(x.stride(), stride)], off, out, _contiguous_strides(shape), 0)
    return out


def _scatter_box(c, shape, start, stride):
    """Zeros of `shape` with c written at start + i * stride (the adjoint of slice)."""
    out = torch.zeros(shape, dtype=c.dtype, device=c.device)          # device memset
    os_ = _contiguous_strides(shape)
    c = _contig(c)
    _copy_box(c, list(c.shape), list(c.stride()), 0, out, [o * st for o, st in zip(os_, stride)],
              sum(s * o for s, o in zip(start, os_)))
    return out


def _concat(xs, dim):
    shape = list(xs[0].shape)
    shape[dim] = sum(x.shape[dim] for x in xs)
    out = torch.empty(shape, dtype=xs[0].dtype, device=xs[0].device)
    os_ = _contiguous_strides(shape)
    at = 0
    for x in xs:
        _copy_box(x, list(x.shape), list(x.stride()), 0, out, os_, at * os_[dim])
        at += x.shape[dim]
    return out


def _reduce(kind, x, dims):
    """Sum or maximum of x over `dims` (removed from the result)."""
    _need_cuda(x)
    dims = sorted(int(d) for d in dims)
    kept = [d for d in range(x.dim()) if d not in dims]
    out_shape = [x.shape[d] for d in kept]
    if not dims:
        return x
    x = _contig(x)
    if dims == list(range(dims[0], dims[-1] + 1)):
        outer, red, inner = _prod(x.shape[:dims[0]]), _prod(x.shape[dims[0]:dims[-1] + 1]), _prod(x.shape[dims[-1] + 1:])
    else:
        x = _permute(x, kept + dims)
        outer, red, inner = _prod(out_shape), _prod(x.shape[len(kept):]), 1
    y = torch.empty(out_shape, dtype=x.dtype, device=x.device)
    if y.numel():
        if red == 0:
            raise ValueError("reduce over an empty dimension")
        if inner > 1 and outer > 65535:
            raise ValueError("reduce: more than 65535 leading slices")
        nbytes = N.lib().emi_reduce_workspace_bytes(outer, red, inner, _code(x))
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device) if nbytes else None
        N.check(N.lib().emi_reduce(_stream(), REDUCE[kind], _p(x), _p(y), _p(ws), nbytes, outer, red, inner, _code(x)))
    return y


def _gemm_into(a, b, trans_a, trans_b, out):
    M, K = (a.shape[1], a.shape[0]) if trans_a else a.shape
    Nn = b.shape[0] if trans_b else b.shape[1]
    nbytes = N.lib().emi_gemm_workspace_bytes(M, Nn, K, int(trans_a), int(trans_b), _code(a))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=a.device) if nbytes else None
    N.check(N.lib().emi_gemm_ws(_stream(), _p(a), _p(b), None, _p(out), _p(ws), nbytes, M, Nn, K, a.shape[1], b.shape[1],
                                0, Nn, int(trans_a), int(trans_b), _code(a)))


def _dot_general(a, b, ba, bb, ca, cb):
    """stablehlo.dot_general: result dims = batch, free dims of a, free dims of b."""
    _need_cuda(a, b)
    if a.dtype != b.dtype:
        raise TypeError("dot_general: mixed dtypes %s and %s" % (a.dtype, b.dtype))
    ba, bb, ca, cb = list(ba), list(bb), list(ca), list(cb)
    fa = [d for d in range(a.dim()) if d not in ba and d not in ca]
    fb = [d for d in range(b.dim()) if d not in bb and d not in cb]
    if [a.shape[d] for d in ba] != [b.shape[d] for d in bb] or [a.shape[d] for d in ca] != [b.shape[d] for d in cb]:
        raise ValueError("dot_general: batch / contracting sizes differ: %s vs %s" % (tuple(a.shape), tuple(b.shape)))
    Bn, M, K, Nn = _prod(a.shape[d] for d in ba), _prod(a.shape[d] for d in fa), _prod(a.shape[d] for d in ca), \
        _prod(b.shape[d] for d in fb)
    out_shape = [a.shape[d] for d in ba] + [a.shape[d] for d in fa] + [b.shape[d] for d in fb]
    out = torch.empty(out_shape, dtype=a.dtype, device=a.device)
    if out.numel() == 0:
        return out
    if K == 0:
        return out.zero_()
    a, b = _contig(a), _contig(b)
    ident_a, ident_b = list(range(a.dim())), list(range(b.dim()))
    if ba + fa + ca == ident_a:
        ta = False
    elif ba + ca + fa == ident_a:
        ta = True
    else:
        a, ta = _permute(a, ba + fa + ca), False
    if bb + fb + cb == ident_b:
        tb = True                       # [batch, N, K]: both operands k-contiguous
    elif bb + cb + fb == ident_b:
        tb = False
    else:
        b, tb = _permute(b, bb + fb + cb), True
    a3 = a.reshape(Bn, K, M) if ta else a.reshape(Bn, M, K)
    b3 = b.reshape(Bn, Nn, K) if tb else b.reshape(Bn, K, Nn)
    o3 = out.reshape(Bn, M, Nn)
    if Bn >= 8 and M * Nn * K <= 256:
        # many tiny products (the 2x2 rotations of test/llama.py:161-168 are 144 of them): one
        # broadcast of each operand to [batch, M, N, K], one multiply, one sum over K
        box = [Bn, M, Nn, K]
        sa = (a3.stride(0), a3.stride(2), 0, a3.stride(1)) if ta else (a3.stride(0), a3.stride(1), 0, a3.stride(2))
        sb = (b3.stride(0), 0, b3.stride(1), b3.stride(2)) if tb else (b3.stride(0), 0, b3.stride(2), b3.stride(1))
        a4 = torch.empty(box, dtype=a.dtype, device=a.device)
        b4 = torch.empty(box, dtype=a.dtype, device=a.device)
        _copy_box(a3, box, sa, 0, a4, _contiguous_strides(box), 0)
        _copy_box(b3, box, sb, 0, b4, _contiguous_strides(box), 0)
        return _reduce("add", _bin("multiply", a4, b4), [3]).reshape(out_shape)
    for i in range(Bn):
        if Nn == 1 and M > 1:
            # matrix-vector product (`w @ x`, test/llama.py:149-157): as a one-row product the
            # weight-streaming kernels apply; [M, 1] and [1, M] are the same memory
            _gemm_into(b3[i].reshape(1, K), a3[i], False, not ta, o3[i].reshape(1, M))
        else:
            _gemm_into(a3[i], b3[i], ta, tb, o3[i])
    return out


def _sum_to_operand(c, x_shape, dims):
    """Adjoint of broadcast_in_dim: sum c over the result dims the operand does not have
    (or has with size 1), then view as the operand."""
    red = [d for d in range(c.dim()) if d not in dims]
    red += [d for i, d in enumerate(dims) if x_shape[i] == 1 and c.shape[d] != 1]
    kept = [d for d in range(c.dim()) if d not in red]
    r = _reduce("add", c, red)
    # kept dims are in result order; bring them into operand order
    order = [kept.index(d) for i, d in enumerate(dims) if d in kept]
    if order != sorted(order):
        r = _permute(r, order)
    return r.reshape(list(x_shape))


# ---------------------------------------------------------------------------
# operators (tape + tangents)
# ---------------------------------------------------------------------------

def _fit(g, like):
    """A cotangent for a rank-0 operand that the kernel broadcast: sum it back."""
    return _reduce("add", g, list(range(g.dim()))) if like.dim() == 0 and g.dim() > 0 else g


def binary(name, a, b):
    y = _bin(name, a, b)

    if name == "add":
        rule = lambda c, acc: (_accumulate(acc[0], _fit(c, a)), _accumulate(acc[1], _fit(c, b)))
        tangent = lambda ta, tb: tb if ta is None else ta if tb is None else _bin("add", ta, tb)
    elif name == "subtract":
        rule = lambda c, acc: (_accumulate(acc[0], _fit(c, a)), _accumulate(acc[1], _fit(_un("negate", c), b)))
        tangent = lambda ta, tb: _un("negate", tb) if ta is None else ta if tb is None else _bin("subtract", ta, tb)
    elif name == "multiply":
        rule = lambda c, acc: (_accumulate(acc[0], _fit(_bin("multiply", c, b), a)),
                               _accumulate(acc[1], _fit(_bin("multiply", c, a), b)))

        def tangent(ta, tb):
            pa = None if ta is None else _bin("multiply", ta, b)
            pb = None if tb is None else _bin("multiply", a, tb)
            return pb if pa is None else pa if pb is None else _bin("add", pa, pb)
    elif name == "divide":
        def rule(c, acc):
            q = _bin("divide", c, b)                                    # da = c / b, db = -(c / b) y
            return _accumulate(acc[0], _fit(q, a)), _accumulate(acc[1], _fit(_bin("nmul", q, y), b))

        def tangent(ta, tb):
            pa = None if ta is None else _bin("divide", ta, b)
            pb = None if tb is None else _bin("nmul", _bin("divide", tb, b), y)
            return pb if pa is None else pa if pb is None else _bin("add", pa, pb)
    elif name in ("maximum", "minimum"):
        def mask():
            return _bin("ge", a, b) if name == "maximum" else _bin("ge", b, a)       # ties go to a

        def rule(c, acc):
            ga = _bin("multiply", c, mask())
            return _accumulate(acc[0], _fit(ga, a)), _accumulate(acc[1], _fit(_bin("subtract", c, ga), b))

        def tangent(ta, tb):
            m = mask()
            za = _bin("multiply", m, ta) if ta is not None else None
            if tb is None:
                return za
            zb = _bin("subtract", tb, _bin("multiply", m, tb))
            return zb if za is None else _bin("add", za, zb)
    elif name == "power":
        rule = lambda c, acc: (_accumulate(acc[0], _fit(_bin("multiply", c, _bin("d_pow_a", a, b)), a)),
                               _accumulate(acc[1], _fit(_bin("multiply", c, _bin("d_pow_b", a, b)), b)))

        def tangent(ta, tb):
            pa = None if ta is None else _bin("multiply", ta, _bin("d_pow_a", a, b))
            pb = None if tb is None else _bin("multiply", tb, _bin("d_pow_b", a, b))
            return pb if pa is None else pa if pb is None else _bin("add", pa, pb)
    elif name == "atan2":
        # y = atan2(a, b): da = c b / (a^2 + b^2), db = -c a / (a^2 + b^2)  (Atan2 rule, HLODerivatives.td:972-978)
        def factors():
            den = _bin("add", _bin("multiply", a, a), _bin("multiply", b, b))
            return _bin("divide", b, den), _un("negate", _bin("divide", a, den))

        def rule(c, acc):
            fa, fb = factors()
            return (_accumulate(acc[0], _fit(_bin("multiply", c, fa), a)), _accumulate(acc[1], _fit(_bin("multiply", c, fb), b)))

        def tangent(ta, tb):
            fa, fb = factors()
            pa = None if ta is None else _bin("multiply", ta, fa)
            pb = None if tb is None else _bin("multiply", tb, fb)
            return pb if pa is None else pa if pb is None else _bin("add", pa, pb)
    else:
        raise NotImplementedError("no differentiation rule for stablehlo.%s" % name)

    Tape.record((a, b), y, rule)
    tans = _tan(a, b)
    if tans is not None and (tans[0] is not None or tans[1] is not None):
        ta, tb = tans
        t = _quiet(lambda: tangent(ta, tb))
        if t.shape != y.shape:                                          # tangent of a broadcast rank-0 operand alone
            t = _broadcast(t, list(y.shape), [])
        _set_tan(y, t)
    return y


_D_UNARY = {   # operator -> (derivative kernel, which saved value it reads)
    "exponential": ("multiply", "y"), "log": ("divide", "x"), "sqrt": ("d_sqrt", "y"), "rsqrt": ("d_rsqrt", "y"),
    "logistic": ("d_logistic", "y"), "tanh": ("d_tanh", "y"), "sine": ("d_sin", "x"), "cosine": ("d_cos", "x"),
    "abs": ("d_abs", "x"), "log_plus_one": ("d_log1p", "x"), "exponential_minus_one": ("d_expm1", "x"), "cbrt": ("d_cbrt", "y"),
}


def unary(name, x):
    y = _un(name, x)
    if name == "negate":
        d = lambda c: _un("negate", c)
    elif name in _D_UNARY:
        kern, which = _D_UNARY[name]
        d = lambda c: _bin(kern, c, y if which == "y" else x)
    else:
        raise NotImplementedError("no differentiation rule for stablehlo.%s" % name)
    Tape.record((x,), y, lambda c, acc: (_accumulate(acc[0], d(c)),))
    tans = _tan(x)
    if tans is not None and tans[0] is not None:
        _set_tan(y, _quiet(lambda: d(tans[0])))
    return y


def unary_copy(x):
    """A fresh contiguous, aligned copy of x (the identity as far as differentiation goes)."""
    y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    _copy_box(x, list(x.shape), list(x.stride()), 0, y, _contiguous_strides(x.shape), 0)
    Tape.record((x,), y, lambda c, acc: (_accumulate(acc[0], c),))
    tans = _tan(x)
    if tans is not None and tans[0] is not None:
        _set_tan(y, tans[0])
    return y


def convert(x, dtype):
    y = _convert(x, dtype)
    Tape.record((x,), y, lambda c, acc: (_accumulate(acc[0], _convert(c, x.dtype)),))
    tans = _tan(x)
    if tans is not None and tans[0] is not None:
        _set_tan(y, _quiet(lambda: _convert(tans[0], dtype)))
    return y


def broadcast_in_dim(x, shape, dims):
    dims = [int(d) for d in dims]
    y = _broadcast(x, shape, dims)
    Tape.record((x,), y, lambda c, acc: (_accumulate(acc[0], _sum_to_operand(c, tuple(x.shape), dims)),))
    tans = _tan(x)
    if tans is not None and tans[0] is not None:
        _set_tan(y, _quiet(lambda: _broadcast(tans[0], shape, dims)))
    return y


def reduce(kind, x, dims):
    dims = sorted(int(d) for d in dims)
    y = _reduce(kind, x, dims)
    kept = [d for d in range(x.dim()) if d not in dims]

    def back(c):
        return _broadcast(c, list(x.shape), kept)

    if kind == "add":
        rule = lambda c, acc: (_accumulate(acc[0], back(c)),)
        tangent = lambda t: _reduce("add", t, dims)
    elif kind == "maximum":
        # every element equal to the maximum receives the cotangent, undivided
        mask = lambda: _bin("eq", x, back(y))
        rule = lambda c, acc: (_accumulate(acc[0], _bin("multiply", mask(), back(c))),)

        def tangent(t):                                   # tangent of the first maximal element... of all, summed
            return _reduce("add", _bin("multiply", mask(), t), dims)
    else:
        raise NotImplementedError("reduce with a stablehlo.%s body" % kind)
    Tape.record((x,), y, rule)
    tans = _tan(x)
    if tans is not None and tans[0] is not None:
        _set_tan(y, _quiet(lambda: tangent(tans[0])))
    return y


def transpose(x, perm):
    perm = [int(p) for p in perm]
    y = _permute(x, perm)
    inv = [perm.index(i) for i in range(len(perm))]
    Tape.record((x,), y, lambda c, acc: (_accumulate(acc[0], _permute(c, inv)),))
    tans = _tan(x)
    if tans is not None and tans[0] is not None:
        _set_tan(y, _quiet(lambda: _permute(tans[0], perm)))
    return y


def dot_general(a, b, batch_a=(), batch_b=(), contract_a=(), contract_b=()):
    ba, bb, ca, cb = [int(d) for d in batch_a], [int(d) for d in batch_b], [int(d) for d in contract_a], \
        [int(d) for d in contract_b]
    y = _dot_general(a, b, ba, bb, ca, cb)
    fa = [d for d in range(a.dim()) if d not in ba and d not in ca]
    fb = [d for d in range(b.dim()) if d not in bb and d not in cb]
    nb, nfa, nfb = len(ba), len(fa), len(fb)

    def grad_a(c, other=None):
        # contract c with b over b's free dims: result dims = batch, free(a), contracting dims in b's order
        other = b if other is None else other
        g = _dot_general(c, other, list(range(nb)), bb, list(range(nb + nfa, nb + nfa + nfb)), fb)
        b_rest = sorted(cb)                                   # b's dims left over, in b's order
        src = {}                                              # a dim -> position in g
        for i, d in enumerate(ba):
            src[d] = i
        for i, d in enumerate(fa):
            src[d] = nb + i
        for i, d in enumerate(b_rest):
            src[ca[cb.index(d)]] = nb + nfa + i
        perm = [src[d] for d in range(a.dim())]
        return g if perm == list(range(len(perm))) else _permute(g, perm)

    def grad_b(c, other=None):
        other = a if other is None else other
        g = _dot_general(c, other, list(range(nb)), ba, list(range(nb, nb + nfa)), fa)   # batch, free(b), rest of a
        a_rest = sorted(ca)
        src = {}
        for i, d in enumerate(bb):
            src[d] = i
        for i, d in enumerate(fb):
            src[d] = nb + i
        for i, d in enumerate(a_rest):
            src[cb[ca.index(d)]] = nb + nfb + i
        perm = [src[d] for d in range(b.dim())]
        return g if perm == list(range(len(perm))) else _permute(g, perm)

    # x.dot(x) (test/llama.py:8) passes one tensor twice: the tape sums the two cotangents
    Tape.record((a, b), y, lambda c, acc: (_accumulate(acc[0], grad_a(c)), _accumulate(acc[1], grad_b(c))))
    tans = _tan(a, b)
    if tans is not None and (tans[0] is not None or tans[1] is not None):
        ta, tb = tans

        def tangent():
            pa = None if ta is None else _dot_general(ta, b, ba, bb, ca, cb)
            pb = None if tb is None else _dot_general(a, tb, ba, bb, ca, cb)
            return pb if pa is None else pa if pb is None else _bin("add", pa, pb)

        _set_tan(y, _quiet(tangent))
    return y


def slice_(x, start, limit, stride=None):
    start, limit = [int(s) for s in start], [int(l) for l in limit]
    stride = [1] * len(start) if stride is None else [int(s) for s in stride]
    y = _slice(x, start, limit, stride)
    if y is x:
        return x

    # only a leaf's cotangent is never handed on to another rule, so only there may a buffer be
    # updated in place
    leaf = Tape._active is not None and id(x) not in Tape._active.produced

    def rule(c, acc):
        g = acc[0]
        if leaf and g is not None and getattr(g, "_emi_slice_owned", False) and all(st == 1 for st in stride):
            box = _slice(g, start, limit, stride)
            if box.is_contiguous() and box.data_ptr() % 16 == 0:
                # the accumulated cotangent is a buffer an earlier slice rule zero-filled and nobody
                # else holds (the per-layer slices of one stacked weight): add the block in place
                c = _contig(c)
                N.check(N.lib().emi_add(_stream(), _p(box), _p(c), _p(box), c.numel(), _code(c)))
                return (g,)
        fresh = _scatter_box(c, list(x.shape), start, stride)
        if g is None:
            fresh._emi_slice_owned = leaf
            return (fresh,)
        return (_accumulate(g, fresh),)

    Tape.record((x,), y, rule)
    tans = _tan(x)
    if tans is not None and tans[0] is not None:
        _set_tan(y, _quiet(lambda: _slice(tans[0], start, limit, stride)))
    return y


def concatenate(xs, dim):
    xs, dim = list(xs), int(dim)
    y = _concat(xs, dim)

    def rule(c, acc):
        out, at = [], 0
        for i, x in enumerate(xs):
            lo = [0] * c.dim()
            hi = list(c.shape)
            lo[dim], hi[dim] = at, at + x.shape[dim]
            at += x.shape[dim]
            out.append(_accumulate(acc[i], _contig(_slice(c, lo, hi, [1] * c.dim()))))
        return out

    Tape.record(tuple(xs), y, rule)
    tans = _tan(*xs)
    if tans is not None and any(t is not None for t in tans):
        parts = [torch.zeros_like(x) if t is None else t for x, t in zip(xs, tans)]
        _set_tan(y, _quiet(lambda: _concat(parts, dim)))
    return y


def pad(x, low, high, interior, shape):
    """stablehlo.pad with a zero padding value: x placed at offset `low` with `interior` zeros
    between neighbours (Pad is the adjoint of Slice, StableHLOAutoDiffOpInterfaceImpl.cpp:1586-1620,
    and the other way round)."""
    low, high, interior = [int(v) for v in low], [int(v) for v in high], [int(v) for v in interior]
    if any(v < 0 for v in low + high + interior):
        raise NotImplementedError("stablehlo.pad with negative padding")
    stride = [i + 1 for i in interior]
    want = [l + h + (n - 1) * st + 1 if n else l + h for l, h, n, st in zip(low, high, x.shape, stride)]
    if list(shape) != want:
        raise ValueError("pad: result shape %s, operands give %s" % (list(shape), want))
    y = _scatter_box(x, list(shape), low, stride)
    limit = [l + (n - 1) * st + 1 for l, n, st in zip(low, x.shape, stride)]
    Tape.record((x,), y, lambda c, acc: (_accumulate(acc[0], _contig(_slice(c, low, limit, stride))),))
    tans = _tan(x)
    if tans is not None and tans[0] is not None:
        _set_tan(y, _quiet(lambda: _scatter_box(tans[0], list(shape), low, stride)))
    return y


def compare(direction, a, b):
    """stablehlo.compare: no derivative (the result is an i1 tensor)."""
    return _compare(direction, a, b)


def select(m, a, b):
    """stablehlo.select (Select rule HLODerivatives.td:1297): the cotangent goes to the chosen
    side, zero to the other."""
    y = _select(m, a, b)
    zero = lambda like: torch.zeros((), dtype=like.dtype, device=like.device)

    def rule(c, acc):
        ga = _select(m, c, zero(c))
        gb = _select(m, zero(c), c)
        return None, _accumulate(acc[1], _fit(ga, a)), _accumulate(acc[2], _fit(gb, b))

    Tape.record((m, a, b), y, rule)
    tans = _tan(a, b)
    if tans is not None and (tans[0] is not None or tans[1] is not None):
        ta = zero(y) if tans[0] is None else tans[0]
        tb = zero(y) if tans[1] is None else tans[1]
        t = _quiet(lambda: _select(m, ta, tb))
        if t.shape != y.shape:
            t = _broadcast(t, list(y.shape), [])
        _set_tan(y, t)
    return y
