"""Rewrites on parsed StableHLO functions: lowering of matched clusters to typed-FFI custom calls,
and symbolic reverse mode.

`reverse_function` is the counterpart, for the operators of the llama path, of the reference's
`enzyme-wrap{... mode=ReverseModeCombined}` pass (src/enzyme_ad/jax/primitives.py:1385-1419): from a
function f(args) -> results it builds f_rev(args, cotangents of results) -> cotangents of args,
recomputing the forward values and then walking the operators backwards with the reference's
rules (Implementations/HLODerivatives.td: Add :964, Div :1133, DotGeneral :1166, Exp :1182,
Mul :1221, Neg :1228, Reshape :1271, Rsqrt :1283, Convert :1290, Sub :1312, Sqrt :1320,
Transpose :1334; StableHLOAutoDiffOpInterfaceImpl.cpp: BroadcastInDim :1474, Slice :1586,
Reduce :1833, Concatenate :2015).  Clusters that were matched to fused kernels differentiate
into the matching adjoint custom calls (`emi_rmsnorm_bwd`, `emi_swiglu_bwd`, `emi_rope` with
`inverse`, `emi_attn_step_bwd`), so the printed reverse module is what an XLA client with this
library's handlers would compile for `jax.vjp`.
"""
import re

import numpy as np

from .stablehlo import Func, Op, TensorType, _drop_dead, check_gather

FLOAT = ("f32", "bf16", "f16", "f64")


def _types_of(func):
    types = {a: t for a, t in func.args}
    for op in func.ops:
        for r, t in zip(op.results, op.types):
            types[r] = t
    return types


class _Builder:
    def __init__(self, func, prefix):
        self.ops, self.types, self.prefix = [], _types_of(func), prefix
        used = [int(m.group(1)) for n in self.types for m in [re.fullmatch(r"%%%s(\d+)(?:#\d+)?" % prefix, n)] if m]
        self.n = max(used) + 1 if used else 0

    def new(self, ty):
        name = "%%%s%d" % (self.prefix, self.n)
        self.n += 1
        self.types[name] = ty
        return name

    def emit(self, name, operands, attrs, ty):
        r = self.new(ty)
        self.ops.append(Op(name, [r], list(operands), attrs, [ty]))
        return r

    def const(self, value, ty):
        return self.emit("constant", [], {"value": np.full(ty.shape, value, dtype=np.float32)}, ty)

    def reshape(self, v, shape):
        ty = TensorType(shape, self.types[v].dtype)
        return v if self.types[v].shape == ty.shape else self.emit("reshape", [v], {}, ty)

    def _gemm_workspace(self, target, operands, config):
        """Bytes of scratch the GEMM targets use for split-K partials (0 for most shapes): declared as an extra i8 result,
        which their handlers take when it is there."""
        from . import _native as N
        n = int(config.get("count", 1)) if target == "emi_gemm_grouped" else 1
        ta, tb = bool(config.get("trans_a", False)), bool(config.get("trans_b", False))
        at, bt = self.types[operands[0]], self.types[operands[n]]
        if len(at.shape) != 2 or len(bt.shape) != 2 or at.dtype not in ("f32", "bf16"):
            return 0
        M, K = (at.shape[1], at.shape[0]) if ta else at.shape
        Nn = bt.shape[0] if tb else bt.shape[1]
        code = 16 if at.dtype == "bf16" else 11
        if target == "emi_gemm":
            return int(N.lib().emi_gemm_workspace_bytes(M, Nn, K, int(ta), int(tb), code))
        return int(N.lib().emi_gemm_grouped_workspace_bytes(n, M, Nn, K, int(ta), int(tb), int(bool(config.get("sum", False))), code))

    def custom_call(self, target, operands, config, tys):
        tys = list(tys)
        nres = len(tys)
        if target in ("emi_gemm", "emi_gemm_grouped"):
            nbytes = self._gemm_workspace(target, operands, config)
            if nbytes:
                tys.append(TensorType((nbytes,), "i8"))
        return self._call(target, operands, config, tys)[:nres]

    def _call(self, target, operands, config, tys):
        base = self.new(tys[0])
        names = [base] if len(tys) == 1 else ["%s#%d" % (base, i) for i in range(len(tys))]
        for n, t in zip(names, tys):
            self.types[n] = t
        self.ops.append(Op("custom_call", names, list(operands), {"target": target, "config": dict(config)}, list(tys)))
        return names

    def binary(self, name, a, b):
        return self.emit(name, [a, b], {}, self.types[a])

    def compare(self, direction, a, b):
        return self.emit("compare", [a, b], {"direction": direction}, TensorType(self.types[a].shape, "i1"))

    def unary(self, name, a):
        return self.emit(name, [a], {}, self.types[a])


def _step_workspace(heads, rows, head_dim):
    return heads * ((rows + 511) // 512) * (head_dim + 2) * 4          # emi_attn_step_workspace_bytes for one sequence


def lower_fused(func, blocks=True):
    """A copy of `func` with the matcher's fused operators written as custom calls to this
    library's FFI targets (api_version 4; scalars in backend_config), wrapped in the reshapes
    that bring the operands to the handlers' layouts.  blocks: the two sub-blocks of a decoder layer are written
    with the targets that apply RoPE and the SwiGLU in GEMM epilogues (`emi_gemm_rope`, `emi_gemm_swiglu_fwd`)."""
    if not any(op.name.startswith("emi.") for op in func.ops):
        return func
    from .stablehlo import _fuse_blocks
    b = _Builder(func, "emi")
    T = b.types
    for op in (_fuse_blocks(func.ops, func) if blocks else func.ops):
        n = op.name
        ty = op.types[0] if op.types else None
        if n == "emi.rmsnorm":
            x, w = op.operands
            D = ty.shape[-1]
            y2, = b.custom_call("emi_rmsnorm_fwd", [b.reshape(x, (1, D)), w], {"eps": op.attrs["eps"]}, [TensorType((1, D), ty.dtype)])
            b.ops.append(Op("reshape", op.results, [y2], {}, op.types))
        elif n == "emi.swiglu":
            b.ops.append(Op("custom_call", op.results, list(op.operands), {"target": "emi_swiglu_fwd", "config": {}}, op.types))
        elif n == "emi.rope":
            P = ty.shape[0] // 2
            tab = b.emit("constant", [], {"value": np.asarray(op.attrs["table"], dtype=np.float32).reshape(1, P, 2)},
                         TensorType((1, P, 2), "f32"))
            x4 = b.reshape(op.operands[0], (1, 1, 1, 2 * P))
            y4, = b.custom_call("emi_rope", [x4, tab], {"inverse": False}, [T[x4]])
            b.ops.append(Op("reshape", op.results, [y4], {}, op.types))
        elif n == "emi.linear":
            x, w = op.operands[:2]
            K, Nn = T[x].shape[-1], T[w].shape[0]
            rows = int(np.prod(T[x].shape[:-1])) if len(T[x].shape) > 1 else 1
            operands = [b.reshape(x, (rows, K)), w] + [b.reshape(r_, (rows, Nn)) for r_ in op.operands[2:]]
            c2, = b.custom_call("emi_gemm", operands, {"trans_a": False, "trans_b": True}, [TensorType((rows, Nn), ty.dtype)])
            b.ops.append(Op("reshape", op.results, [c2], {}, op.types))
        elif n == "emi.linear_group":
            x, ws = op.operands[0], list(op.operands[1:])
            K, Nn = T[x].shape[-1], T[ws[0]].shape[0]
            rows = int(np.prod(T[x].shape[:-1])) if len(T[x].shape) > 1 else 1
            x2 = b.reshape(x, (rows, K))
            outs = b.custom_call("emi_gemm_grouped", [x2] * len(ws) + ws, {"count": len(ws), "sum": False, "trans_a": False, "trans_b": True},
                                 [TensorType((rows, Nn), ty.dtype)] * len(ws))
            for r_, c2, t_ in zip(op.results, outs, op.types):
                b.ops.append(Op("reshape", [r_], [c2], {}, [t_]))
        elif n == "emi.ffn":
            # a = x w1^T ; (b, g) = (x w3^T, swiglu(a, b)) in one launch ; y = g w2^T [+ r]   (test/llama.py:224-233)
            x, w1, w3, w2 = op.operands[:4]
            K, Hn = T[x].shape[-1], T[w1].shape[0]
            rows = int(np.prod(T[x].shape[:-1])) if len(T[x].shape) > 1 else 1
            x2 = b.reshape(x, (rows, K))
            hty = TensorType((rows, Hn), ty.dtype)
            a, = b.custom_call("emi_gemm", [x2, w1], {"trans_a": False, "trans_b": True}, [hty])
            _, g = b.custom_call("emi_gemm_swiglu_fwd", [x2, w3, a], {}, [hty, hty])
            Nn = T[w2].shape[0]
            y2, = b.custom_call("emi_gemm", [g, w2] + [b.reshape(r_, (rows, Nn)) for r_ in op.operands[4:]],
                                {"trans_a": False, "trans_b": True}, [TensorType((rows, Nn), ty.dtype)])
            b.ops.append(Op("reshape", op.results, [y2], {}, op.types))
        elif n == "emi.attention_block":
            # q, k = rope(x wq^T), rope(x wk^T) stored rotated by the projections ; v = x wv^T ; attention   (:149-209)
            x, wq, wk, wv = op.operands
            B_, S_, K = T[x].shape
            h = op.attrs["heads"]
            D_ = T[wq].shape[0]
            x2 = b.reshape(x, (B_ * S_, K))
            tab = b.emit("constant", [], {"value": np.asarray(op.attrs["table"], dtype=np.float32)},
                         TensorType(op.attrs["table"].shape, "f32"))
            pty = TensorType((B_ * S_, D_), ty.dtype)
            q2, = b.custom_call("emi_gemm_rope", [x2, wq, tab], {}, [pty])
            k2, = b.custom_call("emi_gemm_rope", [x2, wk, tab], {}, [pty])
            v2, = b.custom_call("emi_gemm", [x2, wv], {"trans_a": False, "trans_b": True}, [pty])
            q4, k4, v4 = (b.reshape(o_, (B_, S_, h, D_ // h)) for o_ in (q2, k2, v2))
            o4, _ = b.custom_call("emi_attn_fwd", [q4, k4, v4], {"scale": op.attrs["scale"], "causal": bool(op.attrs["causal"]), "bshd": True},
                                  [T[q4], TensorType((B_, h, S_), "f32")])
            b.ops.append(Op("reshape", op.results, [o4], {}, op.types))
        elif n == "emi.rmsnorm_rows":
            b.ops.append(Op("custom_call", op.results, list(op.operands), {"target": "emi_rmsnorm_fwd", "config": {"eps": op.attrs["eps"]}},
                            op.types))
        elif n == "emi.rope_rows":
            B_, S_, D_ = ty.shape
            h = op.attrs["heads"]
            tab = b.emit("constant", [], {"value": np.asarray(op.attrs["table"], dtype=np.float32)},
                         TensorType(op.attrs["table"].shape, "f32"))
            x4 = b.reshape(op.operands[0], (B_, S_, h, D_ // h))
            y4, = b.custom_call("emi_rope", [x4, tab], {"inverse": False}, [T[x4]])
            b.ops.append(Op("reshape", op.results, [y4], {}, op.types))
        elif n == "emi.attention":
            B_, S_, D_ = ty.shape
            h = op.attrs["heads"]
            q4, k4, v4 = (b.reshape(o_, (B_, S_, h, D_ // h)) for o_ in op.operands)
            o4, _ = b.custom_call("emi_attn_fwd", [q4, k4, v4], {"scale": op.attrs["scale"], "causal": bool(op.attrs["causal"]), "bshd": True},
                                  [T[q4], TensorType((B_, h, S_), "f32")])
            b.ops.append(Op("reshape", op.results, [o4], {}, op.types))
        elif n == "emi.cross_entropy":
            z, t = op.operands
            V = T[z].shape[-1]
            rows = int(np.prod(T[z].shape[:-1])) if len(T[z].shape) > 1 else 1
            loss, _ = b.custom_call("emi_cross_entropy_fwd", [b.reshape(z, (rows, V)), b.reshape(t, (rows,))], {},
                                    [TensorType((rows,), "f32"), TensorType((rows,), "f32")])
            if op.attrs.get("negated"):
                loss = b.emit("negate", [loss], {}, T[loss])
            if ty.dtype != "f32":
                loss = b.emit("convert", [loss], {}, TensorType((rows,), ty.dtype))
            b.ops.append(Op("reshape", op.results, [loss], {}, op.types))
        elif n in ("emi.softmax_dot", "emi.attention_step"):
            q, k, v = op.operands
            h = op.attrs.get("heads", 1)
            d, S = T[q].shape[0] // h, T[k].shape[0]
            outs = [TensorType((1, h, d), ty.dtype), TensorType((1, h), "f32"), TensorType((_step_workspace(h, S, d),), "i8")]
            o3, _, _ = b.custom_call("emi_attn_step_fwd", [b.reshape(q, (1, h, d)), b.reshape(k, (1, S, h, d)), b.reshape(v, (1, S, h, d))],
                                     {"scale": op.attrs["scale"]}, outs)
            b.ops.append(Op("reshape", op.results, [o3], {}, op.types))
        else:
            b.ops.append(op)
    return Func(func.name, func.args, func.result_types, b.ops)


def inline_calls(funcs, fn="main"):
    """`fn` with every `call` replaced by the callee's operators (renamed), recursively."""
    counter = [0]

    def inline(f, depth=0):
        if depth > 32:
            raise RecursionError("call depth over 32 (recursive functions are not supported)")
        out = []
        for op in f.ops:
            if op.name != "call":
                out.append(op)
                continue
            callee = inline(funcs[op.attrs["callee"]], depth + 1)
            counter[0] += 1
            tag = "%%c%d_" % counter[0]
            ren = {a: o for (a, _), o in zip(callee.args, op.operands)}
            for cop in callee.ops:
                if cop.name == "return":
                    for r, o, t in zip(op.results, cop.operands, op.types):
                        out.append(Op("reshape", [r], [ren.get(o, o)], {}, [t]))        # identity: binds the call's result names
                    continue
                res = [tag + r[1:] for r in cop.results]
                ren.update(zip(cop.results, res))
                out.append(Op(cop.name, res, [ren.get(o, o) for o in cop.operands], cop.attrs, cop.types))
        return Func(f.name, f.args, f.result_types, out)

    return inline(funcs[fn])


def reverse_function(func, name=None, arg_active=None, ret_active=None):
    """f_rev(args..., one cotangent per active result) -> one cotangent per active argument
    (default: every floating-point argument and result; `enzyme_const` entries of the
    reference's activity lists are the inactive ones).  `func` must be call-free (see
    `inline_calls`); fused operators are lowered first."""
    func = lower_fused(func)
    b = _Builder(func, "r")
    T = b.types
    # what the joint rules of the fused targets look at: who produced a value, how often it is used, and which
    # cotangents already are those of the vector before its rotation
    b.producer = {r_: op_ for op_ in func.ops for r_ in op_.results}
    b.uses = {}
    for op_ in func.ops:
        for o_ in op_.operands:
            b.uses[o_] = b.uses.get(o_, 0) + 1
    b.unrotated = set()
    ret = [op for op in func.ops if op.name == "return"]
    if len(ret) != 1:
        raise ValueError("reverse mode needs exactly one return")
    results = list(ret[0].operands)
    primal = [op for op in func.ops if op.name != "return"]
    b.ops = list(primal)
    ct_args = []
    ct = {}

    def accum(v, g):
        if T[v].dtype not in FLOAT:
            return
        if T[g] != T[v]:
            raise RuntimeError("cotangent %r for a value of type %r" % (T[g], T[v]))
        ct[v] = g if v not in ct else b.binary("add", ct[v], g)

    if ret_active is None:
        ret_active = [T[r].dtype in FLOAT for r in results]
    if arg_active is None:
        arg_active = [t.dtype in FLOAT for _, t in func.args]
    if len(ret_active) != len(results) or len(arg_active) != len(func.args):
        raise ValueError("activity lists do not match the function: %d results, %d arguments" % (len(results), len(func.args)))
    for i, r in enumerate(results):
        if not ret_active[i]:
            continue
        a = "%%ct%d" % i
        T[a] = T[r]
        ct_args.append((a, T[r]))
        accum(r, a)

    def splat_like(v, value):
        return b.const(value, T[v])

    for op in reversed(primal):
        cs = [ct.pop(r, None) for r in op.results]
        if all(c is None for c in cs):
            continue
        c = cs[0]
        n, xs = op.name, op.operands
        r = op.results[0]
        if n == "constant":
            continue
        if n == "add":
            accum(xs[0], c)
            accum(xs[1], c)
        elif n == "subtract":
            accum(xs[0], c)
            accum(xs[1], b.unary("negate", c))
        elif n == "multiply":
            accum(xs[0], b.binary("multiply", c, xs[1]))
            accum(xs[1], b.binary("multiply", c, xs[0]))
        elif n == "divide":
            q = b.binary("divide", c, xs[1])
            accum(xs[0], q)
            accum(xs[1], b.unary("negate", b.binary("multiply", q, r)))
        elif n == "negate":
            accum(xs[0], b.unary("negate", c))
        elif n == "exponential":
            accum(xs[0], b.binary("multiply", c, r))
        elif n == "log":
            accum(xs[0], b.binary("divide", c, xs[0]))
        elif n == "sqrt":
            # select(x == 0, 0, c / (2 sqrt(x)))  (Sqrt rule :1320 with its zero guard)
            g = b.binary("divide", c, b.binary("multiply", splat_like(r, 2.0), r))
            accum(xs[0], b.emit("select", [b.compare("EQ", xs[0], splat_like(r, 0.0)), splat_like(r, 0.0), g], {}, T[r]))
        elif n in ("maximum", "minimum"):
            # ties go to the first operand (Max rule :1205, maximum.mlir:25-34)
            m = b.compare("GE" if n == "maximum" else "LE", xs[0], xs[1])
            z = splat_like(r, 0.0)
            accum(xs[0], b.emit("select", [m, c, z], {}, T[r]))
            accum(xs[1], b.emit("select", [m, z, c], {}, T[r]))
        elif n == "power":
            # c y x^(y-1) and c x^y log x (Pow rule :1237-1242)
            ym1 = b.binary("subtract", xs[1], splat_like(r, 1.0))
            accum(xs[0], b.binary("multiply", c, b.binary("multiply", xs[1], b.binary("power", xs[0], ym1))))
            accum(xs[1], b.binary("multiply", c, b.binary("multiply", r, b.unary("log", xs[0]))))
        elif n == "atan2":
            # c x / (x^2 + y^2) and -c y / (x^2 + y^2) for atan2(y, x)  (Atan2 rule :972-978)
            den = b.binary("add", b.binary("multiply", xs[1], xs[1]), b.binary("multiply", xs[0], xs[0]))
            accum(xs[0], b.binary("multiply", c, b.binary("divide", xs[1], den)))
            accum(xs[1], b.binary("multiply", c, b.binary("divide", b.unary("negate", xs[0]), den)))
        elif n == "compare":
            continue
        elif n == "select":
            z = splat_like(r, 0.0)
            accum(xs[1], b.emit("select", [xs[0], c, z], {}, T[r]))
            accum(xs[2], b.emit("select", [xs[0], z, c], {}, T[r]))
        elif n == "rsqrt":
            cube = b.binary("multiply", b.binary("multiply", r, r), r)
            accum(xs[0], b.binary("multiply", b.binary("multiply", splat_like(r, -0.5), c), cube))
        elif n == "logistic":
            accum(xs[0], b.binary("multiply", b.binary("multiply", c, r), b.binary("subtract", splat_like(r, 1.0), r)))
        elif n == "tanh":
            accum(xs[0], b.binary("multiply", c, b.binary("subtract", splat_like(r, 1.0), b.binary("multiply", r, r))))
        elif n == "abs":
            # select(x >= 0, c, -c)  (Abs rule :1244, abs.mlir:21-27)
            accum(xs[0], b.emit("select", [b.compare("GE", xs[0], splat_like(r, 0.0)), c, b.unary("negate", c)], {}, T[r]))
        elif n == "log_plus_one":
            accum(xs[0], b.binary("divide", c, b.binary("add", xs[0], splat_like(r, 1.0))))          # Log1p rule :1201
        elif n == "exponential_minus_one":
            accum(xs[0], b.binary("multiply", c, b.unary("exponential", xs[0])))                     # Expm1 rule :1184
        elif n == "cbrt":
            # c / (3 cbrt(x)^2), finite for negative x (Cbrt rule :1085, cbrt.mlir:19-26)
            accum(xs[0], b.binary("divide", c, b.binary("multiply", splat_like(r, 3.0), b.binary("multiply", r, r))))
        elif n == "sine":
            accum(xs[0], b.binary("multiply", c, b.unary("cosine", xs[0])))
        elif n == "cosine":
            accum(xs[0], b.unary("negate", b.binary("multiply", c, b.unary("sine", xs[0]))))
        elif n == "convert":
            accum(xs[0], c if T[xs[0]].dtype == T[c].dtype else b.emit("convert", [c], {}, T[xs[0]]))
        elif n == "reshape":
            g = b.reshape(c, T[xs[0]].shape)
            if c in b.unrotated:
                b.unrotated.add(g)
            accum(xs[0], g)
        elif n == "transpose":
            perm = list(op.attrs["perm"])
            accum(xs[0], b.emit("transpose", [c], {"perm": [perm.index(i) for i in range(len(perm))]}, T[xs[0]]))
        elif n == "broadcast_in_dim":
            dims, xt, ot = list(op.attrs["dims"]), T[xs[0]], T[r]
            red = [d for d in range(len(ot.shape)) if d not in dims] + \
                  [d for i, d in enumerate(dims) if xt.shape[i] == 1 and ot.shape[d] != 1]
            g = c
            if red:
                kept = [ot.shape[d] for d in range(len(ot.shape)) if d not in red]
                zero = b.const(0.0, TensorType((), ot.dtype))
                g = b.emit("reduce", [c, zero], {"dims": sorted(red), "body": "add"}, TensorType(kept, ot.dtype))
                order = [d for d in dims if d not in red]
                if order != sorted(order):
                    rank = sorted(order)
                    perm = [rank.index(d) for d in order]
                    g = b.emit("transpose", [g], {"perm": perm}, TensorType([kept[p] for p in perm], ot.dtype))
            accum(xs[0], b.reshape(g, xt.shape))
        elif n == "reduce":
            xt = T[xs[0]]
            kept = [d for d in range(len(xt.shape)) if d not in op.attrs["dims"]]
            back = b.emit("broadcast_in_dim", [c], {"dims": kept}, xt)
            if op.attrs["body"] == "add":
                accum(xs[0], back)
            elif op.attrs["body"] == "maximum":
                # every element equal to the maximum gets the cotangent, undivided
                # (StableHLOAutoDiffOpInterfaceImpl.cpp:1881-1916)
                m = b.compare("EQ", xs[0], b.emit("broadcast_in_dim", [r], {"dims": kept}, xt))
                accum(xs[0], b.emit("select", [m, back, b.const(0.0, xt)], {}, xt))
            else:
                raise NotImplementedError("symbolic reverse mode of reduce with a %s body" % op.attrs["body"])
        elif n == "dot_general":
            _reverse_dot_general(b, op, c, accum)
        elif n == "slice":
            xt, a = T[xs[0]], op.attrs
            shape = T[r].shape
            high = [xt.shape[i] - (a["start"][i] + (shape[i] - 1) * a["stride"][i] + 1) if shape[i] else xt.shape[i] - a["start"][i]
                    for i in range(len(shape))]
            zero = b.const(0.0, TensorType((), xt.dtype))
            accum(xs[0], b.emit("pad", [c, zero], {"low": list(a["start"]), "high": high, "interior": [s - 1 for s in a["stride"]]}, xt))
        elif n == "pad":
            a, xt = op.attrs, T[xs[0]]
            stride = [i + 1 for i in a["interior"]]
            limit = [l + (m - 1) * st + 1 for l, m, st in zip(a["low"], xt.shape, stride)]
            accum(xs[0], b.emit("slice", [c], {"start": list(a["low"]), "limit": limit, "stride": stride}, xt))
        elif n == "concatenate":
            dim, at = op.attrs["dim"], 0
            for x in xs:
                xt = T[x]
                start = [0] * len(xt.shape)
                limit = list(T[r].shape)
                start[dim], limit[dim] = at, at + xt.shape[dim]
                at += xt.shape[dim]
                accum(x, b.emit("slice", [c], {"start": start, "limit": limit, "stride": [1] * len(start)}, xt))
        elif n == "gather":
            # the adjoint of the row lookup table[indices] is a scatter-add of the cotangent rows into a zero table
            # (reference rule: HLODerivatives.td:1022-1046): the emi_embedding_bwd target; the indices are inactive
            check_gather(op.attrs, T[xs[0]], T[xs[1]], T[r])
            idx = b.emit("reshape", [xs[1]], {}, TensorType(T[xs[1]].shape[:-1], T[xs[1]].dtype))
            from . import _native as N
            tt = T[xs[0]]
            nbytes = int(N.lib().emi_embedding_bwd_workspace_bytes(tt.shape[0], tt.shape[1], 16 if tt.dtype == "bf16" else 11))
            if nbytes:         # bf16: the rows are summed in an fp32 table that the handler takes as an extra result
                dt_, _ = b.custom_call("emi_embedding_bwd", [idx, c], {}, [tt, TensorType((nbytes,), "i8")])
            else:
                dt_, = b.custom_call("emi_embedding_bwd", [idx, c], {}, [tt])
            accum(xs[0], dt_)
        elif n == "custom_call":
            _reverse_custom_call(b, op, cs, accum)
        elif n == "call":
            raise NotImplementedError("symbolic reverse mode needs a call-free function (inline_calls)")
        else:
            raise NotImplementedError("symbolic reverse mode of stablehlo.%s" % n)

    outs = []
    for (a, t), active in zip(func.args, arg_active):
        if not active:
            continue
        if t.dtype not in FLOAT:
            raise ValueError("argument %s of type %r cannot be active" % (a, t))
        outs.append(ct[a] if a in ct else b.const(0.0, t))
    outs = _group_adjoint_products(b, outs)
    b.ops.append(Op("return", [], outs, {}, []))
    rev = Func(name or func.name + "_rev", list(func.args) + ct_args, [T[o] for o in outs], b.ops)
    _drop_dead(rev)
    return rev


def _group_adjoint_products(b, outs):
    """The adjoint products of sibling projections as the tape issues them (ops._group_rule): the fan-in
    dX = dY_0 . W_0 + dY_1 . W_1 + ... of single products and adds becomes one summed emi_gemm_grouped (one rounding
    instead of one per product and add), and the weight gradients dW_i = dY_i^T . X that share X become one grouped
    call.  Works on the emitted list in place; returns the (renamed) results."""
    ops, T = b.ops, b.types
    uses = {}
    for op in ops:
        for o in op.operands:
            uses[o] = uses.get(o, 0) + 1
    for o in outs:
        uses[o] = uses.get(o, 0) + 1
    prod = {r: op for op in ops for r in op.results}

    def gemm_flags(op):
        if op is None or op.name != "custom_call" or op.attrs["target"] != "emi_gemm" or len(op.operands) != 2:
            return None
        cfg = op.attrs["config"]
        return bool(cfg.get("trans_a", False)), bool(cfg.get("trans_b", False))

    # fan-in sums: trees of adds whose leaves are all single-use results of plain products of one shape (2 to 4 of them:
    # what the emi_gemm_grouped handler takes)
    absorbed, sum_rename = set(), {}
    for idx in range(len(ops) - 1, -1, -1):
        op = ops[idx]
        if op.name != "add" or id(op) in absorbed:
            continue
        leaves, inner, stack = [], [], [op]
        while stack:
            a = stack.pop()
            for v in a.operands:
                p_ = prod.get(v)
                if p_ is not None and p_.name == "add" and uses.get(v, 0) == 1:
                    inner.append(p_)
                    stack.append(p_)
                else:
                    leaves.append(v)
        srcs = [prod.get(v) for v in leaves]
        if not (2 <= len(leaves) <= 4) or len(set(leaves)) != len(leaves) or \
                any(gemm_flags(g) != (False, False) or uses.get(v, 0) != 1 for v, g in zip(leaves, srcs)):
            continue
        if any(T[g.operands[0]] != T[srcs[0].operands[0]] or T[g.operands[1]] != T[srcs[0].operands[1]] for g in srcs):
            continue
        srcs.sort(key=lambda g: next(i for i, o in enumerate(ops) if o is g))       # the order the products were emitted in
        cfg_ = {"count": len(srcs), "sum": True, "trans_a": False, "trans_b": False}
        operands_ = [g.operands[0] for g in srcs] + [g.operands[1] for g in srcs]
        nbytes = b._gemm_workspace("emi_gemm_grouped", operands_, cfg_)
        if nbytes:                    # the sum and its scratch as results #0, #1 of one call
            base = b.new(op.types[0])
            names_ = [base + "#0", base + "#1"]
            T[names_[0]], T[names_[1]] = op.types[0], TensorType((nbytes,), "i8")
            sum_rename[op.results[0]] = names_[0]
            ops[idx] = Op("custom_call", names_, operands_, {"target": "emi_gemm_grouped", "config": cfg_}, [op.types[0], T[names_[1]]])
        else:
            ops[idx] = Op("custom_call", list(op.results), operands_, {"target": "emi_gemm_grouped", "config": cfg_}, list(op.types))
        absorbed.update(id(a) for a in inner)
    # weight gradients that share their second operand: one grouped call where the last of them stood
    groups = {}
    for idx, op in enumerate(ops):
        if gemm_flags(op) == (True, False):
            groups.setdefault((op.operands[1], repr(T[op.operands[0]]), repr(op.types[0])), []).append(idx)
    first_use = {}
    for idx, op in enumerate(ops):
        for o in op.operands:
            first_use.setdefault(o, idx)
    rename, drop = dict(sum_rename), set()
    for (x, _, _), idxs in groups.items():
        last = idxs[-1]
        idxs = [i for i in idxs if first_use.get(ops[i].results[0], len(ops)) > last][-4:]      # 2 to 4 products per call
        if len(idxs) < 2 or idxs[-1] != last:
            continue
        tys = [ops[i].types[0] for i in idxs]
        base = b.new(tys[0])
        names = ["%s#%d" % (base, k) for k in range(len(idxs))]
        for n_, t_ in zip(names, tys):
            T[n_] = t_
        for i, n_ in zip(idxs, names):
            rename[ops[i].results[0]] = n_
        cfg_ = {"count": len(idxs), "sum": False, "trans_a": True, "trans_b": False}
        operands_ = [ops[i].operands[0] for i in idxs] + [x] * len(idxs)
        nbytes = b._gemm_workspace("emi_gemm_grouped", operands_, cfg_)
        if nbytes:
            names = names + ["%s#%d" % (base, len(idxs))]
            tys = tys + [TensorType((nbytes,), "i8")]
            T[names[-1]] = tys[-1]
        grouped = Op("custom_call", names, operands_, {"target": "emi_gemm_grouped", "config": cfg_}, tys)
        drop.update(idxs[:-1])
        ops[last] = grouped
    if rename:
        for op in ops:
            op.operands = [rename.get(o, o) for o in op.operands]
        outs = [rename.get(o, o) for o in outs]
    b.ops = [op for i, op in enumerate(ops) if i not in drop]
    return outs


def forward_function(func, name=None, arg_active=None):
    """f_fwd(arg0[, tangent of arg0], arg1[, ...]) -> (result0, tangent of result0, ...): the
    program of the reference's `enzyme-wrap{... mode=ForwardMode}` pass with `enzyme_dup`
    arguments (each followed by its tangent), `enzyme_const` arguments (no tangent) and
    `enzyme_dup` results (primitives.py:1160-1203).  Every operator is followed by the
    operators of its tangent; matched clusters call the tangent targets (`emi_rmsnorm_jvp`,
    `emi_swiglu_jvp`, `emi_attn_step_jvp`, `emi_rope` on the tangent)."""
    func = lower_fused(func, blocks=False)
    b = _Builder(func, "f")
    T = b.types
    if arg_active is None:
        arg_active = [t.dtype in FLOAT for _, t in func.args]
    if len(arg_active) != len(func.args):
        raise ValueError("activity list does not match the function: %d arguments" % len(func.args))
    args, tan = [], {}
    for (a, t), active in zip(func.args, arg_active):
        args.append((a, t))
        if active:
            if t.dtype not in FLOAT:
                raise ValueError("argument %s of type %r cannot be active" % (a, t))
            ta = "%%t_%s" % a[1:]
            T[ta] = t
            args.append((ta, t))
            tan[a] = ta

    def zero(ty):
        return b.const(0.0, ty)

    def tz(v):
        return tan[v] if v in tan else zero(T[v])

    def add(x, y):
        return y if x is None else x if y is None else b.binary("add", x, y)

    outs = None
    for op in func.ops:
        n, xs = op.name, op.operands
        if n == "return":
            outs = []
            for o in xs:
                outs += [o, tz(o)]
            continue
        b.ops.append(op)
        ts = [tan.get(x) for x in xs]
        if all(t is None for t in ts) or not op.results:
            continue
        r = op.results[0]
        t = ts[0]
        if n == "add":
            tan[r] = add(ts[0], ts[1])
        elif n == "subtract":
            tan[r] = ts[0] if ts[1] is None else b.unary("negate", ts[1]) if ts[0] is None else b.binary("subtract", ts[0], ts[1])
        elif n == "multiply":
            tan[r] = add(None if ts[0] is None else b.binary("multiply", ts[0], xs[1]),
                         None if ts[1] is None else b.binary("multiply", ts[1], xs[0]))
        elif n == "divide":
            # (ta b - tb a) / b^2, the form of the reference's FORWARD lines (divide.mlir:9-17)
            num = None if ts[0] is None else b.binary("multiply", ts[0], xs[1])
            if ts[1] is not None:
                sub = b.binary("multiply", ts[1], xs[0])
                num = b.unary("negate", sub) if num is None else b.binary("subtract", num, sub)
            tan[r] = b.binary("divide", num, b.binary("multiply", xs[1], xs[1]))
        elif n == "negate":
            tan[r] = b.unary("negate", t)
        elif n == "exponential":
            tan[r] = b.binary("multiply", t, r)
        elif n == "log":
            tan[r] = b.binary("divide", t, xs[0])
        elif n == "sqrt":
            g = b.binary("divide", t, b.binary("multiply", b.const(2.0, T[r]), r))
            tan[r] = b.emit("select", [b.compare("EQ", xs[0], b.const(0.0, T[r])), b.const(0.0, T[r]), g], {}, T[r])
        elif n in ("maximum", "minimum"):
            m = b.compare("GE" if n == "maximum" else "LE", xs[0], xs[1])
            tan[r] = b.emit("select", [m, tz(xs[0]), tz(xs[1])], {}, T[r])
        elif n == "power":
            ym1 = b.binary("subtract", xs[1], b.const(1.0, T[r]))
            tan[r] = add(None if ts[0] is None else b.binary("multiply", ts[0], b.binary("multiply", xs[1], b.binary("power", xs[0], ym1))),
                         None if ts[1] is None else b.binary("multiply", ts[1], b.binary("multiply", r, b.unary("log", xs[0]))))
        elif n == "atan2":
            # (x ty - y tx) / (x^2 + y^2), the reference's forward form
            den = b.binary("add", b.binary("multiply", xs[1], xs[1]), b.binary("multiply", xs[0], xs[0]))
            num = None if ts[0] is None else b.binary("multiply", xs[1], ts[0])
            if ts[1] is not None:
                sub = b.binary("multiply", xs[0], ts[1])
                num = b.unary("negate", sub) if num is None else b.binary("subtract", num, sub)
            tan[r] = b.binary("divide", num, den)
        elif n == "compare":
            continue
        elif n == "select":
            if ts[1] is not None or ts[2] is not None:
                tan[r] = b.emit("select", [xs[0], tz(xs[1]), tz(xs[2])], {}, T[r])
        elif n == "rsqrt":
            tan[r] = b.binary("multiply", b.binary("multiply", b.const(-0.5, T[r]), t), b.binary("multiply", b.binary("multiply", r, r), r))
        elif n == "logistic":
            tan[r] = b.binary("multiply", b.binary("multiply", t, r), b.binary("subtract", b.const(1.0, T[r]), r))
        elif n == "tanh":
            tan[r] = b.binary("multiply", t, b.binary("subtract", b.const(1.0, T[r]), b.binary("multiply", r, r)))
        elif n == "abs":
            tan[r] = b.emit("select", [b.compare("GE", xs[0], b.const(0.0, T[r])), t, b.unary("negate", t)], {}, T[r])
        elif n == "log_plus_one":
            tan[r] = b.binary("divide", t, b.binary("add", xs[0], b.const(1.0, T[r])))
        elif n == "exponential_minus_one":
            tan[r] = b.binary("multiply", t, b.unary("exponential", xs[0]))
        elif n == "cbrt":
            tan[r] = b.binary("divide", t, b.binary("multiply", b.const(3.0, T[r]), b.binary("multiply", r, r)))
        elif n == "sine":
            tan[r] = b.binary("multiply", t, b.unary("cosine", xs[0]))
        elif n == "cosine":
            tan[r] = b.unary("negate", b.binary("multiply", t, b.unary("sine", xs[0])))
        elif n in ("convert", "reshape", "transpose", "broadcast_in_dim", "slice"):
            tan[r] = b.emit(n, [t], op.attrs, T[r])
        elif n == "reduce":
            if t is None:
                continue
            z0 = zero(TensorType((), T[r].dtype))
            if op.attrs["body"] == "add":
                tan[r] = b.emit("reduce", [t, z0], op.attrs, T[r])
            elif op.attrs["body"] == "maximum":
                # the transpose of the reverse rule: tangents of all maximal elements, summed
                xt = T[xs[0]]
                kept = [d for d in range(len(xt.shape)) if d not in op.attrs["dims"]]
                m = b.compare("EQ", xs[0], b.emit("broadcast_in_dim", [r], {"dims": kept}, xt))
                tan[r] = b.emit("reduce", [b.emit("select", [m, t, b.const(0.0, xt)], {}, xt), z0],
                                {"dims": op.attrs["dims"], "body": "add"}, T[r])
            else:
                raise NotImplementedError("symbolic forward mode of reduce with a %s body" % op.attrs["body"])
        elif n == "pad":
            if t is not None:
                tan[r] = b.emit("pad", [t, zero(TensorType((), T[r].dtype))], op.attrs, T[r])
        elif n == "concatenate":
            tan[r] = b.emit("concatenate", [tz(x) for x in xs], op.attrs, T[r])
        elif n == "gather":
            if ts[0] is not None:              # linear in the table; the indices carry no tangent
                tan[r] = b.emit("gather", [ts[0], xs[1]], op.attrs, T[r])
        elif n == "dot_general":
            tan[r] = add(None if ts[0] is None else b.emit("dot_general", [ts[0], xs[1]], op.attrs, T[r]),
                         None if ts[1] is None else b.emit("dot_general", [xs[0], ts[1]], op.attrs, T[r]))
        elif n == "custom_call":
            target, cfg = op.attrs["target"], op.attrs["config"]
            if target == "emi_rmsnorm_fwd":
                tan[r], = b.custom_call("emi_rmsnorm_jvp", [xs[0], xs[1], tz(xs[0]), tz(xs[1])], {"eps": cfg.get("eps", 1e-5)}, [T[r]])
            elif target == "emi_swiglu_fwd":
                tan[r], = b.custom_call("emi_swiglu_jvp", [xs[0], xs[1], tz(xs[0]), tz(xs[1])], {}, [T[r]])
            elif target == "emi_add":
                tan[r] = add(ts[0], ts[1])
            elif target == "emi_rope":
                if ts[0] is not None:
                    tan[r], = b.custom_call("emi_rope", [ts[0], xs[1]], dict(cfg), [T[r]])
            elif target == "emi_gemm":
                flags = {"trans_a": bool(cfg.get("trans_a", False)), "trans_b": bool(cfg.get("trans_b", False))}
                acc_t = ts[2] if len(xs) > 2 else None
                if ts[0] is not None:
                    acc_t, = b.custom_call("emi_gemm", [ts[0], xs[1]] + ([acc_t] if acc_t is not None else []), flags, [T[r]])
                if ts[1] is not None:
                    acc_t, = b.custom_call("emi_gemm", [xs[0], ts[1]] + ([acc_t] if acc_t is not None else []), flags, [T[r]])
                if acc_t is not None:
                    tan[r] = acc_t
            elif target == "emi_gemm_grouped":
                # sibling projections y_i = x . w_i^T: ty_i = tx . w_i^T + x . tw_i^T, product after product
                n_ = int(cfg["count"])
                if cfg.get("sum", False) or cfg.get("trans_a", False) or not cfg.get("trans_b", False) or len(xs) != 2 * n_:
                    raise NotImplementedError("symbolic forward mode of emi_gemm_grouped other than sibling projections")
                flags = {"trans_a": False, "trans_b": True}
                for i in range(n_):
                    acc_t = None
                    if ts[i] is not None:
                        acc_t, = b.custom_call("emi_gemm", [ts[i], xs[n_ + i]], flags, [T[op.results[i]]])
                    if ts[n_ + i] is not None:
                        acc_t, = b.custom_call("emi_gemm", [xs[i], ts[n_ + i]] + ([acc_t] if acc_t is not None else []), flags,
                                               [T[op.results[i]]])
                    if acc_t is not None:
                        tan[op.results[i]] = acc_t
            elif target == "emi_attn_fwd":
                o, lse = op.results[:2]
                tan[o], = b.custom_call("emi_attn_jvp", [xs[0], xs[1], xs[2], lse, tz(xs[0]), tz(xs[1]), tz(xs[2])],
                                        {"scale": cfg["scale"], "causal": bool(cfg.get("causal", True)), "bshd": bool(cfg.get("bshd", False))},
                                        [T[o]])
            elif target == "emi_cross_entropy_fwd":
                if ts[0] is not None:          # the targets carry no tangent
                    loss, lse = op.results
                    tan[loss], = b.custom_call("emi_cross_entropy_jvp", [xs[0], xs[1], lse, ts[0]], {}, [T[loss]])
            elif target == "emi_attn_step_fwd":
                o, lse, ws = op.results
                tan[o], _ = b.custom_call("emi_attn_step_jvp", [xs[0], xs[1], xs[2], o, lse, tz(xs[0]), tz(xs[1]), tz(xs[2])],
                                          {"scale": cfg["scale"]}, [T[o], T[ws]])
            else:
                raise NotImplementedError("symbolic forward mode of custom call '%s'" % target)
        elif n == "call":
            raise NotImplementedError("symbolic forward mode needs a call-free function (inline_calls)")
        else:
            raise NotImplementedError("symbolic forward mode of stablehlo.%s" % n)
    if outs is None:
        raise ValueError("forward mode needs a return")
    b.ops.append(Op("return", [], outs, {}, []))
    fwd = Func(name or func.name + "_fwd", args, [T[o] for o in outs], b.ops)
    _drop_dead(fwd)
    return fwd


def _reverse_dot_general(b, op, c, accum):
    T = b.types
    a_, b_ = op.operands
    at, bt = T[a_], T[b_]
    ba, bb, ca, cb = (list(op.attrs[k]) for k in ("batch_a", "batch_b", "contract_a", "contract_b"))
    fa = [d for d in range(len(at.shape)) if d not in ba and d not in ca]
    fb = [d for d in range(len(bt.shape)) if d not in bb and d not in cb]
    nb, nfa, nfb = len(ba), len(fa), len(fb)

    def grad(other, ot, obatch, ofree, ocontract, mine_t, mine_batch, mine_free, mine_contract, cfree_at):
        # contract c with `other` over other's free dims: batch, my free dims, other's contracting dims (in its order)
        rest = sorted(ocontract)
        shape = [ot.shape[d] for d in obatch] + [mine_t.shape[d] for d in mine_free] + [ot.shape[d] for d in rest]
        g = b.emit("dot_general", [c, other], {"batch_a": list(range(nb)), "batch_b": list(obatch),
                                                "contract_a": list(range(cfree_at, cfree_at + len(ofree))), "contract_b": list(ofree)},
                   TensorType(shape, mine_t.dtype))
        src = {}
        for i, d in enumerate(mine_batch):
            src[d] = i
        for i, d in enumerate(mine_free):
            src[d] = nb + i
        for i, d in enumerate(rest):
            src[mine_contract[ocontract.index(d)]] = nb + len(mine_free) + i
        perm = [src[d] for d in range(len(mine_t.shape))]
        if perm != list(range(len(perm))):
            g = b.emit("transpose", [g], {"perm": perm}, mine_t)
        return g

    # c dims: batch (nb), free of a (nfa), free of b (nfb)
    accum(a_, grad(b_, bt, bb, fb, cb, at, ba, fa, ca, nb + nfa))
    # for b: c's free-of-a dims (from position nb) meet a's free dims; c's free-of-b dims stay
    accum(b_, grad(a_, at, ba, fa, ca, bt, bb, fb, cb, nb))


def _reverse_custom_call(b, op, cs, accum):
    T = b.types
    target, cfg, xs = op.attrs["target"], op.attrs["config"], op.operands
    c = cs[0]
    if target == "emi_rmsnorm_fwd":
        from . import _native as N
        x, w = xs
        rows = int(np.prod(T[x].shape[:-1])) if len(T[x].shape) > 1 else 1
        nbytes = int(N.lib().emi_rmsnorm_bwd_workspace_bytes(rows, T[x].shape[-1]))
        dx, dg, _ = b.custom_call("emi_rmsnorm_bwd", [x, w, c], {"eps": cfg.get("eps", 1e-5)},
                                  [T[x], T[w], TensorType((nbytes,), "i8")])
        accum(x, dx)
        accum(w, dg)
    elif target == "emi_swiglu_fwd":
        da, db = b.custom_call("emi_swiglu_bwd", [xs[0], xs[1], c], {}, [T[xs[0]], T[xs[1]]])
        accum(xs[0], da)
        accum(xs[1], db)
    elif target == "emi_add":
        accum(xs[0], c)
        accum(xs[1], c)
    elif target == "emi_rope":
        g, = b.custom_call("emi_rope", [c, xs[1]], {"inverse": not cfg.get("inverse", False)}, [T[xs[0]]])
        accum(xs[0], g)
    elif target == "emi_gemm":
        # C = op(A) . op(B) [+ R]: the DotGeneral rule (HLODerivatives.td:1166-1178) in the GEMM's own flags
        ta, tb_ = bool(cfg.get("trans_a", False)), bool(cfg.get("trans_b", False))
        A, Bm = xs[0], xs[1]
        gemm = lambda p, q, fa, fb, ty: b.custom_call("emi_gemm", [p, q], {"trans_a": fa, "trans_b": fb}, [ty])[0]
        src = getattr(b, "producer", {}).get(A)
        if (not ta and tb_ and src is not None and src.name == "custom_call" and src.attrs["target"] == "emi_gemm_swiglu_fwd"
                and A == src.results[1] and b.uses.get(A, 0) == 1):
            # y = g . w2^T with g = swiglu(a, b) of the launch before: dg = c . w2 goes through the SwiGLU adjoint in the
            # epilogue of that product (emi_gemm_swiglu_bwd on the transposed down projection) and never reaches memory;
            # da is the cotangent of a, db becomes the cotangent of the b result of the forward call
            from . import _native as N
            a_, b_res = src.operands[2], src.results[0]
            w2t = b.emit("transpose", [Bm], {"perm": [1, 0]}, TensorType(tuple(reversed(T[Bm].shape)), T[Bm].dtype))
            M_, K_, Hn = T[c].shape[0], T[c].shape[1], T[Bm].shape[1]
            code = 16 if T[c].dtype == "bf16" else 11
            nbytes = int(N.lib().emi_gemm_swiglu_bwd_workspace_bytes(M_, Hn, K_, code))
            da, db, _ = b.custom_call("emi_gemm_swiglu_bwd", [c, w2t, a_, b_res], {}, [T[a_], T[b_res], TensorType((max(nbytes, 16),), "i8")])
            accum(a_, da)
            accum(b_res, db)
            accum(Bm, gemm(c, A, True, False, T[Bm]))
            if len(xs) > 2:
                accum(xs[2], c)
            return
        accum(A, gemm(c, Bm, False, not tb_, T[A]) if not ta else gemm(Bm, c, tb_, True, T[A]))
        accum(Bm, gemm(A, c, not ta, False, T[Bm]) if not tb_ else gemm(c, A, True, ta, T[Bm]))
        if len(xs) > 2:
            accum(xs[2], c)
    elif target == "emi_gemm_grouped":
        # sibling projections y_i = x . w_i^T (DotGeneral rule per product): dX = sum_i dY_i . w_i as one summed
        # launch, dW_i = dY_i^T . x as one grouped launch; a result without a cotangent contributes nothing
        n_ = int(cfg["count"])
        if cfg.get("sum", False) or cfg.get("trans_a", False) or not cfg.get("trans_b", False) or len(xs) != 2 * n_ or \
                any(x != xs[0] for x in xs[:n_]):
            raise NotImplementedError("symbolic reverse mode of emi_gemm_grouped other than sibling projections of one operand")
        live = [i for i in range(n_) if cs[i] is not None]
        x = xs[0]
        if len(live) >= 2:
            dx, = b.custom_call("emi_gemm_grouped", [cs[i] for i in live] + [xs[n_ + i] for i in live],
                                {"count": len(live), "sum": True, "trans_a": False, "trans_b": False}, [T[x]])
            accum(x, dx)
            dws = b.custom_call("emi_gemm_grouped", [cs[i] for i in live] + [x] * len(live),
                                {"count": len(live), "sum": False, "trans_a": True, "trans_b": False}, [T[xs[n_ + i]] for i in live])
            for i, dw in zip(live, dws):
                accum(xs[n_ + i], dw)
        else:
            for i in live:
                accum(x, b.custom_call("emi_gemm", [cs[i], xs[n_ + i]], {"trans_a": False, "trans_b": False}, [T[x]])[0])
                accum(xs[n_ + i], b.custom_call("emi_gemm", [cs[i], x], {"trans_a": True, "trans_b": False}, [T[xs[n_ + i]]])[0])
    elif target == "emi_gemm_rope":
        # y = rope(x . w^T): the cotangent is turned back by the angle (unless the attention adjoint already did that as
        # it stored dq / dk), then the DotGeneral rule
        x, w, tab = xs
        if c not in getattr(b, "unrotated", ()):
            S_, d = T[tab].shape[0], 2 * T[tab].shape[1]
            M_, D_ = T[c].shape
            c4 = b.reshape(c, (M_ // S_, S_, D_ // d, d))
            g4, = b.custom_call("emi_rope", [c4, tab], {"inverse": True}, [T[c4]])
            c = b.reshape(g4, (M_, D_))
        accum(x, b.custom_call("emi_gemm", [c, w], {"trans_a": False, "trans_b": False}, [T[x]])[0])
        accum(w, b.custom_call("emi_gemm", [c, x], {"trans_a": True, "trans_b": False}, [T[w]])[0])
    elif target == "emi_gemm_swiglu_fwd":
        # (b, g) = (x . w3^T, swiglu(a, b)): a cotangent of g goes through the SwiGLU adjoint (the joint rule of the
        # product that consumes g has usually taken it already), the total cotangent of b through the DotGeneral rule
        x, w3, a_ = xs
        cb, cg = cs[0], cs[1] if len(cs) > 1 else None
        if cg is not None:
            da, db = b.custom_call("emi_swiglu_bwd", [a_, op.results[0], cg], {}, [T[a_], T[op.results[0]]])
            accum(a_, da)
            cb = db if cb is None else b.binary("add", cb, db)
        if cb is not None:
            accum(x, b.custom_call("emi_gemm", [cb, w3], {"trans_a": False, "trans_b": False}, [T[x]])[0])
            accum(w3, b.custom_call("emi_gemm", [cb, x], {"trans_a": True, "trans_b": False}, [T[w3]])[0])
    elif target == "emi_attn_fwd":
        if any(x is not None for x in cs[1:]):
            raise NotImplementedError("cotangents of the log-sum-exp or workspace results of emi_attn_fwd")
        if c is None:
            return
        from . import _native as N
        q, k, v = xs
        o, lse = op.results[:2]
        bshd = bool(cfg.get("bshd", False))
        qs = T[q].shape
        B_, S_, h, d = (qs[0], qs[1], qs[2], qs[3]) if bshd else (qs[0], qs[2], qs[1], qs[3])
        nbytes = int(N.lib().emi_attn_bwd_workspace_bytes(B_, h, S_, d))
        # q and k that are (reshapes of) projections stored rotated with one table, each with this one use: the adjoint
        # turns dq and dk back as it stores them
        def rotated_projection(v_):
            p_ = getattr(b, "producer", {}).get(v_)
            if p_ is not None and p_.name == "reshape" and b.uses.get(v_, 0) == 1:
                v_ = p_.operands[0]
                p_ = b.producer.get(v_)
            if p_ is not None and p_.name == "custom_call" and p_.attrs["target"] == "emi_gemm_rope" and b.uses.get(v_, 0) == 1:
                return p_.operands[2]
            return None
        tq, tk = rotated_projection(q), rotated_projection(k)
        if bshd and tq is not None and tq == tk and q != k:
            dq, dk, dv, _ = b.custom_call("emi_attn_bwd_rope", [q, k, v, o, lse, c, tq],
                                          {"scale": cfg["scale"], "causal": bool(cfg.get("causal", True)), "bshd": True},
                                          [T[q], T[k], T[v], TensorType((nbytes,), "i8")])
            b.unrotated.update((dq, dk))
            accum(q, dq)
            accum(k, dk)
            accum(v, dv)
            return
        dq, dk, dv, _ = b.custom_call("emi_attn_bwd", [q, k, v, o, lse, c],
                                      {"scale": cfg["scale"], "causal": bool(cfg.get("causal", True)), "bshd": bshd},
                                      [T[q], T[k], T[v], TensorType((nbytes,), "i8")])
        accum(q, dq)
        accum(k, dk)
        accum(v, dv)
    elif target == "emi_attn_step_fwd":
        if cs[1] is not None or (len(cs) > 2 and cs[2] is not None):
            raise NotImplementedError("cotangents of the log-sum-exp or workspace results of emi_attn_step_fwd")
        if c is None:
            return
        q, k, v = xs
        o, lse, ws = op.results
        dq, dk, dv, _ = b.custom_call("emi_attn_step_bwd", [q, k, v, o, lse, c], {"scale": cfg["scale"]}, [T[q], T[k], T[v], T[ws]])
        accum(q, dq)
        accum(k, dk)
        accum(v, dv)
    elif target == "emi_cross_entropy_fwd":
        if len(cs) > 1 and cs[1] is not None:
            raise NotImplementedError("cotangent of the log-sum-exp result of emi_cross_entropy_fwd")
        if c is None:
            return
        z, t = xs
        lse = op.results[1]
        dz, = b.custom_call("emi_cross_entropy_bwd", [z, t, lse, c], {}, [T[z]])       # the targets are inactive
        accum(z, dz)
    else:
        raise NotImplementedError("symbolic reverse mode of custom call '%s'" % target)


def reverse_module_text(text, fn="main", arg_active=None, ret_active=None):
    """StableHLO text in, StableHLO text of the reverse-mode program out: calls inlined,
    constants folded, clusters matched, `reverse_function`, printed with the fused operators
    and their adjoints as typed-FFI custom calls."""
    from .stablehlo import fold_constants, fuse_clusters, parse_module, print_module

    f = inline_calls(parse_module(text), fn)
    fold_constants(f)
    fuse_clusters(f)
    rev = reverse_function(f, name="main", arg_active=arg_active, ret_active=ret_active)
    return print_module({"main": rev})


def forward_module_text(text, fn="main", arg_active=None):
    """StableHLO text in, StableHLO text of the forward-mode program out (see `forward_function`)."""
    from .stablehlo import fold_constants, fuse_clusters, parse_module, print_module

    f = inline_calls(parse_module(text), fn)
    fold_constants(f)
    fuse_clusters(f)
    return print_module({"main": forward_function(f, name="main", arg_active=arg_active)})
