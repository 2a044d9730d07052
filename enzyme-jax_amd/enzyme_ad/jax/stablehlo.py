"""StableHLO text front end: parse a module, match the llama clusters to the fused kernels,
and run the rest operator by operator on the device.

The reference hands StableHLO text (`hlo_call`, src/enzyme_ad/jax/primitives.py:1052-1108; the
text of an `enzyme_jax_ir`-decorated function, :626-692) to MLIR passes and XLA's code
generator.  Here the text is parsed into a small SSA graph (`parse_module`), rewritten by
`fuse_clusters` (RMSNorm, SwiGLU and softmax-attention clusters of test/llama.py become one
fused operator each), and executed by `Executable.run` through `enzyme_ad.jax.ops` /
`hlo_ops`, whose operators carry the forward- and reverse-mode rules: `jvp` and `vjp` of a
function that calls `hlo_call` differentiate through the parsed graph.

The accepted text is MLIR's printed form of the operators JAX emits for such functions
(pretty or quoted-generic operator names): constant, add, subtract, multiply, divide, maximum,
minimum, power, atan2, clamp (as maximum + minimum), negate, exponential, log, sqrt, rsqrt, logistic, tanh, sine, cosine, abs, log_plus_one,
exponential_minus_one, cbrt, convert, reshape,
transpose, broadcast_in_dim, reduce (add / maximum), dot_general, slice, pad, concatenate, compare,
select, call,
custom_call (this library's targets), return.  Anything else raises `NotImplementedError` naming the operator.
"""
import math
import re

import numpy as np
import torch

from . import _native as N
from . import hlo_ops as H
from . import ops


class ParseError(ValueError):
    pass


class TensorType:
    __slots__ = ("shape", "dtype")

    def __init__(self, shape, dtype):
        self.shape, self.dtype = tuple(shape), dtype

    def __eq__(self, o):
        return isinstance(o, TensorType) and self.shape == o.shape and self.dtype == o.dtype

    def __repr__(self):
        return "tensor<%s>" % "x".join([str(s) for s in self.shape] + [self.dtype])


class Op:
    __slots__ = ("name", "results", "operands", "attrs", "types")

    def __init__(self, name, results, operands, attrs, types):
        self.name, self.results, self.operands, self.attrs, self.types = name, results, operands, attrs, types

    def __repr__(self):
        return "%s = %s(%s) %s" % (", ".join(self.results), self.name, ", ".join(self.operands), self.attrs)


class Func:
    def __init__(self, name, args, result_types, ops_):
        self.name, self.args, self.result_types, self.ops = name, args, result_types, ops_


TORCH_DTYPES = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16, "f64": torch.float64,
                "i32": torch.int32, "i64": torch.int64, "i1": torch.bool, "ui32": torch.int32, "i8": torch.int8}
NUMPY_DTYPES = {"f32": np.float32, "f64": np.float64, "f16": np.float16, "i32": np.int32, "i64": np.int64,
                "i1": np.bool_, "ui32": np.uint32, "i8": np.int8}

BINARY_OPS = {"add", "subtract", "multiply", "divide", "maximum", "minimum", "power", "atan2"}
UNARY_OPS = {"negate", "exponential", "log", "sqrt", "rsqrt", "logistic", "tanh", "sine", "cosine", "abs", "log_plus_one",
             "exponential_minus_one", "cbrt"}


# ---------------------------------------------------------------------------
# parser
# ---------------------------------------------------------------------------

_WS = re.compile(r"(?:\s+|//[^\n]*)*")
_SSA = re.compile(r"%[A-Za-z0-9_.$-]+(?:#\d+)?")
_SYM = re.compile(r"@[A-Za-z0-9_.$-]+|@\"[^\"]*\"")
_IDENT = re.compile(r"[A-Za-z_][A-Za-z0-9_.$]*")
_INT = re.compile(r"-?\d+")
_OPEN = {"(": ")", "[": "]", "{": "}", "<": ">"}


class _Scanner:
    def __init__(self, text):
        self.s, self.i = text, 0

    def ws(self):
        self.i = _WS.match(self.s, self.i).end()

    def eof(self):
        self.ws()
        return self.i >= len(self.s)

    def peek(self, lit):
        self.ws()
        return self.s.startswith(lit, self.i)

    def accept(self, lit):
        if self.peek(lit):
            self.i += len(lit)
            return True
        return False

    def expect(self, lit):
        if not self.accept(lit):
            self.fail("expected '%s'" % lit)

    def match(self, rx):
        self.ws()
        m = rx.match(self.s, self.i)
        if m:
            self.i = m.end()
            return m.group(0)
        return None

    def need(self, rx, what):
        v = self.match(rx)
        if v is None:
            self.fail("expected %s" % what)
        return v

    def fail(self, msg):
        line = self.s.count("\n", 0, self.i) + 1
        near = self.s[self.i:self.i + 40].split("\n")[0]
        raise ParseError("StableHLO text, line %d: %s near '%s'" % (line, msg, near))

    def balanced(self):
        """The text of one bracketed group starting at the cursor, brackets included.
        '->' does not close an angle bracket; strings are skipped."""
        self.ws()
        start = self.i
        stack = []
        while self.i < len(self.s):
            c = self.s[self.i]
            if c == '"':
                j = self.s.find('"', self.i + 1)
                if j < 0:
                    self.fail("unterminated string")
                self.i = j + 1
                continue
            if c in _OPEN:
                stack.append(_OPEN[c])
            elif c in ")]}>":
                if c == ">" and self.s[self.i - 1] == "-":
                    self.i += 1
                    continue
                if not stack or stack[-1] != c:
                    self.fail("unbalanced '%s'" % c)
                stack.pop()
                if not stack:
                    self.i += 1
                    return self.s[start:self.i]
            self.i += 1
        self.fail("unbalanced bracket")

    def ints(self):
        """[1, 2, 3] -> [1, 2, 3]"""
        body = self.balanced()
        if body[0] != "[":
            self.fail("expected an integer list")
        return [int(t) for t in re.findall(r"-?\d+", body)]

    def type(self):
        self.ws()
        if not self.accept("tensor"):
            self.fail("expected a tensor type")
        body = self.balanced()[1:-1].strip()
        parts = body.split("x")
        dtype = parts[-1].strip()
        # element types such as 'bf16' contain no 'x'; dimensions are integers
        dims = []
        for p in parts[:-1]:
            p = p.strip()
            if not re.fullmatch(r"\d+", p):
                self.fail("dynamic or malformed dimension '%s'" % p)
            dims.append(int(p))
        if dtype not in TORCH_DTYPES:
            self.fail("unsupported element type '%s'" % dtype)
        return TensorType(dims, dtype)

    def signature(self):
        """': type' or ': (types) -> type | (types)': returns (operand types or None, result types)."""
        self.expect(":")
        if self.peek("("):
            self.expect("(")
            ins = []
            if not self.accept(")"):
                while True:
                    ins.append(self.type())
                    if self.accept(")"):
                        break
                    self.expect(",")
            self.expect("->")
            return ins, self.type_list()
        first = self.type()
        types = [first]
        while self.accept(","):
            types.append(self.type())
        if self.accept("->"):
            return types, self.type_list()
        return None, types

    def type_list(self):
        if self.accept("("):
            outs = []
            if not self.accept(")"):
                while True:
                    outs.append(self.type())
                    if self.peek("{"):
                        self.balanced()
                    if self.accept(")"):
                        break
                    self.expect(",")
            return outs
        return [self.type()]


def _dense(body, ty):
    """dense<...> payload -> numpy array of the tensor type."""
    body = body.strip()
    n = int(np.prod(ty.shape)) if ty.shape else 1
    width = {"f32": 4, "bf16": 2, "f16": 2, "f64": 8, "i32": 4, "i64": 8, "i1": 1, "ui32": 4, "i8": 1}[ty.dtype]

    def from_bits(raw):
        if ty.dtype == "bf16":
            u = np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16
            return u.view(np.float32)
        return np.frombuffer(raw, dtype=np.dtype(NUMPY_DTYPES[ty.dtype]).newbyteorder("<"))

    if body.startswith('"'):                                   # "0x..." raw little-endian bytes
        hexs = body.strip('"')
        if not hexs.startswith("0x"):
            raise ParseError("dense string payload must be hex")
        raw = bytes.fromhex(hexs[2:])
        arr = from_bits(raw)
        if arr.size == 1 and n > 1:
            arr = np.repeat(arr, n)
        if arr.size != n:
            raise ParseError("dense payload has %d elements, type %r wants %d" % (arr.size, ty, n))
        return np.array(arr).reshape(ty.shape)

    def scalar(tok):
        tok = tok.strip()
        if tok in ("true", "false"):
            return tok == "true"
        if tok.lower().startswith("0x") and ty.dtype in ("f32", "bf16", "f16", "f64"):
            bits = int(tok, 16)
            return from_bits(bits.to_bytes(width, "little"))[0]
        if ty.dtype.startswith("f") or ty.dtype == "bf16":
            return float(tok)
        return int(tok, 0)

    toks = [t for t in re.split(r"[\[\],\s]+", body) if t]
    vals = [scalar(t) for t in toks]
    if len(vals) == 1:
        vals = vals * n
    if len(vals) != n:
        raise ParseError("dense payload has %d elements, type %r wants %d" % (len(vals), ty, n))
    npdt = np.float32 if ty.dtype == "bf16" else NUMPY_DTYPES[ty.dtype]
    return np.array(vals, dtype=npdt).reshape(ty.shape)


def _i64_array(text, key):
    """key = array<i64: 1, 0> or key = dense<[1, 0]> : tensor<2xi64> -> [1, 0]"""
    m = re.search(key + r"\s*=\s*(array<i64:?([^>]*)>|dense<([^>]*)>)", text)
    if not m:
        raise ParseError("attribute %s not found" % key)
    return [int(t) for t in re.findall(r"-?\d+", m.group(2) if m.group(2) is not None else m.group(3))]


def _backend_config(text):
    """{name: value} of the `backend_config = {...}` dictionary of a custom call (numbers and
    booleans; the wire format of typed-FFI calls, Passes/LowerEnzymeXLABLAS.cpp:463-479)."""
    m = re.search(r"backend_config\s*=\s*\{", text)
    if not m:
        return {}
    body = _Scanner(text[m.end() - 1:]).balanced()[1:-1]
    out = {}
    for key, val in re.findall(r"([A-Za-z_][A-Za-z0-9_]*)\s*=\s*([^,:}]+)", body):
        val = val.strip()
        if val in ("true", "false"):
            out[key] = val == "true"
        else:
            try:
                out[key] = int(val)
            except ValueError:
                out[key] = float(val)
    return out


def _attr_lists(text, key):
    m = re.search(key + r"\s*=\s*\[([^\]]*)\]", text)
    return [int(t) for t in re.findall(r"-?\d+", m.group(1))] if m else []


def _parse_op(sc):
    results = []
    save = sc.i
    first = sc.match(_SSA)
    if first is not None:
        names = [first]
        count = 1
        if sc.accept(":"):
            count = int(sc.need(_INT, "result count"))
        while sc.accept(","):
            names.append(sc.need(_SSA, "result name"))
        sc.expect("=")
        results = names if count == 1 else ["%s#%d" % (first, k) for k in range(count)]
    else:
        sc.i = save
    generic = sc.peek('"')
    if generic:
        sc.expect('"')
        name = sc.need(_IDENT, "operator name")
        sc.expect('"')
    else:
        name = sc.need(_IDENT, "operator name")
    short = name.split(".", 1)[1] if name.startswith(("stablehlo.", "mhlo.", "func.", "arith.")) else name
    attrs = {}

    def operand_list():
        out = []
        while True:
            v = sc.match(_SSA)
            if v is None:
                break
            out.append(v)
            before = sc.i
            if not sc.accept(","):
                break
            if not sc.peek("%"):
                sc.i = before      # the comma belongs to a trailing attribute
                break
        return out

    if short in ("return",):
        operands = operand_list()
        if operands:
            sc.signature()
        return Op("return", [], operands, attrs, [])

    if generic:
        sc.expect("(")
        operands = operand_list()
        sc.expect(")")
        text = ""
        while sc.peek("<{") or sc.peek("{"):
            if sc.accept("<"):
                text += sc.balanced()
                sc.expect(">")
            else:
                text += sc.balanced()
        if sc.peek("("):                                       # regions of a generic operator
            sc.fail("regions of quoted operators are not supported")
        _, types = sc.signature()
        if short == "dot_general":
            attrs = {"batch_a": _attr_lists(text, "lhs_batching_dimensions"),
                     "batch_b": _attr_lists(text, "rhs_batching_dimensions"),
                     "contract_a": _attr_lists(text, "lhs_contracting_dimensions"),
                     "contract_b": _attr_lists(text, "rhs_contracting_dimensions")}
        elif short == "transpose":
            attrs = {"perm": _i64_array(text, "permutation")}
        elif short == "broadcast_in_dim":
            attrs = {"dims": _i64_array(text, "broadcast_dimensions")}
        elif short == "concatenate":
            attrs = {"dim": int(re.search(r"dimension\s*=\s*(\d+)", text).group(1))}
        elif short == "constant":
            m = re.search(r"value\s*=\s*dense<", text)
            if not m:
                sc.fail("constant without a dense value")
            sub = _Scanner(text[m.end() - 1:])
            attrs = {"value": _dense(sub.balanced()[1:-1], types[0])}
        elif short == "gather":
            attrs = _gather_attrs(text)
        elif short in BINARY_OPS or short in UNARY_OPS or short in ("reshape", "convert"):
            pass
        else:
            raise NotImplementedError("StableHLO operator '%s' in quoted form is not supported" % name)
        return Op(short, results, operands, attrs, types)

    if short == "constant":
        sc.expect("dense")
        body = sc.balanced()[1:-1]
        _, types = sc.signature()
        return Op("constant", results, [], {"value": _dense(body, types[0])}, types)
    if short == "reduce":
        sc.expect("(")
        x = sc.need(_SSA, "operand")
        sc.expect("init")
        sc.expect(":")
        init = sc.need(_SSA, "init value")
        sc.expect(")")
        body = None
        if sc.accept("applies"):
            body = sc.need(_IDENT, "reduction operator")
        sc.expect("across")
        sc.expect("dimensions")
        sc.expect("=")
        dims = sc.ints()
        _, types = sc.signature()
        if body is None:
            sc.expect("reducer")
            sc.balanced()                       # block arguments
            region = sc.balanced()
            found = re.findall(r"(?:stablehlo|mhlo)\.(add|maximum|minimum|multiply)\b", region)
            if len(found) != 1:
                sc.fail("reduce body must be one add or maximum")
            body = found[0]
        body = body.split(".")[-1]
        return Op("reduce", results, [x, init], {"dims": dims, "body": body}, types)
    if short == "custom_call":
        target = sc.need(_SYM, "custom-call target")[1:].strip('"')
        sc.expect("(")
        operands = operand_list()
        sc.expect(")")
        text = sc.balanced() if sc.peek("{") else "{}"
        _, types = sc.signature()
        return Op("custom_call", results, operands, {"target": target, "config": _backend_config(text)}, types)
    if short == "iota":
        sc.expect("dim")
        sc.expect("=")
        dim = int(sc.need(_INT, "iota dimension"))
        _, types = sc.signature()
        return Op("iota", results, [], {"dim": dim}, types)
    if short == "compare":
        direction = sc.need(_IDENT, "comparison direction")
        sc.expect(",")
        operands = operand_list()
        if sc.accept(","):
            sc.need(_IDENT, "comparison type")               # FLOAT / TOTALORDER / SIGNED: floats compare as IEEE here
        _, types = sc.signature()
        if direction not in H.COMPARE:
            sc.fail("unknown comparison direction '%s'" % direction)
        return Op("compare", results, operands, {"direction": direction}, types[-1:])
    if short == "select":
        operands = operand_list()
        _, types = sc.signature()
        return Op("select", results, operands, {}, types[-1:])
    if short == "clamp":
        # clamp(min, x, max) = minimum(maximum(x, min), max): two operators, so that every rule and rewrite of
        # those applies (an operand at a bound keeps its cotangent, outside it gets none: clamp.mlir:14-26)
        operands = operand_list()
        in_types, types = sc.signature()
        in_types = in_types or []
        if len(operands) != 3:
            sc.fail("clamp takes (min, operand, max)")
        out, seq = types[-1], []
        bounds = []
        for tag, v, ty in (("lo", operands[0], in_types[0] if len(in_types) == 3 else out),
                           ("hi", operands[2], in_types[2] if len(in_types) == 3 else out)):
            if ty.shape == () and out.shape != ():          # rank-0 bounds are allowed: broadcast them
                wide = "%s__clamp_%s" % (results[0], tag)
                seq.append(Op("broadcast_in_dim", [wide], [v], {"dims": []}, [out]))
                v = wide
            bounds.append(v)
        inner = results[0] + "__clamp_max"
        return seq + [Op("maximum", [inner], [operands[1], bounds[0]], {}, [out]),
                      Op("minimum", results, [inner, bounds[1]], {}, [out])]
    if short == "call":
        callee = sc.need(_SYM, "callee")
        sc.expect("(")
        operands = operand_list()
        sc.expect(")")
        if sc.peek("{"):
            sc.balanced()
        _, types = sc.signature()
        return Op("call", results, operands, {"callee": callee[1:].strip('"')}, types)
    if short == "slice":
        x = sc.need(_SSA, "operand")
        body = sc.balanced()
        if body[0] != "[":
            sc.fail("expected slice bounds")
        start, limit, stride = [], [], []
        for part in body[1:-1].split(","):
            nums = [int(t) for t in part.strip().split(":")]
            start.append(nums[0])
            limit.append(nums[1])
            stride.append(nums[2] if len(nums) > 2 else 1)
        _, types = sc.signature()
        return Op("slice", results, [x], {"start": start, "limit": limit, "stride": stride}, types)

    operands = operand_list()
    # trailing attributes: ', key = value'
    while sc.accept(","):
        key = sc.need(_IDENT, "attribute name")
        sc.expect("=")
        if sc.peek("["):
            v = sc.ints() if not re.match(r"\s*\[\s*[A-Za-z]", sc.s[sc.i:]) else sc.balanced()
            if sc.accept("x"):
                v = (v, sc.ints())
        elif sc.peek("<") or sc.peek("{") or sc.peek("("):
            v = sc.balanced()
        else:
            v = sc.need(re.compile(r"[A-Za-z0-9_.+-]+"), "attribute value")
        attrs[key] = v
    if sc.peek("{"):
        sc.balanced()                            # a discardable attribute dictionary
    _, types = sc.signature()
    if short == "dot_general":
        b = attrs.get("batching_dims", ([], []))
        c = attrs.get("contracting_dims", ([], []))
        attrs = {"batch_a": b[0], "batch_b": b[1], "contract_a": c[0], "contract_b": c[1]}
    elif short == "transpose":
        attrs = {"perm": attrs["dims"]}
    elif short == "broadcast_in_dim":
        attrs = {"dims": attrs["dims"]}
    elif short == "concatenate":
        attrs = {"dim": int(attrs["dim"])}
    elif short == "pad":
        attrs = {"low": attrs["low"], "high": attrs["high"], "interior": attrs.get("interior", [0] * len(attrs["low"]))}
    elif short in BINARY_OPS or short in UNARY_OPS or short in ("reshape", "convert"):
        attrs = {}
    else:
        raise NotImplementedError("StableHLO operator '%s' is not supported by the HIP front end" % name)
    return Op(short, results, operands, attrs, types)


def _gather_attrs(text):
    """Attributes of a quoted `stablehlo.gather`; only the row lookup `table[indices]` an embedding traces to is
    accepted (checked against the operand types by `check_gather`): whole rows of a rank-2 operand selected by one
    index each."""
    def ints(key):
        m = re.search(key + r"\s*=\s*\[([^\]]*)\]", text)
        return [int(v) for v in m.group(1).split(",") if v.strip()] if m else []
    m = re.search(r"index_vector_dim\s*=\s*(\d+)", text)
    ss = re.search(r"slice_sizes\s*=\s*(?:array<i64:\s*([^>]*)>|dense<\[([^\]]*)\]>)", text)
    if m is None or ss is None:
        raise ParseError("stablehlo.gather without index_vector_dim / slice_sizes")
    return {"offset_dims": ints("offset_dims"), "collapsed_slice_dims": ints("collapsed_slice_dims"),
            "operand_batching_dims": ints("operand_batching_dims"),
            "start_indices_batching_dims": ints("start_indices_batching_dims"), "start_index_map": ints("start_index_map"),
            "index_vector_dim": int(m.group(1)),
            "slice_sizes": [int(v) for v in (ss.group(1) or ss.group(2)).split(",") if v.strip()]}


def check_gather(attrs, table_t, idx_t, out_t):
    """Raises NotImplementedError unless the gather is `table[indices]`: operand [V, D], indices [..., 1] (the index
    vector last), one collapsed dimension 0, slices of one whole row, result [..., D]."""
    lead = tuple(idx_t.shape[:-1])
    ok = (len(table_t.shape) == 2 and len(idx_t.shape) >= 1 and idx_t.shape[-1] == 1
          and attrs["index_vector_dim"] == len(idx_t.shape) - 1 and attrs["collapsed_slice_dims"] == [0]
          and attrs["start_index_map"] == [0] and not attrs["operand_batching_dims"]
          and attrs["offset_dims"] == [len(lead)] and attrs["slice_sizes"] == [1, table_t.shape[1]]
          and tuple(out_t.shape) == lead + (table_t.shape[1],) and idx_t.dtype in ("i32", "i64"))
    if not ok:
        raise NotImplementedError("stablehlo.gather other than a row lookup table[indices] (operand %r, indices %r, %s)" %
                                  (table_t, idx_t, attrs))


def _parse_func(sc):
    for vis in ("public", "private", "nested"):
        sc.accept(vis)
    name = sc.need(_SYM, "function name")[1:].strip('"')
    sc.expect("(")
    args = []
    if not sc.accept(")"):
        while True:
            a = sc.need(_SSA, "argument name")
            sc.expect(":")
            t = sc.type()
            if sc.peek("{"):
                sc.balanced()
            args.append((a, t))
            if sc.accept(")"):
                break
            sc.expect(",")
    result_types = []
    if sc.accept("->"):
        result_types = sc.type_list()
    if sc.accept("attributes"):
        sc.balanced()
    sc.expect("{")
    body = []
    while not sc.accept("}"):
        op = _parse_op(sc)
        body.extend(op if isinstance(op, list) else [op])
    return Func(name, args, result_types, body)


def _strip_locations(text):
    """Debug locations (`loc(...)` trailers, nested to any depth, and `#loc = ...` alias lines)
    carry nothing the executor uses."""
    if "loc(" not in text:
        return text
    text = "\n".join(l for l in text.split("\n") if not l.lstrip().startswith("#loc"))
    out, i, n = [], 0, len(text)
    while i < n:
        j = text.find("loc(", i)
        if j < 0:
            out.append(text[i:])
            break
        if j > 0 and (text[j - 1].isalnum() or text[j - 1] in "_.#"):
            out.append(text[i:j + 4])                      # part of a longer name
            i = j + 4
            continue
        out.append(text[i:j])
        k, depth = j + 3, 0
        while k < n:
            c = text[k]
            if c == '"':
                k = text.find('"', k + 1)
                if k < 0:
                    raise ParseError("unterminated string in a location")
            elif c == "(":
                depth += 1
            elif c == ")":
                depth -= 1
                if depth == 0:
                    break
            k += 1
        i = k + 1
    return "".join(out)


def parse_module(text):
    """{function name: Func} of a StableHLO module (or of bare func.func definitions)."""
    sc = _Scanner(_strip_locations(text))
    funcs = {}
    wrapped = False
    if sc.accept("module"):
        wrapped = True
        sc.match(_SYM)
        if sc.accept("attributes"):
            sc.balanced()
        sc.expect("{")
    while not sc.eof():
        if wrapped and sc.accept("}"):
            break
        if sc.accept("func.func"):
            f = _parse_func(sc)
            funcs[f.name] = f
        else:
            sc.fail("expected func.func")
    if not funcs:
        raise ParseError("StableHLO text holds no function")
    return funcs


# ---------------------------------------------------------------------------
# cluster matcher
# ---------------------------------------------------------------------------

def _users(func):
    use = {}
    for op in func.ops:
        for o in op.operands:
            use.setdefault(o, []).append(op)
    return use


def _splat(op):
    """The value of a constant whose elements are all equal, else None."""
    if op is None or op.name != "constant":
        return None
    v = op.attrs["value"]
    flat = np.asarray(v).reshape(-1)
    if flat.size == 0 or not np.all(flat == flat[0]):
        return None
    return float(flat[0])


_FOLD_UNARY = {"negate": np.negative, "exponential": np.exp, "log": np.log, "sqrt": np.sqrt,
               "rsqrt": lambda v: 1.0 / np.sqrt(v), "tanh": np.tanh, "sine": np.sin, "cosine": np.cos,
               "logistic": lambda v: 1.0 / (1.0 + np.exp(-v)), "abs": np.abs, "log_plus_one": np.log1p,
               "exponential_minus_one": np.expm1, "cbrt": np.cbrt}
_FOLD_BINARY = {"add": np.add, "subtract": np.subtract, "multiply": np.multiply, "divide": np.divide,
                "maximum": np.maximum, "minimum": np.minimum, "power": np.power, "atan2": np.arctan2}


_FOLD_COMPARE = {"EQ": np.equal, "NE": np.not_equal, "GE": np.greater_equal, "GT": np.greater, "LE": np.less_equal,
                 "LT": np.less}
MASK_LIMIT = 1 << 25          # elements of a trace-time mask (iota / compare / broadcast of i1) folded at parse


def fold_constants(func, limit=4096):
    """Evaluates, at parse time, operators whose operands are all constants (like
    `jnp.sqrt(head_size)`, test/llama.py:196, which reaches the text as sqrt of a constant),
    up to `limit` result elements, in the element type's precision; then drops operators
    whose results nothing uses."""
    defs = {}
    out = []
    for op in func.ops:
        srcs = [defs.get(o) for o in op.operands]
        ty = op.types[0] if op.types else None
        new = None
        # masks that depend on no argument (`jnp.tril`-style causal masks: iota, iota, compare)
        if ty is not None and int(np.prod(ty.shape or (1,))) <= MASK_LIMIT and all(c is not None and c.name == "constant" for c in srcs):
            mask = None
            if op.name == "iota" and ty.dtype in ("i32", "i64"):
                shape = [1] * len(ty.shape)
                shape[op.attrs["dim"]] = ty.shape[op.attrs["dim"]]
                mask = np.broadcast_to(np.arange(ty.shape[op.attrs["dim"]], dtype=NUMPY_DTYPES[ty.dtype]).reshape(shape), ty.shape)
            elif op.name == "compare" and ty.dtype == "i1":
                mask = _FOLD_COMPARE[op.attrs["direction"]](np.asarray(srcs[0].attrs["value"]), np.asarray(srcs[1].attrs["value"]))
            elif op.name == "broadcast_in_dim" and ty.dtype == "i1":
                v = np.asarray(srcs[0].attrs["value"])
                shape = [1] * len(ty.shape)
                for i, d in enumerate(op.attrs["dims"]):
                    shape[d] = v.shape[i]
                mask = np.broadcast_to(v.reshape(shape), ty.shape)
            if mask is not None:
                op = Op("constant", op.results, [], {"value": mask}, op.types)
                for r in op.results:
                    defs[r] = op
                out.append(op)
                continue
        if op.operands and all(c is not None and c.name == "constant" for c in srcs) and ty is not None \
                and ty.dtype in ("f32", "bf16") and int(np.prod(ty.shape or (1,))) <= limit:
            vals = [np.asarray(c.attrs["value"], dtype=np.float32) for c in srcs]
            if op.name in _FOLD_UNARY:
                new = _FOLD_UNARY[op.name](vals[0])
            elif op.name in _FOLD_BINARY:
                new = _FOLD_BINARY[op.name](vals[0], vals[1])
            elif op.name == "reshape":
                new = vals[0].reshape(ty.shape)
            elif op.name == "transpose":
                new = vals[0].transpose(op.attrs["perm"])
            elif op.name == "broadcast_in_dim" and _splat(srcs[0]) is not None:
                new = np.full(ty.shape, vals[0].reshape(-1)[0], dtype=np.float32)       # tables stay tables
            elif op.name == "convert":
                new = vals[0]
            if new is not None:
                new = np.asarray(new, dtype=np.float32)
                if ty.dtype == "bf16":
                    new = torch.from_numpy(np.array(new)).to(torch.bfloat16).float().numpy()
                op = Op("constant", op.results, [], {"value": np.array(new).reshape(ty.shape)}, op.types)
        for r in op.results:
            defs[r] = op
        out.append(op)
    func.ops = out
    _drop_dead(func)


def _drop_dead(func):
    live = set()
    kept = []
    for op in reversed(func.ops):
        if op.name == "return" or any(r in live for r in op.results):
            kept.append(op)
            live.update(op.operands)
    func.ops = list(reversed(kept))


ALL_KINDS = ("rmsnorm", "swiglu", "rope", "softmax_dot", "attention_step", "rmsnorm_rows", "rope_rows", "attention", "cross_entropy",
             "linear", "linear_group")


def fuse_clusters(func, kinds=ALL_KINDS):
    """Rewrites, in place, the operator clusters test/llama.py traces into fused operators:

      emi.rmsnorm  w * (x * (1 / sqrt(dot(x, x) / n + eps)))           (llama.py:6-10), also with
                   rsqrt in place of 1 / sqrt (EnzymeHLOOpt.cpp:14907-14923)
      emi.swiglu   a * (1 / (1 + exp(-a))) * b, or a * logistic(a) * b  (llama.py:21-28,229-231)
      emi.rope     reshape(dot_general(R, reshape(x, (P, 2)))) with constant 2x2 rotations R[P]
                   (llama.py:127-140,161-168)
      emi.softmax_dot  softmax(dot(K, q) / c) followed by the dot with V  (llama.py:13-18,193-204)
      emi.attention_step  the concatenation of emi.softmax_dot over consecutive head slices of
                   one query and one pair of caches (llama.py:178-209)
      emi.cross_entropy  sum(onehot(targets) * log_softmax(logits)) over the vocabulary, the one-hot built at run
                   time from integer targets (iota, compare EQ, convert or select): the loss after the classifier
                   of llama.py:236

    A cluster is fused only when none of its interior values is used outside it.  Returns
    the number of clusters fused per kind."""
    counts = {"rmsnorm": 0, "swiglu": 0, "rope": 0, "softmax_dot": 0, "attention_step": 0, "rmsnorm_rows": 0, "rope_rows": 0,
              "attention": 0, "cross_entropy": 0, "linear": 0, "linear_group": 0}
    matchers = [m for k, m in (("rmsnorm", _match_rmsnorm), ("swiglu", _match_swiglu), ("rope", _match_rope),
                               ("softmax_dot", _match_softmax_dot), ("attention_step", _match_heads),
                               ("rmsnorm_rows", _match_rmsnorm_rows), ("rope_rows", _match_rope_rows),
                               ("attention", _match_attention), ("cross_entropy", _match_cross_entropy)) if k in kinds]
    want_linear = "linear" in kinds
    changed = True
    while changed:
        changed = False
        defs = {r: op for op in func.ops for r in op.results}
        use = _users(func)
        rets = set(o for op in func.ops if op.name == "return" for o in op.operands)

        def d(name):
            return defs.get(name)

        d.types = {a: t for a, t in func.args}            # for matchers that need the type of a function argument
        for o_ in func.ops:
            for r_, t_ in zip(o_.results, o_.types):
                d.types[r_] = t_

        def through_broadcast(name):
            """The rank-0 value behind a broadcast_in_dim (or the name itself)."""
            op = d(name)
            if op is not None and op.name == "broadcast_in_dim" and not op.attrs["dims"]:
                return op.operands[0], op
            return name, None

        def only_used_by(names, inside):
            ids = set(id(o) for o in inside)
            for n in names:
                if n in rets:
                    return False
                for u in use.get(n, []):
                    if id(u) not in ids:
                        return False
            return True

        for op in func.ops:
            m = None
            for matcher in matchers:
                m = matcher(op, d, through_broadcast)
                if m is not None:
                    break
            if m is None:
                continue
            kind, new_op, interior = m
            interior = [o for o in interior if o.name != "constant"]
            inner_names = [r for o in interior if o is not op for r in o.results]
            if not only_used_by(inner_names, interior):
                continue
            # drop interior operators whose results nobody else needs; keep shared constants
            dead = set(id(o) for o in interior if o is not op)
            func.ops = [new_op if o is op else o for o in func.ops if id(o) not in dead]
            counts[kind] += 1
            changed = True
            break
    if want_linear:
        changed = True
        while changed:
            changed = False
            defs = {r: op for op in func.ops for r in op.results}
            use = _users(func)
            rets = set(o for op in func.ops if op.name == "return" for o in op.operands)
            types = {a: t for a, t in func.args}
            for op in func.ops:
                for r, t in zip(op.results, op.types):
                    types[r] = t
            for op in func.ops:
                m = _match_linear(op, defs.get, None, types.get)
                if m is None:
                    continue
                kind, new_op, interior = m
                inner = [o for o in interior if o is not op]
                if any(r in rets or any(u is not op for u in use.get(r, [])) for o in inner for r in o.results):
                    continue
                dead = set(id(o) for o in inner)
                func.ops = [new_op if o is op else o for o in func.ops if id(o) not in dead]
                if not inner:
                    counts["linear"] += 1
                changed = True
                break
    if want_linear and "linear_group" in kinds:
        counts["linear_group"] = _group_linears(func)
    _drop_dead(func)
    return counts


def _group_linears(func):
    """Sibling projections of one activation against weights of one shape (q, k, v of test/llama.py:149-157; w1, w3 of
    :224-227) become one `emi.linear_group` (operands x, w_1 .. w_n; results y_1 .. y_n; at most four): one grouped
    launch forward, one for the weight gradients and one summed launch for dX.  A member's weight must be a function
    argument or a slice / reshape chain of one, so that the operators that produce it can move in front of the
    group.  Returns the number of groups formed."""
    args = set(a for a, _ in func.args)
    types = {a: t for a, t in func.args}
    defs = {}
    for op in func.ops:
        for r, t in zip(op.results, op.types):
            defs[r] = op
            types[r] = t
    pos = {id(op): i for i, op in enumerate(func.ops)}

    def chain(name):
        out = []
        while name not in args:
            op = defs.get(name)
            if op is None or op.name not in ("slice", "reshape"):
                return None
            out.append(op)
            name = op.operands[0]
        return out[::-1]

    groups = {}
    for op in func.ops:
        if op.name == "emi.linear" and len(op.operands) == 2 and chain(op.operands[1]) is not None:
            xt = types[op.operands[0]]
            if len(xt.shape) < 2 or int(np.prod(xt.shape[:-1])) < 16:
                continue                 # the single-token step: each mat-vec streams its weight through its own kernel
            wt = types[op.operands[1]]
            groups.setdefault((op.operands[0], tuple(wt.shape), wt.dtype), []).append(op)
    formed = 0
    for members in groups.values():
        for k in range(0, len(members) - 1, 4):
            part = members[k:k + 4]
            if len(part) < 2:
                continue
            first = part[0]
            hoist, seen = [], set()
            for m in part[1:]:
                for c in chain(m.operands[1]):
                    if pos[id(c)] > pos[id(first)] and id(c) not in seen:
                        seen.add(id(c))
                        hoist.append(c)
            new = Op("emi.linear_group", [r for m in part for r in m.results], [first.operands[0]] + [m.operands[1] for m in part], {},
                     [t for m in part for t in m.types])
            drop = set(id(m) for m in part[1:]) | seen
            out = []
            for o in func.ops:
                if o is first:
                    out.extend(hoist)
                    out.append(new)
                elif id(o) not in drop:
                    out.append(o)
            func.ops = out
            pos = {id(op): i for i, op in enumerate(func.ops)}
            formed += 1
    return formed


def _fold_selects(func):
    """The operator list `Executable.run` walks: `reshape(slice(w, [i:i+1, 0:, ...]))` of a stacked function argument
    (`wq[i, :, :]`, test/llama.py:149) becomes `emi.select` {index}, which the tape differentiates in place (the
    slice's gradient is written straight into slice i of one buffer shaped like the stack).  The printed and the
    symbolic forms keep slice + reshape."""
    arg_t = {a: t for a, t in func.args}
    use = _users(func)
    rets = set(o for op in func.ops if op.name == "return" for o in op.operands)
    out, dropped = [], {}
    for op in func.ops:
        if op.name == "slice" and op.operands[0] in arg_t and op.results[0] not in rets:
            t = arg_t[op.operands[0]]
            a = op.attrs
            users = use.get(op.results[0], [])
            if (len(t.shape) >= 2 and len(users) == 1 and users[0].name == "reshape" and all(st == 1 for st in a["stride"])
                    and a["limit"][0] == a["start"][0] + 1 and list(a["start"][1:]) == [0] * (len(t.shape) - 1)
                    and list(a["limit"][1:]) == list(t.shape[1:]) and tuple(users[0].types[0].shape) == tuple(t.shape[1:])):
                dropped[op.results[0]] = (op.operands[0], a["start"][0])
                continue
        if op.name == "reshape" and op.operands[0] in dropped:
            w, i = dropped[op.operands[0]]
            out.append(Op("emi.select", op.results, [w], {"index": i}, op.types))
            continue
        out.append(op)
    return out


def _fuse_blocks(run_ops, func):
    """On the operator list `Executable.run` walks, the two sub-blocks of a decoder layer become the operators that apply
    their elementwise parts in GEMM and attention epilogues (`ops.ffn`, `ops.attention_block`):
      linear_group(x; w1, w3) -> swiglu -> linear(g, w2 [, r])               =>  emi.ffn
      linear_group(x; wq, wk, wv) -> rope_rows(q), rope_rows(k) -> attention  =>  emi.attention_block
    when every interior value has that one use (test/llama.py:149-209, 224-233).  The printed and the symbolic forms
    keep the separate clusters."""
    rets = set(o for op in func.ops if op.name == "return" for o in op.operands)
    use = {}
    for op in run_ops:
        for o in op.operands:
            use.setdefault(o, []).append(op)
    producer = {r: op for op in run_ops for r in op.results}

    def only_use(name, user):
        return name not in rets and len(use.get(name, [])) == 1 and use[name][0] is user

    drop, place = set(), {}
    for op in run_ops:
        if op.name == "emi.linear" and producer.get(op.operands[0]) is not None and producer[op.operands[0]].name == "emi.swiglu":
            sg = producer[op.operands[0]]
            ga, gb = producer.get(sg.operands[0]), producer.get(sg.operands[1])
            if (ga is not None and ga is gb and ga.name == "emi.linear_group" and len(ga.results) == 2 and sg.operands[0] != sg.operands[1]
                    and only_use(sg.results[0], op) and only_use(sg.operands[0], sg) and only_use(sg.operands[1], sg)
                    and id(ga) not in drop):
                ia, ib = ga.results.index(sg.operands[0]), ga.results.index(sg.operands[1])
                operands = [ga.operands[0], ga.operands[1 + ia], ga.operands[1 + ib], op.operands[1]] + list(op.operands[2:])
                place[id(op)] = Op("emi.ffn", op.results, operands, {}, op.types)
                drop.update((id(ga), id(sg)))
        if op.name == "emi.attention" and op.attrs.get("causal") is not None:
            rq, rk, g = (producer.get(o) for o in op.operands)
            if (rq is not None and rk is not None and g is not None and rq.name == "emi.rope_rows" and rk.name == "emi.rope_rows"
                    and rq is not rk and g.name == "emi.linear_group" and len(g.results) == 3 and producer.get(rq.operands[0]) is g
                    and producer.get(rk.operands[0]) is g and id(g) not in drop
                    and g.results.index(rq.operands[0]) == 0 and g.results.index(rk.operands[0]) == 1 and op.operands[2] == g.results[2]
                    and rq.attrs["heads"] == rk.attrs["heads"] == op.attrs["heads"]
                    and np.array_equal(rq.attrs["table"], rk.attrs["table"])
                    and only_use(rq.results[0], op) and only_use(rk.results[0], op) and only_use(g.results[0], rq)
                    and only_use(g.results[1], rk) and only_use(g.results[2], op)):
                attrs = {"table": rq.attrs["table"], "heads": op.attrs["heads"], "scale": op.attrs["scale"], "causal": op.attrs["causal"]}
                place[id(op)] = Op("emi.attention_block", op.results, list(g.operands), attrs, op.types)
                drop.update((id(g), id(rq), id(rk)))
    if not place:
        return run_ops
    return [place.get(id(op), op) for op in run_ops if id(op) not in drop]


def _match_rmsnorm(op, d, tb):
    # root: a product of three factors, (w * x) * bcast(ss) or w * (x * bcast(ss)) in any
    # operand order, ss = 1 / sqrt(dot(x, x) / n + eps) or rsqrt(...)
    if op.name != "multiply":
        return None
    for ii in (0, 1):
        inner = d(op.operands[ii])
        if inner is None or inner.name != "multiply":
            continue
        leaves = [op.operands[1 - ii]] + list(inner.operands)
        for si, leaf in enumerate(leaves):
            ss_name, bc = tb(leaf)
            if bc is None:
                continue
            ss = d(ss_name)
            if ss is None:
                continue
            interior = [op, inner, bc, ss]
            if ss.name == "rsqrt":
                arg = d(ss.operands[0])
            elif ss.name == "divide" and _splat(d(ss.operands[0])) == 1.0:
                sq = d(ss.operands[1])
                if sq is None or sq.name != "sqrt":
                    continue
                interior.append(sq)
                arg = d(sq.operands[0])
            else:
                continue
            if arg is None or arg.name != "add":
                continue
            eps = mean = None
            for ei in (0, 1):
                e = _splat(d(arg.operands[ei]))
                if e is not None:
                    eps, mean = e, d(arg.operands[1 - ei])
            if eps is None or mean is None or mean.name != "divide":
                continue
            n = _splat(d(mean.operands[1]))
            dot = d(mean.operands[0])
            if n is None or dot is None or dot.name != "dot_general":
                continue
            if dot.operands[0] != dot.operands[1] or dot.attrs["batch_a"] or len(dot.attrs["contract_a"]) != 1:
                continue
            x = dot.operands[0]
            rest = [l for k, l in enumerate(leaves) if k != si]
            if x not in rest:
                continue
            rest.remove(x)
            w = rest[0]
            xt = op.types[0]
            if len(xt.shape) != 1 or n != float(xt.shape[0]):
                continue
            interior += [arg, mean, dot]
            return "rmsnorm", Op("emi.rmsnorm", op.results, [x, w], {"eps": eps}, op.types), interior
    return None


def _match_sigmoid(name, d, tb):
    """name = logistic(a) or 1 / (1 + exp(-a)): returns (a, interior ops) or None."""
    s = d(name)
    if s is None:
        return None
    if s.name == "logistic":
        return s.operands[0], [s]
    if s.name != "divide":
        return None
    num, nbc = tb(s.operands[0])
    if _splat(d(num)) != 1.0:
        return None
    den = d(s.operands[1])
    if den is None or den.name != "add":
        return None
    for oi in (0, 1):
        one, obc = tb(den.operands[oi])
        ex = d(den.operands[1 - oi])
        if _splat(d(one)) != 1.0 or ex is None or ex.name != "exponential":
            continue
        ng = d(ex.operands[0])
        if ng is None or ng.name != "negate":
            continue
        interior = [s, den, ex, ng] + [b for b in (nbc, obc) if b is not None]
        return ng.operands[0], interior
    return None


def _match_swiglu(op, d, tb):
    # root: multiply(multiply(a, sigmoid(a)), b) in any operand order
    if op.name != "multiply":
        return None
    for bi in (0, 1):
        b, inner = op.operands[bi], d(op.operands[1 - bi])
        if inner is None or inner.name != "multiply":
            continue
        for ai in (0, 1):
            a = inner.operands[ai]
            sg = _match_sigmoid(inner.operands[1 - ai], d, tb)
            if sg is None or sg[0] != a:
                continue
            return "swiglu", Op("emi.swiglu", op.results, [a, b], {}, op.types), [op, inner] + sg[1]
    return None


def _match_softmax_dot(op, d, tb):
    # root: dot_general(att, V) or dot_general(V, att) contracting the sequence index, with
    # att = e / bcast(sum(e)), e = exp(s - bcast(max(s))), s = dot_general(K, q) / c  (or * c)
    if op.name != "dot_general" or op.attrs["batch_a"] or len(op.attrs["contract_a"]) != 1:
        return None
    for ai in (0, 1):
        att, v = d(op.operands[ai]), op.operands[1 - ai]
        if att is None or att.name != "divide":
            continue
        e = d(att.operands[0])
        sum_name, sbc = tb(att.operands[1])
        sm = d(sum_name)
        if e is None or e.name != "exponential" or sbc is None or sm is None or sm.name != "reduce":
            continue
        if sm.attrs["body"] != "add" or sm.operands[0] != att.operands[0]:
            continue
        sub = d(e.operands[0])
        if sub is None or sub.name != "subtract":
            continue
        s_name = sub.operands[0]
        max_name, mbc = tb(sub.operands[1])
        mx = d(max_name)
        if mbc is None or mx is None or mx.name != "reduce" or mx.attrs["body"] != "maximum" or mx.operands[0] != s_name:
            continue
        s = d(s_name)
        if s is None or s.name not in ("divide", "multiply"):
            continue
        c_name, cbc = tb(s.operands[1])
        c = _splat(d(c_name))
        sdot = d(s.operands[0])
        if c is None or sdot is None or sdot.name != "dot_general" or sdot.attrs["batch_a"]:
            continue
        scale = 1.0 / c if s.name == "divide" else c
        # K [S, d] . q [d] -> [S]
        if sdot.attrs["contract_a"] != [1] or sdot.attrs["contract_b"] != [0]:
            continue
        k, q = sdot.operands
        seq_type = s.types[0]
        if len(seq_type.shape) != 1:
            continue
        # att [S] . V [S, d] -> [d]: contraction over index 0 of V
        att_side, v_side = ("contract_a", "contract_b") if ai == 0 else ("contract_b", "contract_a")
        if op.attrs[att_side] != [0] or op.attrs[v_side] != [0]:
            continue
        interior = [op, att, e, sbc, sm, sub, mbc, mx, s, sdot] + ([cbc] if cbc is not None else [])
        return ("softmax_dot", Op("emi.softmax_dot", op.results, [q, k, v], {"scale": scale}, op.types), interior)
    return None


def _per_row_source(name, d, through=()):
    """Follows `name`, a value of shape rows + (V,), back through the broadcast_in_dim / reshape operators that only
    spread a per-row value along the last axis (shapes rows, rows + (1,), rows + (V,)) and through the unary
    operators named in `through`.  Returns (source name, operators passed, unary names passed) or None."""
    ty = d.types.get(name)
    if ty is None or not ty.shape:
        return None
    rows = tuple(ty.shape[:-1])
    passed, unary = [], []
    while True:
        op = d(name)
        if op is None:
            break
        if op.name in through:
            passed.append(op)
            unary.append(op.name)
            name = op.operands[0]
            continue
        if op.name not in ("broadcast_in_dim", "reshape"):
            break
        src = d.types.get(op.operands[0])
        if src is None or tuple(src.shape) not in (rows, rows + (1,)):
            break
        if op.name == "broadcast_in_dim" and list(op.attrs["dims"]) != list(range(len(src.shape))):
            break
        passed.append(op)
        name = op.operands[0]
    if not passed or tuple(d.types[name].shape) not in (rows, rows + (1,)):
        return None
    return name, passed, unary


def _is_class_index(name, d):
    """True (with the operators passed) when `name` holds, at every position, its index along the last axis: an iota
    over that axis, or the constant it folds to, possibly broadcast over the leading axes."""
    ty = d.types.get(name)
    passed = []
    while True:
        op = d(name)
        if op is None or ty is None:
            return None
        V = ty.shape[-1]
        if op.name == "iota":
            return passed + [op] if op.attrs["dim"] == len(op.types[0].shape) - 1 and op.types[0].shape[-1] == V else None
        if op.name == "constant":
            v = np.asarray(op.attrs["value"])
            if v.dtype.kind not in "iu" or v.shape[-1:] != (V,):
                return None
            return passed if np.array_equal(v.reshape(-1, V), np.broadcast_to(np.arange(V), (v.size // V, V))) else None
        if op.name not in ("broadcast_in_dim", "reshape"):
            return None
        src = d.types.get(op.operands[0])
        if src is None or not src.shape or src.shape[-1] != V or any(x != 1 for x in src.shape[:-1]):
            return None
        if op.name == "broadcast_in_dim":
            dims = list(op.attrs["dims"])
            if dims[-1] != len(op.types[0].shape) - 1:
                return None
        passed.append(op)
        name = op.operands[0]


def _log_softmax(logp_name, d):
    """(logits, interior operators) when `logp_name` is jax.nn.log_softmax over the last axis:
    shifted - spread(log(reduce-add(exp(shifted)))) with shifted = logits - spread(reduce-max(logits))."""
    logp = d(logp_name)
    if logp is None or logp.name != "subtract":
        return None
    shifted = d(logp.operands[0])
    norm = _per_row_source(logp.operands[1], d, through=("log",))
    if shifted is None or shifted.name != "subtract" or norm is None or norm[2] != ["log"]:
        return None
    sm = d(norm[0])
    if sm is None or sm.name != "reduce" or sm.attrs["body"] != "add" or _splat(d(sm.operands[1])) != 0.0:
        return None
    ex = d(sm.operands[0])
    rank = len(shifted.types[0].shape)
    if ex is None or ex.name != "exponential" or ex.operands[0] != logp.operands[0] or list(sm.attrs["dims"]) != [rank - 1]:
        return None
    logits = shifted.operands[0]
    top = _per_row_source(shifted.operands[1], d)
    if top is None:
        return None
    mx = d(top[0])
    if mx is None or mx.name != "reduce" or mx.attrs["body"] != "maximum" or mx.operands[0] != logits or \
            list(mx.attrs["dims"]) != [rank - 1] or _splat(d(mx.operands[1])) != -math.inf:
        return None
    if d.types[logits].dtype not in ("f32", "bf16"):
        return None
    return logits, [logp, shifted, sm, ex, mx] + norm[1] + top[1]


def _match_cross_entropy(op, d, tb):
    # Two spellings of minus the per-row cross-entropy of jax.nn.log_softmax(logits) against run-time integer targets:
    # (1) root: reduce-add over the last axis of onehot * logp (either order) or select(eq, logp, 0), with
    #       eq     = compare EQ of the targets spread along the last axis and the class index along it
    #       onehot = convert(eq)                                     (jax.nn.one_hot)
    # (2) root: gather(logp, targets[..., None]) picking one class per row (jnp.take_along_axis): every leading index a
    #     batching index of operand and indices, the last one collapsed, slices of one element.
    # A target outside [0, V) gives 0, as the kernel does.
    if op.name == "gather":
        a = op.attrs
        logp_name, idx_name = op.operands
        lt, it = d.types.get(logp_name), d.types.get(idx_name)
        if lt is None or it is None or len(lt.shape) < 2 or it.dtype != "i32":
            return None
        R = len(lt.shape) - 1
        rows = tuple(lt.shape[:-1])
        lead = list(range(R))
        if not (tuple(it.shape) == rows + (1,) and a["index_vector_dim"] == R and a["collapsed_slice_dims"] == [R]
                and a["operand_batching_dims"] == lead and a.get("start_indices_batching_dims", []) == lead
                and a["start_index_map"] == [R] and a["offset_dims"] == [] and a["slice_sizes"] == [1] * (R + 1)
                and tuple(op.types[0].shape) == rows):
            return None
        ls = _log_softmax(logp_name, d)
        if ls is None:
            return None
        src = d(idx_name)                       # targets[..., None]: a reshape or broadcast of the [rows] targets
        passed = []
        targets = idx_name
        if src is not None and src.name in ("reshape", "broadcast_in_dim") and tuple(d.types[src.operands[0]].shape) == rows:
            targets, passed = src.operands[0], [src]
        return ("cross_entropy", Op("emi.cross_entropy", op.results, [ls[0], targets], {"negated": True}, op.types),
                [op] + passed + ls[1])
    if op.name != "reduce" or op.attrs["body"] != "add" or _splat(d(op.operands[1])) != 0.0:
        return None
    prod = d(op.operands[0])
    if prod is None or not prod.types[0].shape or list(op.attrs["dims"]) != [len(prod.types[0].shape) - 1]:
        return None
    interior = [op, prod]
    if prod.name == "multiply":
        for oi in (0, 1):
            cv = d(prod.operands[oi])
            if cv is not None and cv.name == "convert" and d(cv.operands[0]) is not None and d(cv.operands[0]).name == "compare":
                eq, logp_name = d(cv.operands[0]), prod.operands[1 - oi]
                interior.append(cv)
                break
        else:
            return None
    elif prod.name == "select":
        eq, logp_name = d(prod.operands[0]), prod.operands[1]
        if eq is None or eq.name != "compare" or _splat(d(prod.operands[2])) != 0.0:
            return None
    else:
        return None
    if eq.attrs["direction"] != "EQ":
        return None
    interior.append(eq)
    targets = None
    for ti in (0, 1):
        src = _per_row_source(eq.operands[ti], d)
        idx = _is_class_index(eq.operands[1 - ti], d)
        if src is not None and idx is not None and d.types[src[0]].dtype == "i32":
            targets = src[0]
            interior += src[1] + idx
            break
    if targets is None:
        return None
    ls = _log_softmax(logp_name, d)
    if ls is None:
        return None
    return ("cross_entropy", Op("emi.cross_entropy", op.results, [ls[0], targets], {"negated": True}, op.types), interior + ls[1])


def _bcast(name, d, dims=None):
    """(operand, op) when `name` is a broadcast_in_dim (with the given dims), else (None, None)."""
    op = d(name)
    if op is not None and op.name == "broadcast_in_dim" and (dims is None or list(op.attrs["dims"]) == list(dims)):
        return op.operands[0], op
    return None, None


def _match_rmsnorm_rows(op, d, tb):
    # batched form: (x * bcast(1 / sqrt(sum(x * x, last) / n + eps))) * bcast(w, last), x [..., n]
    if op.name != "multiply":
        return None
    rank = len(op.types[0].shape)
    if rank < 2:
        return None
    lead = list(range(rank - 1))
    for wi in (0, 1):
        w, wb = _bcast(op.operands[wi], d, [rank - 1])
        inner = d(op.operands[1 - wi])
        if wb is None or inner is None or inner.name != "multiply":
            continue
        for xi in (0, 1):
            x = inner.operands[xi]
            r_name, rb = _bcast(inner.operands[1 - xi], d, lead)
            if rb is None:
                continue
            ss = d(r_name)
            if ss is None:
                continue
            interior = [op, wb, inner, rb, ss]
            if ss.name == "rsqrt":
                arg = d(ss.operands[0])
            elif ss.name == "divide" and _splat(d(tb(ss.operands[0])[0])) == 1.0:
                sq = d(ss.operands[1])
                if sq is None or sq.name != "sqrt":
                    continue
                interior += [sq] + [o for o in [tb(ss.operands[0])[1]] if o is not None]
                arg = d(sq.operands[0])
            else:
                continue
            if arg is None or arg.name != "add":
                continue
            eps = mean = None
            for ei in (0, 1):
                en, eb = tb(arg.operands[ei])
                e = _splat(d(en))
                if e is not None:
                    eps, mean = e, d(arg.operands[1 - ei])
                    interior += [o for o in [eb] if o is not None]
            if eps is None or mean is None or mean.name != "divide":
                continue
            nn, nbc = tb(mean.operands[1])
            n = _splat(d(nn))
            red = d(mean.operands[0])
            if n is None or red is None or red.name != "reduce" or red.attrs["body"] != "add" or list(red.attrs["dims"]) != [rank - 1]:
                continue
            sq2 = d(red.operands[0])
            if sq2 is None or sq2.name != "multiply" or sq2.operands != [x, x] or n != float(op.types[0].shape[-1]):
                continue
            interior += [arg, mean, red, sq2] + [o for o in [nbc] if o is not None]
            return "rmsnorm_rows", Op("emi.rmsnorm_rows", op.results, [x, w], {"eps": eps}, op.types), interior
    return None


def _match_rope_rows(op, d, tb):
    # reshape(concat([reshape(x0 c - x1 s), reshape(x0 s + x1 c)], last)) with x0 / x1 the even / odd
    # elements of reshape(x, [B, S, h, P, 2]) and c, s constant tables [S, P] broadcast over dims (1, 3)
    if op.name != "reshape" or len(op.types[0].shape) != 3:
        return None
    cat = d(op.operands[0])
    if cat is None or cat.name != "concatenate" or cat.attrs["dim"] != 4 or len(cat.operands) != 2:
        return None
    r0, r1 = d(cat.operands[0]), d(cat.operands[1])
    if r0 is None or r1 is None or r0.name != "reshape" or r1.name != "reshape":
        return None
    o0, o1 = d(r0.operands[0]), d(r1.operands[0])
    if o0 is None or o1 is None or o0.name != "subtract" or o1.name != "add":
        return None
    m = [d(o) for o in (o0.operands[0], o0.operands[1], o1.operands[0], o1.operands[1])]
    if any(t is None or t.name != "multiply" for t in m):
        return None
    (x0, cb0), (x1, sb0), (x0b, sb1), (x1b, cb1) = (t.operands for t in m)
    if x0 != x0b or x1 != x1b or cb0 != cb1 or sb0 != sb1:
        return None
    cn, cbc = _bcast(cb0, d, [1, 3])
    sn, sbc = _bcast(sb0, d, [1, 3])
    if cbc is None or sbc is None:
        return None
    extra = []

    def table_const(name):
        op_ = d(name)
        if op_ is not None and op_.name == "convert":           # fp32 tables converted to the storage dtype
            extra.append(op_)
            op_ = d(op_.operands[0])
        return op_

    cconst, sconst = table_const(cn), table_const(sn)
    if cconst is None or sconst is None or cconst.name != "constant" or sconst.name != "constant":
        return None
    e0, e1 = d(x0), d(x1)
    if e0 is None or e1 is None or e0.name != "reshape" or e1.name != "reshape":
        return None
    s0, s1 = d(e0.operands[0]), d(e1.operands[0])
    if s0 is None or s1 is None or s0.name != "slice" or s1.name != "slice" or s0.operands != s1.operands:
        return None
    xr = d(s0.operands[0])
    if xr is None or xr.name != "reshape" or len(xr.types[0].shape) != 5 or xr.types[0].shape[4] != 2:
        return None
    B, S, h, P, _ = xr.types[0].shape
    if s0.attrs["start"] != [0, 0, 0, 0, 0] or s0.attrs["limit"] != [B, S, h, P, 1] or s1.attrs["start"] != [0, 0, 0, 0, 1] or \
            s1.attrs["limit"] != [B, S, h, P, 2]:
        return None
    c, s_ = np.asarray(cconst.attrs["value"], dtype=np.float64), np.asarray(sconst.attrs["value"], dtype=np.float64)
    if c.shape != (S, P) or s_.shape != (S, P) or np.max(np.abs(c * c + s_ * s_ - 1.0)) > 2e-2:
        return None
    if tuple(op.types[0].shape) != (B, S, h * 2 * P):
        return None
    table = np.stack([c, s_], axis=2).astype(np.float32)                      # [S, P, 2]
    # the converts of the tables may serve other clusters too: they stay until nothing uses them
    interior = [op, cat, r0, r1, o0, o1] + m + [cbc, sbc, e0, e1, s0, s1, xr]
    return "rope_rows", Op("emi.rope_rows", op.results, [xr.operands[0]], {"table": table, "heads": h}, op.types), interior


def _match_attention(op, d, tb):
    # reshape(transpose(dot(P, Vh))) with P = softmax over keys of select(mask, dot(Qh, Kh) / c, -inf),
    # Xh = transpose(reshape(X, [B, S, h, d]), [0, 2, 1, 3]); mask constant, lower triangular or all true
    if op.name != "reshape" or len(op.types[0].shape) != 3:
        return None
    tr = d(op.operands[0])
    if tr is None or tr.name != "transpose" or list(tr.attrs["perm"]) != [0, 2, 1, 3]:
        return None
    pv = d(tr.operands[0])
    if pv is None or pv.name != "dot_general" or pv.attrs["batch_a"] != [0, 1] or pv.attrs["batch_b"] != [0, 1] or \
            pv.attrs["contract_a"] != [3] or pv.attrs["contract_b"] != [2]:
        return None
    p, vh = d(pv.operands[0]), d(pv.operands[1])
    if p is None or p.name != "divide":
        return None
    e = d(p.operands[0])
    sum_name, sbc = _bcast(p.operands[1], d, [0, 1, 2])
    sm = d(sum_name) if sbc is not None else None
    if e is None or e.name != "exponential" or sm is None or sm.name != "reduce" or sm.attrs["body"] != "add" or \
            list(sm.attrs["dims"]) != [3] or sm.operands[0] != p.operands[0]:
        return None
    sub = d(e.operands[0])
    if sub is None or sub.name != "subtract":
        return None
    s_name = sub.operands[0]
    max_name, mbc = _bcast(sub.operands[1], d, [0, 1, 2])
    mx = d(max_name) if mbc is not None else None
    if mx is None or mx.name != "reduce" or mx.attrs["body"] != "maximum" or list(mx.attrs["dims"]) != [3] or mx.operands[0] != s_name:
        return None
    interior = [op, tr, pv, p, e, sbc, sm, sub, mbc, mx]
    s = d(s_name)
    causal = False
    if s is not None and s.name == "select":
        fill_name, fill_bc = tb(s.operands[2])
        mask = d(s.operands[0])
        mask_bc = None
        if mask is not None and mask.name == "broadcast_in_dim" and list(mask.attrs["dims"]) == [2, 3]:
            mask_bc, mask = mask, d(mask.operands[0])                   # a [S, S] mask shared by every batch and head
        if mask is None or mask.name != "constant" or _splat(d(fill_name)) != -np.inf:
            return None
        interior += [o for o in (fill_bc, mask_bc) if o is not None]
        mv = np.asarray(mask.attrs["value"])
        S = mv.shape[-1]
        m2 = mv.reshape(-1, S, S)
        if not np.all(m2 == m2[0]):
            return None
        if np.array_equal(m2[0], np.tril(np.ones((S, S), dtype=bool))):
            causal = True
        elif not np.all(m2[0]):
            return None
        interior.append(s)
        s = d(s.operands[1])
    if s is None or s.name not in ("divide", "multiply"):
        return None
    c_name, cbc = tb(s.operands[1])
    c = _splat(d(c_name))
    qk = d(s.operands[0])
    if c is None or qk is None or qk.name != "dot_general" or qk.attrs["batch_a"] != [0, 1] or qk.attrs["batch_b"] != [0, 1] or \
            qk.attrs["contract_a"] != [3] or qk.attrs["contract_b"] != [3]:
        return None
    scale = 1.0 / c if s.name == "divide" else c
    interior += [s, qk] + ([cbc] if cbc is not None else [])
    srcs = []
    for hname in (qk.operands[0], qk.operands[1], pv.operands[1]):
        ht = d(hname)
        if ht is None or ht.name != "transpose" or list(ht.attrs["perm"]) != [0, 2, 1, 3]:
            return None
        rs = d(ht.operands[0])
        if rs is None or rs.name != "reshape" or len(rs.types[0].shape) != 4:
            return None
        interior += [ht, rs]
        srcs.append(rs.operands[0])
    B, h, S, hd = qk.types[0].shape[0], qk.types[0].shape[1], qk.types[0].shape[2], d(qk.operands[0]).types[0].shape[3]
    if tuple(op.types[0].shape) != (B, S, h * hd):
        return None
    new = Op("emi.attention", op.results, srcs, {"scale": scale, "heads": h, "causal": causal}, op.types)
    return "attention", new, interior


def _linear_form(op, types):
    """(x, w) when dot_general `op` is y = x . w^T for a weight w [out, in]: either x[..., in]
    contracted over its last index with index 1 of w (batched form), or w contracted over
    index 1 with a vector x[in] (the step's `w @ x`, test/llama.py:149-157)."""
    if op is None or op.name != "dot_general" or op.attrs["batch_a"] or len(op.attrs["contract_a"]) != 1:
        return None
    a, b_ = op.operands
    ta, tb_ = types(a), types(b_)
    if ta is None or tb_ is None or ta.dtype not in ("f32", "bf16"):
        return None
    ca, cb = op.attrs["contract_a"][0], op.attrs["contract_b"][0]
    if len(tb_.shape) == 2 and cb == 1 and ca == len(ta.shape) - 1 and len(ta.shape) >= 1:
        return a, b_
    if len(ta.shape) == 2 and ca == 1 and len(tb_.shape) == 1 and cb == 0:
        return b_, a
    return None


def _match_linear(op, d, tb, types=None):
    # root: add(r, dot) with the product used only here -> projection with the residual added in
    # the GEMM epilogue (test/llama.py:211-215,231-233); or a bare projection
    if op.name == "add":
        for di in (0, 1):
            inner = d(op.operands[di])
            if inner is not None and inner.name == "emi.linear" and len(inner.operands) == 2:
                new = Op("emi.linear", op.results, list(inner.operands) + [op.operands[1 - di]], {}, op.types)
                return "linear", new, [op, inner]
        return None
    lf = _linear_form(op, types)
    if lf is None:
        return None
    return "linear", Op("emi.linear", op.results, [lf[0], lf[1]], {}, op.types), [op]


def _match_rope(op, d, tb):
    # root: reshape(dot_general(R [P,2,2] constant, reshape(x, [P,2]), batch [0]x[0], contract [2]x[1])) -> [2P]
    if op.name != "reshape" or len(op.types[0].shape) != 1:
        return None
    dot = d(op.operands[0])
    if dot is None or dot.name != "dot_general" or dot.attrs["batch_a"] != [0] or dot.attrs["batch_b"] != [0]:
        return None
    if dot.attrs["contract_a"] != [2] or dot.attrs["contract_b"] != [1]:
        return None
    rot, inner = d(dot.operands[0]), d(dot.operands[1])
    if rot is None or rot.name != "constant" or inner is None or inner.name != "reshape":
        return None
    R = np.asarray(rot.attrs["value"], dtype=np.float64)
    P = op.types[0].shape[0] // 2
    if R.shape != (P, 2, 2) or tuple(inner.types[0].shape) != (P, 2):
        return None
    c, s_ = R[:, 0, 0], R[:, 1, 0]
    if not (np.array_equal(R[:, 1, 1], c) and np.array_equal(R[:, 0, 1], -s_)):
        return None
    if np.max(np.abs(c * c + s_ * s_ - 1.0)) > 1e-5:
        return None
    table = np.stack([c, s_], axis=1).astype(np.float32)
    return "rope", Op("emi.rope", op.results, [inner.operands[0]], {"table": table}, op.types), [op, dot, inner]


def _match_heads(op, d, tb):
    # root: concatenate(dim 0) of emi.softmax_dot(q_h, K_h, V_h) over head slices h = 0..n-1
    if op.name != "concatenate" or op.attrs["dim"] != 0 or len(op.operands) < 2:
        return None
    heads = [d(o) for o in op.operands]
    if any(h is None or h.name != "emi.softmax_dot" for h in heads):
        return None
    scale = heads[0].attrs["scale"]
    q = kc = vc = None
    hs = heads[0].types[0].shape[0]
    interior = [op]
    for h, sd in enumerate(heads):
        if sd.attrs["scale"] != scale or tuple(sd.types[0].shape) != (hs,):
            return None
        sl = [d(o) for o in sd.operands]
        if any(x is None or x.name != "slice" for x in sl):
            return None
        qs, ks, vs = sl
        if qs.attrs["start"] != [h * hs] or qs.attrs["limit"] != [(h + 1) * hs] or qs.attrs["stride"] != [1]:
            return None
        for cs in (ks, vs):
            if len(cs.attrs["start"]) != 2 or cs.attrs["start"][0] != 0 or cs.attrs["stride"] != [1, 1]:
                return None
            if cs.attrs["start"][1] != h * hs or cs.attrs["limit"][1] != (h + 1) * hs:
                return None
        if h == 0:
            q, kc, vc = qs.operands[0], ks.operands[0], vs.operands[0]
            rows = ks.attrs["limit"][0]
        if (qs.operands[0], ks.operands[0], vs.operands[0]) != (q, kc, vc):
            return None
        if ks.attrs["limit"][0] != rows or vs.attrs["limit"][0] != rows:
            return None
        interior += [sd, qs, ks, vs]
    n = len(heads)
    if tuple(op.types[0].shape) != (n * hs,):
        return None
    # the caches must be exactly [rows, n * hs] and the query [n * hs]: checked when run
    new = Op("emi.attention_step", op.results, [q, kc, vc], {"scale": scale, "heads": n, "rows": rows}, op.types)
    return "attention_step", new, interior


# ---------------------------------------------------------------------------
# executor
# ---------------------------------------------------------------------------

class Executable:
    """A parsed module ready to run on one device."""

    def __init__(self, text, fuse=True):
        """fuse: True (all clusters), False (none), or a tuple of cluster kinds."""
        self.funcs = parse_module(text)
        self.fused = {}
        for f in self.funcs.values():
            fold_constants(f)
            if fuse:
                kinds = fuse if isinstance(fuse, (tuple, list)) else ALL_KINDS
                for k, v in fuse_clusters(f, kinds).items():
                    if v:
                        self.fused[k] = self.fused.get(k, 0) + v
        self._consts = {}
        for f in self.funcs.values():
            f.run_ops = _fuse_blocks(_fold_selects(f), f) if fuse else f.ops

    def signature(self, fn="main"):
        f = self._func(fn)
        return [t for _, t in f.args], list(f.result_types)

    def _func(self, fn):
        if fn not in self.funcs:
            raise AssertionError("Could not find desired function %s options are %s" % (fn, sorted(self.funcs)))
        return self.funcs[fn]

    def _const(self, op, device):
        key = (id(op), str(device))
        hit = self._consts.get(key)
        if hit is None:
            ty = op.types[0]
            host = torch.from_numpy(np.ascontiguousarray(op.attrs["value"]).reshape(-1)).reshape(ty.shape)
            hit = self._consts[key] = host.to(TORCH_DTYPES[ty.dtype]).to(device)       # trace-time constant upload
        return hit

    def run(self, args, fn="main"):
        f = self._func(fn)
        if len(args) != len(f.args):
            raise ValueError("%s takes %d arguments, %d given" % (fn, len(f.args), len(args)))
        env = {}
        device = None
        if getattr(f, "defs", None) is None:
            f.defs = {r: op for op in f.ops for r in op.results}
        for (name, ty), a in zip(f.args, args):
            if not isinstance(a, torch.Tensor):
                raise TypeError("argument %s is not a tensor" % name)
            if tuple(a.shape) != ty.shape or a.dtype != TORCH_DTYPES[ty.dtype]:
                raise ValueError("argument %s is %s/%s, the module wants %r" % (name, tuple(a.shape), a.dtype, ty))
            if not a.is_cuda:
                raise RuntimeError("argument %s is not in device memory: the HIP path has no CPU fallback" % name)
            device = a.device
            env[name] = a
        if device is None:
            device = torch.device("cuda", torch.cuda.current_device())
        for op in getattr(f, "run_ops", f.ops):
            if op.name == "return":
                return [env[o] for o in op.operands]
            outs = self._apply(f, op, [env[o] for o in op.operands], device)
            if len(outs) != len(op.results):
                raise RuntimeError("%s produced %d values for %d results" % (op.name, len(outs), len(op.results)))
            for r, v, ty in zip(op.results, outs, op.types):
                if v is not None and tuple(v.shape) != ty.shape:
                    raise RuntimeError("%s: result %s has shape %s, the text says %r" % (op.name, r, tuple(v.shape), ty))
                env[r] = v
        raise ParseError("function %s has no return" % fn)

    def _apply(self, f, op, xs, device):
        n = op.name
        if n == "constant":
            return [self._const(op, device)]
        if n in BINARY_OPS:
            return [H.binary(n, xs[0], xs[1])]
        if n in UNARY_OPS:
            return [H.unary(n, xs[0])]
        if n == "convert":
            dt = TORCH_DTYPES[op.types[0].dtype]
            return [xs[0] if xs[0].dtype == dt else H.convert(xs[0], dt)]
        if n == "reshape":
            x = xs[0] if xs[0].is_contiguous() else H.unary_copy(xs[0])      # a tracked copy: cotangents reach the view
            return [ops.reshape(x, op.types[0].shape)]
        if n == "transpose":
            return [H.transpose(xs[0], op.attrs["perm"])]
        if n == "broadcast_in_dim":
            return [H.broadcast_in_dim(xs[0], op.types[0].shape, op.attrs["dims"])]
        if n == "reduce":
            kind = op.attrs["body"]
            y = H.reduce(kind, xs[0], op.attrs["dims"])
            init = _splat(f.defs.get(op.operands[1]))
            if init is not None and ((kind == "add" and init == 0.0) or (kind == "maximum" and init == -math.inf)):
                return [y]
            return [H.binary(kind, y, xs[1])]
        if n == "dot_general":
            return [H.dot_general(xs[0], xs[1], op.attrs["batch_a"], op.attrs["batch_b"], op.attrs["contract_a"],
                                  op.attrs["contract_b"])]
        if n == "slice":
            return [H.slice_(xs[0], op.attrs["start"], op.attrs["limit"], op.attrs["stride"])]
        if n == "concatenate":
            return [H.concatenate(xs, op.attrs["dim"])]
        if n == "gather":
            names = {v: k for k, v in TORCH_DTYPES.items() if k != "ui32"}
            check_gather(op.attrs, TensorType(xs[0].shape, names[xs[0].dtype]), TensorType(xs[1].shape, names[xs[1].dtype]),
                         op.types[0])
            if xs[1].dtype != torch.int32:
                raise NotImplementedError("stablehlo.gather with %s indices (s32 wanted)" % xs[1].dtype)
            return [ops.embedding(xs[1].reshape(xs[1].shape[:-1]), xs[0])]
        if n == "iota":
            raise NotImplementedError("stablehlo.iota of type %r (integer iotas feeding masks are folded at parse time)" % op.types[0])
        if n == "compare":
            if not xs[0].is_floating_point():
                raise NotImplementedError("stablehlo.compare on integer operands that are not trace-time constants")
            return [H.compare(op.attrs["direction"], xs[0], xs[1])]
        if n == "select":
            return [H.select(xs[0], xs[1], xs[2])]
        if n == "pad":
            if _splat(f.defs.get(op.operands[1])) != 0.0:
                raise NotImplementedError("stablehlo.pad with a padding value other than a zero constant")
            return [H.pad(xs[0], op.attrs["low"], op.attrs["high"], op.attrs["interior"], op.types[0].shape)]
        if n == "call":
            return self.run(xs, op.attrs["callee"])
        if n == "custom_call":
            return self._custom_call(op, xs)
        if n == "emi.linear":
            x, w = _packed(xs[0]), _packed(xs[1])
            r = _packed(xs[2]) if len(xs) > 2 else None
            return [ops.matmul_nt(x, w, residual=r)]
        if n == "emi.linear_group":
            return list(ops.matmul_nt_group(_packed(xs[0]), [_packed(w) for w in xs[1:]]))
        if n == "emi.select":
            return [ops.select(xs[0], op.attrs["index"])]
        if n == "emi.ffn":
            x, w1, w3, w2 = (_packed(t) for t in xs[:4])
            return [ops.ffn(x, w1, w3, w2, residual=_packed(xs[4]) if len(xs) > 4 else None)]
        if n == "emi.attention_block":
            key = (id(op), "table", str(device))
            table = self._consts.get(key)
            if table is None:
                table = self._consts[key] = torch.from_numpy(op.attrs["table"]).to(device).contiguous()
            x, wq, wk, wv = (_packed(t) for t in xs)
            return [ops.attention_block(x, wq, wk, wv, op.attrs["heads"], scale=op.attrs["scale"], causal=op.attrs["causal"],
                                        table=table)]
        if n == "emi.rmsnorm_rows":
            x, w = _packed(xs[0]), _packed(xs[1])
            return [ops.rmsnorm(x, w, op.attrs["eps"])]
        if n == "emi.rope_rows":
            key = (id(op), "table", str(device))
            table = self._consts.get(key)
            if table is None:
                table = self._consts[key] = torch.from_numpy(op.attrs["table"]).to(device)
            return [ops.rope_rows(_packed(xs[0]), op.attrs["heads"], table)]
        if n == "emi.attention":
            q, k, v = (_packed(t) for t in xs)
            return [ops.attention(q, k, v, op.attrs["heads"], op.attrs["scale"], causal=op.attrs["causal"], layout="bshd")]
        if n == "emi.cross_entropy":
            z = _packed(xs[0])
            loss = ops.cross_entropy(z, xs[1].reshape(z.shape[:-1]).contiguous())          # fp32 per-row losses
            if op.attrs.get("negated"):
                loss = H.unary("negate", loss)
            dt = TORCH_DTYPES[op.types[0].dtype]
            if loss.dtype != dt:
                loss = H.convert(loss, dt)
            return [ops.reshape(loss, op.types[0].shape)]
        if n == "emi.rmsnorm":
            x, w = _packed(xs[0]), _packed(xs[1])
            return [ops.reshape(ops.rmsnorm(ops.reshape(x, (1, x.shape[0])), w, op.attrs["eps"]), tuple(x.shape))]
        if n == "emi.swiglu":
            return [ops.swiglu(_packed(xs[0]), _packed(xs[1]))]
        if n == "emi.rope":
            key = (id(op), "table", str(device))
            table = self._consts.get(key)
            if table is None:
                table = self._consts[key] = torch.from_numpy(op.attrs["table"]).to(device)
            return [ops.rotate_pairs(_packed(xs[0]), table)]
        if n == "emi.softmax_dot":
            q, k, v = xs
            return [ops.attention_step(_packed(q), _packed(k), _packed(v), 1, op.attrs["scale"])]
        if n == "emi.attention_step":
            q, k, v = xs
            heads, rows = op.attrs["heads"], op.attrs["rows"]
            if q.dim() != 1 or k.shape != (rows, q.shape[0]) or v.shape != k.shape:
                raise RuntimeError("attention cluster: query %s, caches %s / %s do not form %d heads over %d rows" %
                                   (tuple(q.shape), tuple(k.shape), tuple(v.shape), heads, rows))
            return [ops.attention_step(_packed(q), _packed(k), _packed(v), heads, op.attrs["scale"])]
        raise NotImplementedError("StableHLO operator '%s' is not supported by the HIP front end" % n)


def _custom_call_impl(self, op, xs):
    """Typed-FFI custom calls to this library's targets (the form `lower_to_custom_calls` prints),
    run through the same operators the matcher would have picked."""
    target, cfg = op.attrs["target"], op.attrs["config"]
    if target == "emi_rmsnorm_fwd":
        x, w = _packed(xs[0]), _packed(xs[1])
        y = ops.rmsnorm(ops.reshape(x, (-1, x.shape[-1])), w, cfg.get("eps", 1e-5))
        return [ops.reshape(y, tuple(x.shape))]
    if target == "emi_swiglu_fwd":
        return [ops.swiglu(_packed(xs[0]), _packed(xs[1]))]
    if target == "emi_gemm":
        a, b_ = _packed(xs[0]), _packed(xs[1])
        r = _packed(xs[2]) if len(xs) > 2 else None
        ta, tb_ = bool(cfg.get("trans_a", False)), bool(cfg.get("trans_b", False))
        ws = [None] * (len(op.results) - 1)                             # a declared scratch result: ops brings its own
        if not ta and tb_:
            return [ops.matmul_nt(a, b_, residual=r)] + ws              # the projection form: differentiable on the tape
        return [ops.gemm(a, b_, ta, tb_, r)] + ws                       # the forms derivative programs use
    if target == "emi_gemm_grouped":
        n_, sum_ = int(cfg["count"]), bool(cfg.get("sum", False))
        ta, tb_ = bool(cfg.get("trans_a", False)), bool(cfg.get("trans_b", False))
        As, Bs = [_packed(t) for t in xs[:n_]], [_packed(t) for t in xs[n_:2 * n_]]
        rs = [_packed(t) for t in xs[2 * n_:]] or None
        if not ta and tb_ and not sum_ and rs is None and all(a is As[0] for a in As):
            return list(ops.matmul_nt_group(As[0], Bs)) + [None] * (len(op.results) - n_)      # sibling projections: differentiable on the tape
        out = ops.gemm_grouped(As, Bs, ta, tb_, rs, sum_into_one=sum_)   # the forms derivative programs use
        return ([out] if sum_ else list(out)) + [None] * (len(op.results) - (1 if sum_ else n_))
    if target == "emi_add":
        return [ops.add(_packed(xs[0]), _packed(xs[1]))]
    if target == "emi_gemm_rope":
        return [ops.gemm_rope(_packed(xs[0]), _packed(xs[1]), _packed(xs[2]))]
    if target == "emi_gemm_swiglu_fwd":
        return list(ops.gemm_swiglu(_packed(xs[0]), _packed(xs[1]), _packed(xs[2])))
    if target == "emi_rope":
        x, table = _packed(xs[0]), _packed(xs[1])
        if x.dim() != 4 or tuple(table.shape) != (x.shape[1], x.shape[3] // 2, 2):
            raise ValueError("custom call emi_rope: x %s, table %s" % (tuple(x.shape), tuple(table.shape)))
        B_, S_, h, d = x.shape
        y = ops.rope_rows(ops.reshape(x, (B_, S_, h * d)), h, table, bool(cfg.get("inverse", False)))
        return [ops.reshape(y, tuple(x.shape))]
    if target == "emi_attn_fwd":
        q, k, v = (_packed(t) for t in xs)
        if q.dim() != 4:
            raise ValueError("custom call emi_attn_fwd: rank-4 operands wanted")
        if cfg.get("bshd", False):
            B_, S_, h, d = q.shape
            flat = lambda t: ops.reshape(t, (B_, S_, h * d))
            o, lse = ops.attention(flat(q), flat(k), flat(v), h, cfg["scale"], causal=bool(cfg.get("causal", True)), layout="bshd",
                                   return_lse=True)
            o = ops.reshape(o, (B_, S_, h, d))
        else:
            o, lse = ops.attention(q, k, v, q.shape[1], cfg["scale"], causal=bool(cfg.get("causal", True)), layout="bhsd", return_lse=True)
        return [o, lse, None][:len(op.results)]
    if target == "emi_attn_step_fwd":
        q, k, v = (_packed(t) for t in xs)
        if q.dim() != 3 or q.shape[0] != 1 or k.dim() != 4:
            raise NotImplementedError("custom call emi_attn_step_fwd is run for one sequence per call (batch = 1)")
        h, d = q.shape[1], q.shape[2]
        o, lse = ops.attention_step(ops.reshape(q, (h * d,)), ops.reshape(k, (k.shape[1], h * d)),
                                    ops.reshape(v, (v.shape[1], h * d)), h, cfg["scale"], return_lse=True)
        return [ops.reshape(o, (1, h, d)), lse, None][:len(op.results)]           # the workspace stays inside the operator
    # adjoint targets: what a reverse-mode module calls; they run the kernels directly and are
    # not themselves differentiable
    lib, st = N.lib(), ops._stream()
    P = lambda t: None if t is None else t.data_ptr()
    if target == "emi_rmsnorm_jvp":
        x, w, tx, tw = (_packed(t) for t in xs)
        ty = torch.empty_like(x)
        N.check(lib.emi_rmsnorm_jvp(st, P(x), P(w), P(tx), P(tw), P(ty), x.numel() // x.shape[-1], x.shape[-1],
                                    float(cfg.get("eps", 1e-5)), ops._code(x)))
        return [ty]
    if target == "emi_swiglu_jvp":
        a, b_, ta, tb = (_packed(t) for t in xs)
        tg = torch.empty_like(a)
        N.check(lib.emi_swiglu_jvp(st, P(a), P(b_), P(ta), P(tb), P(tg), a.numel(), ops._code(a)))
        return [tg]
    if target == "emi_attn_step_jvp":
        q, k, v, o, lse, tq, tk, tv = (_packed(t) for t in xs)
        if q.dim() != 3 or q.shape[0] != 1 or k.dim() != 4:
            raise NotImplementedError("custom call emi_attn_step_jvp is run for one sequence per call (batch = 1)")
        h, d, S = q.shape[1], q.shape[2], k.shape[1]
        to = torch.empty_like(q)
        nbytes = lib.emi_attn_step_workspace_bytes(1, h, S, d)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
        N.check(lib.emi_attn_step_jvp(st, P(q), P(k), P(v), P(o), P(lse), P(tq), P(tk), P(tv), P(to), P(ws), nbytes, 1, h, S, d,
                                      h * d, d, S * h * d, d, h * d, float(cfg["scale"]), ops._code(q)))
        return [to, None][:len(op.results)]
    if target == "emi_gemm_swiglu_bwd":
        dy, w2t, a, b_ = (_packed(t) for t in xs)
        T_, K, Hn = dy.shape[0], dy.shape[1], w2t.shape[0]
        da, db = torch.empty_like(a), torch.empty_like(a)
        nbytes = lib.emi_gemm_swiglu_bwd_workspace_bytes(T_, Hn, K, ops._code(dy))
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dy.device)
        N.check(lib.emi_gemm_swiglu_bwd(st, P(dy), P(w2t), P(a), P(b_), P(da), P(db), P(ws), nbytes, T_, Hn, K, ops._code(dy)))
        return [da, db, None][:len(op.results)]
    if target == "emi_attn_bwd_rope":
        bshd = bool(cfg.get("bshd", False))
        q, k, v, o, lse, do, table = (_packed(t) for t in xs)
        B_, S_, h, d = (q.shape if bshd else (q.shape[0], q.shape[2], q.shape[1], q.shape[3]))
        sb, sh, ss = (S_ * h * d, d, h * d) if bshd else (h * S_ * d, S_ * d, d)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        nbytes = lib.emi_attn_bwd_workspace_bytes(B_, h, S_, d)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
        N.check(lib.emi_attn_bwd_rope(st, P(q), P(k), P(v), P(o), P(lse), P(do), P(dq), P(dk), P(dv), P(table), P(ws), nbytes, B_, h,
                                      S_, d, sb, sh, ss, float(cfg["scale"]), int(bool(cfg.get("causal", True))), ops._code(q)))
        return [dq, dk, dv, None][:len(op.results)]
    if target in ("emi_attn_bwd", "emi_attn_jvp"):
        bshd = bool(cfg.get("bshd", False))
        q = _packed(xs[0])
        B_, S_, h, d = (q.shape if bshd else (q.shape[0], q.shape[2], q.shape[1], q.shape[3]))
        sb, sh, ss = (S_ * h * d, d, h * d) if bshd else (h * S_ * d, S_ * d, d)
        causal = int(bool(cfg.get("causal", True)))
        if target == "emi_attn_bwd":
            q, k, v, o, lse, do = (_packed(t) for t in xs)
            dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
            nbytes = lib.emi_attn_bwd_workspace_bytes(B_, h, S_, d)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
            N.check(lib.emi_attn_bwd(st, P(q), P(k), P(v), P(o), P(lse), P(do), P(dq), P(dk), P(dv), P(ws), nbytes, B_, h, S_, d,
                                     sb, sh, ss, float(cfg["scale"]), causal, ops._code(q)))
            return [dq, dk, dv, None][:len(op.results)]
        q, k, v, lse, tq, tk, tv = (_packed(t) for t in xs)
        to = torch.empty_like(q)
        N.check(lib.emi_attn_jvp(st, P(q), P(k), P(v), P(lse), P(tq), P(tk), P(tv), P(to), B_, h, S_, d, sb, sh, ss,
                                 float(cfg["scale"]), causal, ops._code(q)))
        return [to]
    if target == "emi_rmsnorm_bwd":
        x, w, dy = (_packed(t) for t in xs[:3])
        rows, dim = x.numel() // x.shape[-1], x.shape[-1]
        dx, dg = torch.empty_like(x), torch.empty_like(w)
        nbytes = lib.emi_rmsnorm_bwd_workspace_bytes(rows, dim)
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
        N.check(lib.emi_rmsnorm_bwd(st, P(x), P(w), P(dy), None, P(dx), P(dg), P(ws), nbytes, rows, dim, float(cfg.get("eps", 1e-5)),
                                    ops._code(x)))
        return [dx, dg, None][:len(op.results)]
    if target == "emi_swiglu_bwd":
        a, b_, dg = (_packed(t) for t in xs)
        da, db = torch.empty_like(a), torch.empty_like(a)
        N.check(lib.emi_swiglu_bwd(st, P(a), P(b_), P(dg), P(da), P(db), a.numel(), ops._code(a)))
        return [da, db]
    if target == "emi_attn_step_bwd":
        q, k, v, o, lse, do = (_packed(t) for t in xs)
        if q.dim() != 3 or q.shape[0] != 1 or k.dim() != 4:
            raise NotImplementedError("custom call emi_attn_step_bwd is run for one sequence per call (batch = 1)")
        h, d, S = q.shape[1], q.shape[2], k.shape[1]
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        nbytes = lib.emi_attn_step_workspace_bytes(1, h, S, d)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
        N.check(lib.emi_attn_step_bwd(st, P(q), P(k), P(v), P(o), P(lse), P(do), P(dq), P(dk), P(dv), P(ws), nbytes, 1, h, S, d,
                                      h * d, d, S * h * d, d, h * d, float(cfg["scale"]), ops._code(q)))
        return [dq, dk, dv, None][:len(op.results)]
    if target == "emi_cross_entropy_fwd":
        z, t = _packed(xs[0]), xs[1].contiguous()
        loss, lse = ops.cross_entropy(z, t, return_lse=True)
        return [loss, lse][:len(op.results)]
    if target in ("emi_cross_entropy_bwd", "emi_cross_entropy_jvp"):
        z, t, lse, w = (_packed(x) for x in xs)
        rows, V = z.numel() // z.shape[-1], z.shape[-1]
        if t.dtype != torch.int32 or lse.dtype != torch.float32 or t.numel() != rows or lse.numel() != rows:
            raise ValueError("custom call %s: logits %s, targets %s %s, lse %s %s" %
                             (target, tuple(z.shape), t.dtype, tuple(t.shape), lse.dtype, tuple(lse.shape)))
        if target == "emi_cross_entropy_bwd":
            if w.dtype != torch.float32 or w.numel() != rows:
                raise ValueError("custom call emi_cross_entropy_bwd: the cotangent of the losses must be f32[%d]" % rows)
            dz = torch.empty_like(z)
            N.check(lib.emi_cross_entropy_bwd(st, P(z), P(t), P(lse), P(w), P(dz), rows, V, ops._code(z)))
            return [dz]
        if w.dtype != z.dtype or tuple(w.shape) != tuple(z.shape):
            raise ValueError("custom call emi_cross_entropy_jvp: the tangent must have the logits' type")
        tl = torch.empty(t.shape, dtype=torch.float32, device=z.device)
        N.check(lib.emi_cross_entropy_jvp(st, P(z), P(t), P(lse), P(w), P(tl), rows, V, ops._code(z)))
        return [tl]
    if target == "emi_embedding_fwd":
        tok, table = _packed(xs[0]), _packed(xs[1])
        return [ops.embedding(tok, table)]
    if target == "emi_embedding_bwd":
        tok, dx = _packed(xs[0]), _packed(xs[1])
        V, D = op.types[0].shape
        if tok.dtype != torch.int32 or tuple(dx.shape) != tuple(tok.shape) + (D,):
            raise ValueError("custom call emi_embedding_bwd: tokens %s %s, dx %s, table [%d, %d]" %
                             (tok.dtype, tuple(tok.shape), tuple(dx.shape), V, D))
        dt = torch.empty((V, D), dtype=dx.dtype, device=dx.device)
        nbytes = lib.emi_embedding_bwd_workspace_bytes(V, D, ops._code(dx))
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dx.device)
        N.check(lib.emi_embedding_bwd(st, P(tok), P(dx), P(dt), P(ws), nbytes, tok.numel(), V, D, ops._code(dx)))
        return [dt, None][:len(op.results)]
    raise NotImplementedError("custom call target '%s' is not one of this library's" % target)


Executable._custom_call = _custom_call_impl


def _packed(t):
    """Contiguous and 16-byte aligned, as the fused kernels want their operands; a view that
    is neither is copied (tracked, so cotangents flow back to the view's source)."""
    if t.is_contiguous() and t.data_ptr() % 16 == 0:
        return t
    return H.unary_copy(t)


# ---------------------------------------------------------------------------
# printer: the module with its clusters lowered to typed-FFI custom calls
# ---------------------------------------------------------------------------

def _fmt_float(v):
    v = float(v)
    if v == math.inf:
        return "0x7F800000"
    if v == -math.inf:
        return "0xFF800000"
    return "%.9e" % v


def _dense_text(value, ty):
    a = np.asarray(value)
    flat = a.reshape(-1)
    is_float = ty.dtype in ("f32", "bf16", "f16", "f64")
    one = (lambda x: _fmt_float(x)) if is_float else (lambda x: str(bool(x)).lower() if ty.dtype == "i1" else str(int(x)))
    if flat.size and np.all(flat == flat[0]) and not (is_float and np.isinf(flat[0]) and ty.dtype != "f32"):
        return one(flat[0])

    if flat.size > 1024 and ty.dtype in ("f32", "bf16"):           # large tables: raw little-endian bytes as hex
        if ty.dtype == "bf16":
            raw = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).view(torch.int16).numpy().astype("<i2").tobytes()
        else:
            raw = np.ascontiguousarray(a, dtype="<f4").tobytes()
        return '"0x%s"' % raw.hex().upper()

    def lit(x):
        return "[" + ", ".join(lit(y) for y in x) + "]" if x.ndim else one(x)

    return lit(a)


def _layouts(types):
    def one(t):
        r = len(t.shape)
        body = "" if r == 0 else "0" if r == 1 else "[" + ", ".join(str(i) for i in reversed(range(r))) + "]"
        return "dense<%s> : tensor<%dxindex>" % (body, r)
    return "[" + ", ".join(one(t) for t in types) + "]"


class _Printer:
    def __init__(self, func):
        self.f, self.lines, self.n = func, [], 0
        self.types = {a: t for a, t in func.args}
        for op in func.ops:
            for r, t in zip(op.results, op.types):
                self.types[r] = t

    def fresh(self, ty):
        name = "%%emi%d" % self.n
        self.n += 1
        self.types[name] = ty
        return name

    def emit(self, text):
        self.lines.append("    " + text)

    def reshape(self, v, shape):
        ty = TensorType(shape, self.types[v].dtype)
        if self.types[v].shape == ty.shape:
            return v
        r = self.fresh(ty)
        self.emit("%s = stablehlo.reshape %s : (%r) -> %r" % (r, v, self.types[v], ty))
        return r

    def custom_call(self, results, target, operands, config, out_types):
        cfg = ", ".join("%s = %s" % (k, ("true" if v else "false") if isinstance(v, bool) else
                                     ("%d : i64" % v if isinstance(v, int) else "%s : f32" % _fmt_float(v))) for k, v in config.items())
        lhs = results[0] if len(results) == 1 else "%s:%d" % (results[0].split("#")[0], len(results))
        outs = repr(out_types[0]) if len(out_types) == 1 else "(" + ", ".join(repr(t) for t in out_types) + ")"
        self.emit("%s = stablehlo.custom_call @%s(%s) {api_version = 4 : i32, backend_config = {%s}, operand_layouts = %s, "
                  "result_layouts = %s} : (%s) -> %s" % (lhs, target, ", ".join(operands), cfg,
                                                       _layouts([self.types[o] for o in operands]), _layouts(out_types),
                                                       ", ".join(repr(self.types[o]) for o in operands), outs))

    def op(self, op):
        T = self.types
        n, r = op.name, (op.results[0] if op.results else None)
        ty = op.types[0] if op.types else None
        if n == "return":
            self.emit("return %s : %s" % (", ".join(op.operands), ", ".join(repr(T[o]) for o in op.operands)))
        elif n == "constant":
            self.emit("%s = stablehlo.constant dense<%s> : %r" % (r, _dense_text(op.attrs["value"], ty), ty))
        elif n in BINARY_OPS:
            self.emit("%s = stablehlo.%s %s, %s : %r" % (r, n, op.operands[0], op.operands[1], ty))
        elif n in UNARY_OPS:
            self.emit("%s = stablehlo.%s %s : %r" % (r, n, op.operands[0], ty))
        elif n in ("reshape", "convert"):
            self.emit("%s = stablehlo.%s %s : (%r) -> %r" % (r, n, op.operands[0], T[op.operands[0]], ty))
        elif n == "transpose":
            self.emit("%s = stablehlo.transpose %s, dims = %s : (%r) -> %r" % (r, op.operands[0], list(op.attrs["perm"]), T[op.operands[0]], ty))
        elif n == "broadcast_in_dim":
            self.emit("%s = stablehlo.broadcast_in_dim %s, dims = %s : (%r) -> %r" % (r, op.operands[0], list(op.attrs["dims"]), T[op.operands[0]], ty))
        elif n == "reduce":
            self.emit("%s = stablehlo.reduce(%s init: %s) applies stablehlo.%s across dimensions = %s : (%r, %r) -> %r" % (
                r, op.operands[0], op.operands[1], op.attrs["body"], list(op.attrs["dims"]), T[op.operands[0]], T[op.operands[1]], ty))
        elif n == "dot_general":
            a = op.attrs
            dims = ("batching_dims = %s x %s, " % (list(a["batch_a"]), list(a["batch_b"])) if a["batch_a"] else "") + \
                "contracting_dims = %s x %s" % (list(a["contract_a"]), list(a["contract_b"]))
            self.emit("%s = stablehlo.dot_general %s, %s, %s, precision = [DEFAULT, DEFAULT] : (%r, %r) -> %r" % (
                r, op.operands[0], op.operands[1], dims, T[op.operands[0]], T[op.operands[1]], ty))
        elif n == "slice":
            a = op.attrs
            self.emit("%s = stablehlo.slice %s [%s] : (%r) -> %r" % (r, op.operands[0], ", ".join(
                "%d:%d" % (s_, l) if st == 1 else "%d:%d:%d" % (s_, l, st) for s_, l, st in zip(a["start"], a["limit"], a["stride"])),
                T[op.operands[0]], ty))
        elif n == "concatenate":
            self.emit("%s = stablehlo.concatenate %s, dim = %d : (%s) -> %r" % (r, ", ".join(op.operands), op.attrs["dim"],
                                                                                ", ".join(repr(T[o]) for o in op.operands), ty))
        elif n == "gather":
            a = op.attrs
            self.emit('%s = "stablehlo.gather"(%s, %s) <{dimension_numbers = #stablehlo.gather<offset_dims = %s, '
                      'collapsed_slice_dims = %s, start_index_map = %s, index_vector_dim = %d>, indices_are_sorted = false, '
                      'slice_sizes = array<i64: %s>}> : (%r, %r) -> %r' % (
                          r, op.operands[0], op.operands[1], a["offset_dims"], a["collapsed_slice_dims"], a["start_index_map"],
                          a["index_vector_dim"], ", ".join(str(v) for v in a["slice_sizes"]), T[op.operands[0]], T[op.operands[1]], ty))
        elif n == "call":
            lhs = r if len(op.results) == 1 else "%s:%d" % (op.results[0].split("#")[0], len(op.results))
            outs = repr(ty) if len(op.types) == 1 else "(" + ", ".join(repr(t) for t in op.types) + ")"
            self.emit("%s = call @%s(%s) : (%s) -> %s" % (lhs, _sym(op.attrs["callee"]), ", ".join(op.operands),
                                                         ", ".join(repr(T[o]) for o in op.operands), outs))
        elif n == "custom_call":
            self.custom_call(op.results, op.attrs["target"], op.operands, op.attrs["config"], op.types)
        elif n == "compare":
            self.emit("%s = stablehlo.compare %s, %s, %s, FLOAT : (%r, %r) -> %r" % (r, op.attrs["direction"], op.operands[0],
                                                                                 op.operands[1], T[op.operands[0]], T[op.operands[1]], ty))
        elif n == "select":
            self.emit("%s = stablehlo.select %s, %s, %s : (%s) -> %r" % (r, op.operands[0], op.operands[1], op.operands[2],
                                                                        ", ".join(repr(T[o]) for o in op.operands), ty))
        elif n == "pad":
            a = op.attrs
            self.emit("%s = stablehlo.pad %s, %s, low = %s, high = %s, interior = %s : (%r, %r) -> %r" % (
                r, op.operands[0], op.operands[1], list(a["low"]), list(a["high"]), list(a["interior"]), T[op.operands[0]],
                T[op.operands[1]], ty))
        else:
            raise NotImplementedError("cannot print operator '%s'" % n)


def _sym(name):
    """A symbol name as MLIR prints it: quoted unless it is a plain identifier."""
    return name if re.fullmatch(r"[A-Za-z0-9_.$-]+", name) else '"%s"' % name


def print_module(funcs):
    """StableHLO text of parsed (and possibly rewritten) functions; fused clusters are printed
    as `stablehlo.custom_call @emi_*` with `api_version = 4` and their scalars in
    `backend_config` (the wire format of include/emi_ffi.h), wrapped in the reshapes that bring
    the operands to the handlers' layouts."""
    from .stablehlo_ad import lower_fused

    out = ["module {"]
    for f in funcs.values():
        f = lower_fused(f)
        p = _Printer(f)
        for op in f.ops:
            p.op(op)
        rets = [o for op in f.ops if op.name == "return" for o in op.operands]
        out.append("  func.func %s@%s(%s) -> (%s) {" % ("public " if f.name == "main" else "private ", _sym(f.name),
                                                      ", ".join("%s: %r" % (a, t) for a, t in f.args),
                                                      ", ".join(repr(p.types[o]) for o in rets)))
        out += p.lines
        out.append("  }")
    out.append("}")
    return "\n".join(out) + "\n"


def lower_to_custom_calls(text):
    """Parse, fold constants, match the llama clusters, and print the module back with the
    clusters as typed-FFI custom calls to this library's targets."""
    exe = Executable(text, fuse=True)
    return print_module(exe.funcs), dict(exe.fused)


_CACHE = {}


def compile_text(text, fuse=True):
    key = (text, tuple(fuse) if isinstance(fuse, (tuple, list)) else fuse)
    exe = _CACHE.get(key)
    if exe is None:
        exe = _CACHE[key] = Executable(text, fuse)
    return exe
