"""The single-token llama step of the reference (test/llama.py:35-238) written out as StableHLO
text, operator by operator in the order the Python source applies them, the way a trace of
that function prints: per-layer weight slices, `w @ x` as dot_general, the batched 2x2
rotations against constant matrices, cache append as concatenate, a per-head loop of
dot / softmax / dot, the sigmoid spelled 1 / (1 + exp(-x)), and `jnp.sqrt(head_size)` as a
sqrt of a constant.  For callers that have no tracer at hand (`hlo_call(*args,
source=llama_step_text(config, pos)[0])`), for the front end's tests and for its benchmark;
nothing here computes."""
import numpy as np


class Builder:
    def __init__(self, dtype="f32"):
        self.lines, self.n, self.types, self.dtype = [], 0, {}, dtype

    def ty(self, shape):
        return "tensor<%s>" % "x".join([str(s) for s in shape] + [self.dtype])

    def new(self, shape):
        name = "%%%d" % self.n
        self.n += 1
        self.types[name] = tuple(shape)
        return name

    def arg(self, name, shape):
        self.types[name] = tuple(shape)
        return name

    def emit(self, shape, text):
        r = self.new(shape)
        self.lines.append("    %s = %s" % (r, text))
        return r

    def t(self, v):
        return self.ty(self.types[v])

    def const(self, value, shape=()):
        value = np.asarray(value, dtype=np.float64)
        if value.ndim == 0:
            v = float(value)
            body = ("0xFF80" if self.dtype == "bf16" else "0xFF800000") if v == -np.inf else "%.9e" % v
        else:
            def lit(a):
                return "[" + ", ".join(lit(x) for x in a) + "]" if a.ndim else "%.9e" % float(a)
            body, shape = lit(value), value.shape
        return self.emit(shape, "stablehlo.constant dense<%s> : %s" % (body, self.ty(shape)))

    def binary(self, op, a, b):
        return self.emit(self.types[a], "stablehlo.%s %s, %s : %s" % (op, a, b, self.t(a)))

    def unary(self, op, a):
        return self.emit(self.types[a], "stablehlo.%s %s : %s" % (op, a, self.t(a)))

    def bcast(self, a, shape, dims=()):
        return self.emit(shape, "stablehlo.broadcast_in_dim %s, dims = [%s] : (%s) -> %s" % (
            a, ", ".join(str(d) for d in dims), self.t(a), self.ty(shape)))

    def reshape(self, a, shape):
        return self.emit(shape, "stablehlo.reshape %s : (%s) -> %s" % (a, self.t(a), self.ty(shape)))

    def slice(self, a, start, limit):
        shape = [l - s for s, l in zip(start, limit)]
        return self.emit(shape, "stablehlo.slice %s [%s] : (%s) -> %s" % (
            a, ", ".join("%d:%d" % (s, l) for s, l in zip(start, limit)), self.t(a), self.ty(shape)))

    def concat(self, xs, dim):
        shape = list(self.types[xs[0]])
        shape[dim] = sum(self.types[x][dim] for x in xs)
        return self.emit(shape, "stablehlo.concatenate %s, dim = %d : (%s) -> %s" % (
            ", ".join(xs), dim, ", ".join(self.t(x) for x in xs), self.ty(shape)))

    def reduce(self, a, kind, dims):
        init = self.const(0.0 if kind == "add" else -np.inf)
        shape = [s for i, s in enumerate(self.types[a]) if i not in dims]
        return self.emit(shape, "stablehlo.reduce(%s init: %s) applies stablehlo.%s across dimensions = [%s] : (%s, %s) -> %s" % (
            a, init, kind, ", ".join(str(d) for d in dims), self.t(a), self.ty(()), self.ty(shape)))

    def dot(self, a, b, batch=((), ()), contract=((), ())):
        sa, sb = self.types[a], self.types[b]
        shape = [sa[d] for d in batch[0]] + [s for i, s in enumerate(sa) if i not in batch[0] and i not in contract[0]] + \
            [s for i, s in enumerate(sb) if i not in batch[1] and i not in contract[1]]
        lst = lambda xs: "[" + ", ".join(str(x) for x in xs) + "]"
        dims = ""
        if batch[0]:
            dims += "batching_dims = %s x %s, " % (lst(batch[0]), lst(batch[1]))
        dims += "contracting_dims = %s x %s" % (lst(contract[0]), lst(contract[1]))
        return self.emit(shape, "stablehlo.dot_general %s, %s, %s, precision = [DEFAULT, DEFAULT] : (%s, %s) -> %s" % (
            a, b, dims, self.t(a), self.t(b), self.ty(shape)))


def rotation_constants(dim, head_size, kv_dim, pos):
    """toconv / toconv2 of test/llama.py:127-140 in float32."""
    mats = []
    for i in range(0, dim, 2):
        freq = np.float32(1.0) / np.power(np.float32(10000.0), np.float32((i % head_size) / head_size))
        val = np.float32(pos) * freq
        c, s = np.cos(val, dtype=np.float32), np.sin(val, dtype=np.float32)
        mats.append([[c, -s], [s, c]])
    toconv = np.asarray(mats, dtype=np.float32)
    toconv2 = np.concatenate([toconv[:kv_dim // 2], np.tile(np.eye(2, dtype=np.float32), (dim // 2 - kv_dim // 2, 1, 1))])
    return toconv, toconv2


WEIGHT_ORDER = ["rms_att_weight", "wq", "wk", "wv", "wo", "rms_ffn_weight", "w1", "w2", "w3", "rms_final_weight"]


def llama_step_text(config, pos, dtype="f32"):
    """(text, argument names in order): main(x, <weights in WEIGHT_ORDER>, key_cache, value_cache) -> x."""
    dim, hidden, L, H = config["dim"], config["hidden_dim"], config["n_layers"], config["n_heads"]
    kvh = config["n_kv_heads"]
    hs = dim // H
    kv_dim = hs * kvh
    kv_mul = H // kvh
    b = Builder(dtype)
    shapes = {"x": (dim,), "rms_att_weight": (L, dim), "wq": (L, dim, dim), "wk": (L, kv_dim, dim), "wv": (L, kv_dim, dim),
              "wo": (L, dim, dim), "rms_ffn_weight": (L, dim), "w1": (L, hidden, dim), "w2": (L, dim, hidden),
              "w3": (L, hidden, dim), "rms_final_weight": (dim,), "key_cache": (L, pos, kv_dim),
              "value_cache": (L, pos, kv_dim)}
    order = ["x"] + WEIGHT_ORDER + ["key_cache", "value_cache"]
    a = {n: b.arg("%" + n, shapes[n]) for n in order}

    def rmsnorm(x, w):
        ss = b.dot(x, x, contract=((0,), (0,)))
        ss = b.binary("divide", ss, b.const(float(dim)))
        ss = b.binary("add", ss, b.const(1e-5))
        ss = b.binary("divide", b.const(1.0), b.unary("sqrt", ss))
        return b.binary("multiply", b.binary("multiply", w, x), b.bcast(ss, (dim,)))

    def layer_slice(w, i):
        shape = b.types[w]
        s = b.slice(w, [i] + [0] * (len(shape) - 1), [i + 1] + list(shape[1:]))
        return b.reshape(s, shape[1:])

    def matvec(w, x):
        return b.dot(w, x, contract=((1,), (0,)))

    def softmax(x):
        n = b.types[x]
        mx = b.reduce(x, "maximum", [0])
        e = b.unary("exponential", b.binary("subtract", x, b.bcast(mx, n)))
        return b.binary("divide", e, b.bcast(b.reduce(e, "add", [0]), n))

    toconv, toconv2 = rotation_constants(dim, hs, kv_dim, pos)
    rot_q, rot_k = b.const(toconv), b.const(toconv2)
    x = a["x"]
    for i in range(L):
        xb = rmsnorm(x, layer_slice(a["rms_att_weight"], i))
        q = matvec(layer_slice(a["wq"], i), xb)
        k = matvec(layer_slice(a["wk"], i), xb)
        v = matvec(layer_slice(a["wv"], i), xb)
        q_tmp, k_tmp = b.reshape(q, (dim // 2, 2)), b.reshape(k, (dim // 2, 2))
        k = b.reshape(b.dot(rot_k, k_tmp, batch=((0,), (0,)), contract=((2,), (1,))), (dim,))
        q = b.reshape(b.dot(rot_q, q_tmp, batch=((0,), (0,)), contract=((2,), (1,))), (dim,))
        kc = b.concat([layer_slice(a["key_cache"], i), b.reshape(k, (1, dim))], 0)
        vc = b.concat([layer_slice(a["value_cache"], i), b.reshape(v, (1, dim))], 0)
        heads = []
        for h in range(H):
            q2 = b.slice(q, [hs * h], [hs * (h + 1)])
            ki = h // kv_mul
            att = b.dot(b.slice(kc, [0, ki * hs], [pos + 1, (ki + 1) * hs]), q2, contract=((1,), (0,)))
            att = b.binary("divide", att, b.bcast(b.unary("sqrt", b.const(float(hs))), (pos + 1,)))
            att = softmax(att)
            heads.append(b.dot(b.slice(vc, [0, ki * hs], [pos + 1, (ki + 1) * hs]), att, contract=((0,), (0,))))
        xb = b.concat(heads, 0)
        x = b.binary("add", x, matvec(layer_slice(a["wo"], i), xb))
        xb = rmsnorm(x, layer_slice(a["rms_ffn_weight"], i))
        hb = matvec(layer_slice(a["w1"], i), xb)
        hb2 = matvec(layer_slice(a["w3"], i), xb)
        sig = b.binary("divide", b.bcast(b.const(1.0), (hidden,)),
                       b.binary("add", b.bcast(b.const(1.0), (hidden,)), b.unary("exponential", b.unary("negate", hb))))
        hb = b.binary("multiply", b.binary("multiply", hb, sig), hb2)
        x = b.binary("add", x, matvec(layer_slice(a["w2"], i), hb))
    x = rmsnorm(x, a["rms_final_weight"])
    head = "module @jit_forward {\n  func.func public @main(%s) -> (%s {jax.result_info = \"\"}) {\n" % (
        ", ".join("%s: %s" % (a[n], b.ty(shapes[n])) for n in order), b.ty((dim,)))
    text = head + "\n".join(b.lines) + "\n    return %s : %s\n  }\n}\n" % (x, b.ty((dim,)))
    return text, order
