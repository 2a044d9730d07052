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

    def blob(self, array, dtype=None):
        """A constant too large to spell out: raw little-endian bytes as a hex string."""
        a = np.ascontiguousarray(array, dtype=np.float32)
        shape = a.shape
        if (dtype or self.dtype) == "bf16":
            bits = a.view(np.uint32)
            raw = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype("<u2").tobytes()      # round to nearest even
        else:
            raw = a.astype("<f4").tobytes()
        ty = "tensor<%s>" % "x".join([str(s) for s in shape] + [dtype or self.dtype])
        r = self.new(shape)
        self.lines.append('    %s = stablehlo.constant dense<"0x%s"> : %s' % (r, raw.hex().upper(), ty))
        return r

    def transpose(self, a, perm):
        shape = [self.types[a][p] for p in perm]
        return self.emit(shape, "stablehlo.transpose %s, dims = [%s] : (%s) -> %s" % (
            a, ", ".join(str(p) for p in perm), self.t(a), self.ty(shape)))

    def iota(self, shape, dim):
        r = self.new(shape)
        self.lines.append("    %s = stablehlo.iota dim = %d : tensor<%s>" % (r, dim, "x".join([str(s) for s in shape] + ["i32"])))
        return r

    def compare(self, direction, a, b, kind="SIGNED", elem="i32"):
        shape = self.types[a]
        ty = "tensor<%s>" % "x".join([str(s) for s in shape] + [elem])
        r = self.new(shape)
        self.lines.append("    %s = stablehlo.compare %s, %s, %s, %s : (%s, %s) -> tensor<%s>" % (
            r, direction, a, b, kind, ty, ty, "x".join([str(s) for s in shape] + ["i1"])))
        return r

    def bcast_pred(self, a, shape, dims):
        r = self.new(shape)
        i1 = lambda sh: "tensor<%s>" % "x".join([str(s) for s in sh] + ["i1"])
        self.lines.append("    %s = stablehlo.broadcast_in_dim %s, dims = [%s] : (%s) -> %s" % (
            r, a, ", ".join(str(d) for d in dims), i1(self.types[a]), i1(shape)))
        return r

    def select(self, p, a, b):
        shape = self.types[a]
        i1 = "tensor<%s>" % "x".join([str(s) for s in shape] + ["i1"])
        return self.emit(shape, "stablehlo.select %s, %s, %s : %s, %s" % (p, a, b, i1, self.t(a)))

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


LAYER_ORDER = ["rms_att_weight", "wq", "wk", "wv", "wo", "rms_ffn_weight", "w1", "w2", "w3"]


def _rope_tables(b, S, hs, theta, dtype):
    pos = np.arange(S, dtype=np.float64)[:, None]
    freq = 1.0 / np.power(theta, (2.0 * np.arange(hs // 2, dtype=np.float64)) / hs)[None, :]
    cos_c, sin_c = b.blob(np.cos(pos * freq), "f32"), b.blob(np.sin(pos * freq), "f32")
    if dtype != "f32":
        cos_c = b.emit((S, hs // 2), "stablehlo.convert %s : (tensor<%dx%dxf32>) -> %s" % (cos_c, S, hs // 2, b.ty((S, hs // 2))))
        sin_c = b.emit((S, hs // 2), "stablehlo.convert %s : (tensor<%dx%dxf32>) -> %s" % (sin_c, S, hs // 2, b.ty((S, hs // 2))))
    return cos_c, sin_c


def _rmsnorm_rows(b, x, w, eps):
    B, S, dim = b.types[x]
    ss = b.reduce(b.binary("multiply", x, x), "add", [2])                          # [B, S]
    ss = b.binary("divide", ss, b.bcast(b.const(float(dim)), (B, S)))
    ss = b.binary("add", ss, b.bcast(b.const(eps), (B, S)))
    ss = b.binary("divide", b.bcast(b.const(1.0), (B, S)), b.unary("sqrt", ss))
    xn = b.binary("multiply", x, b.bcast(ss, (B, S, dim), (0, 1)))
    return b.binary("multiply", xn, b.bcast(w, (B, S, dim), (2,)))


def _linear_rows(b, x, w):
    return b.dot(x, w, contract=((len(b.types[x]) - 1,), (1,)))


def _layer_rows(b, x, a, H, hidden, tables, eps):
    """One decoder layer of test/llama.py:144-233 over x [B, S, dim]; a: weight name -> value name."""
    B, S, dim = b.types[x]
    hs = dim // H
    cos_c, sin_c = tables

    def rope(x):
        xr = b.reshape(x, (B, S, H, hs // 2, 2))
        half = (B, S, H, hs // 2)
        x0 = b.reshape(b.slice(xr, [0, 0, 0, 0, 0], [B, S, H, hs // 2, 1]), half)
        x1 = b.reshape(b.slice(xr, [0, 0, 0, 0, 1], [B, S, H, hs // 2, 2]), half)
        cb, sb = b.bcast(cos_c, half, (1, 3)), b.bcast(sin_c, half, (1, 3))
        o0 = b.binary("subtract", b.binary("multiply", x0, cb), b.binary("multiply", x1, sb))
        o1 = b.binary("add", b.binary("multiply", x0, sb), b.binary("multiply", x1, cb))
        both = b.concat([b.reshape(o0, half + (1,)), b.reshape(o1, half + (1,))], 4)
        return b.reshape(both, (B, S, dim))

    xb = _rmsnorm_rows(b, x, a["rms_att_weight"], eps)
    q, k, v = rope(_linear_rows(b, xb, a["wq"])), rope(_linear_rows(b, xb, a["wk"])), _linear_rows(b, xb, a["wv"])
    heads = lambda t: b.transpose(b.reshape(t, (B, S, H, hs)), [0, 2, 1, 3])                 # [B, H, S, hs]
    qh, kh, vh = heads(q), heads(k), heads(v)
    att = b.dot(qh, kh, batch=((0, 1), (0, 1)), contract=((3,), (3,)))                      # [B, H, S, S]
    att = b.binary("divide", att, b.bcast(b.unary("sqrt", b.const(float(hs))), (B, H, S, S)))
    causal = b.compare("GE", b.iota((S, S), 0), b.iota((S, S), 1))                           # key <= query
    att = b.select(b.bcast_pred(causal, (B, H, S, S), (2, 3)), att, b.bcast(b.const(-np.inf), (B, H, S, S)))
    mx = b.reduce(att, "maximum", [3])
    e = b.unary("exponential", b.binary("subtract", att, b.bcast(mx, (B, H, S, S), (0, 1, 2))))
    p = b.binary("divide", e, b.bcast(b.reduce(e, "add", [3]), (B, H, S, S), (0, 1, 2)))
    o = b.dot(p, vh, batch=((0, 1), (0, 1)), contract=((3,), (2,)))                         # [B, H, S, hs]
    o = b.reshape(b.transpose(o, [0, 2, 1, 3]), (B, S, dim))
    x = b.binary("add", x, _linear_rows(b, o, a["wo"]))
    xb = _rmsnorm_rows(b, x, a["rms_ffn_weight"], eps)
    hb, hb2 = _linear_rows(b, xb, a["w1"]), _linear_rows(b, xb, a["w3"])
    one = b.bcast(b.const(1.0), (B, S, hidden))
    sig = b.binary("divide", one, b.binary("add", one, b.unary("exponential", b.unary("negate", hb))))
    return b.binary("add", x, _linear_rows(b, b.binary("multiply", b.binary("multiply", hb, sig), hb2), a["w2"]))


def llama_layer_text(config, batch, seq, dtype="f32", eps=1e-5, theta=10000.0):
    """(text, argument names): one decoder layer of test/llama.py:144-233 over a whole batch of
    sequences, main(x [B, S, dim], <weights in LAYER_ORDER>) -> x, written the way the batched
    form of that function traces: RMSNorm as sum(x*x) / dim over the last index, projections as
    dot_general against [out, in] weights, the pair rotation with cos / sin tables [S, hs/2]
    (constants: positions are static), scores per head from a batched dot_general, a causal mask
    from two iotas and a compare, softmax over the keys, and the SwiGLU FFN."""
    dim, hidden, H = config["dim"], config["hidden_dim"], config["n_heads"]
    B, S = batch, seq
    b = Builder(dtype)
    shapes = {"x": (B, S, dim), "rms_att_weight": (dim,), "wq": (dim, dim), "wk": (dim, dim), "wv": (dim, dim), "wo": (dim, dim),
              "rms_ffn_weight": (dim,), "w1": (hidden, dim), "w2": (dim, hidden), "w3": (hidden, dim)}
    order = ["x"] + LAYER_ORDER
    a = {n: b.arg("%" + n, shapes[n]) for n in order}
    x = _layer_rows(b, a["x"], a, H, hidden, _rope_tables(b, S, dim // H, theta, dtype), eps)
    head = "module @jit_layer {\n  func.func public @main(%s) -> (%s {jax.result_info = \"\"}) {\n" % (
        ", ".join("%s: %s" % (a[n], b.ty(shapes[n])) for n in order), b.ty((B, S, dim)))
    return head + "\n".join(b.lines) + "\n    return %s : %s\n  }\n}\n" % (x, b.ty((B, S, dim))), order


MODEL_ORDER = ["token_embedding_table"] + WEIGHT_ORDER + ["wcls"]


def llama_model_text(config, batch, seq, dtype="f32", loss=None, eps=1e-5, theta=10000.0):
    """(text, argument names): the whole model over a batch of token sequences, the pieces test/llama.py comments out
    (:109-113, :236) switched on: main(tokens [B, S] i32, <weights in MODEL_ORDER, per-layer ones stacked [L, ...]>
    [, targets [B, S] i32]) -> logits [B, S, vocab], or with `loss` the mean softmax cross-entropy (a scalar) in one
    of the two spellings JAX users write:
      loss="onehot":  -mean(sum(one_hot(targets) * log_softmax(logits), -1))
      loss="gather":  -mean(take_along_axis(log_softmax(logits), targets[..., None], -1))
    The embedding is the row lookup `table[tokens]` (a gather), every layer slices its weights out of the stacks
    (`wq[l, :, :]`, :149) and is written as in `llama_layer_text`."""
    dim, hidden, H, L, V = config["dim"], config["hidden_dim"], config["n_heads"], config["n_layers"], config["vocab_size"]
    B, S, T = batch, seq, batch * seq
    if loss not in (None, "onehot", "gather"):
        raise ValueError("loss must be None, 'onehot' or 'gather'")
    b = Builder(dtype)
    shapes = {"token_embedding_table": (V, dim), "rms_att_weight": (L, dim), "wq": (L, dim, dim), "wk": (L, dim, dim), "wv": (L, dim, dim),
              "wo": (L, dim, dim), "rms_ffn_weight": (L, dim), "w1": (L, hidden, dim), "w2": (L, dim, hidden), "w3": (L, hidden, dim),
              "rms_final_weight": (dim,), "wcls": (V, dim)}
    a = {n: b.arg("%" + n, shapes[n]) for n in MODEL_ORDER}
    i32 = lambda shape: "tensor<%s>" % "x".join([str(s) for s in shape] + ["i32"])

    def raw(shape, text):               # an operator whose result the float-typed helpers do not describe
        r = b.new(shape)
        b.lines.append("    %s = %s" % (r, text))
        return r

    idx = raw((T, 1), "stablehlo.reshape %%tokens : (%s) -> %s" % (i32((B, S)), i32((T, 1))))
    rows = b.emit((T, dim), '"stablehlo.gather"(%s, %s) <{dimension_numbers = #stablehlo.gather<offset_dims = [1], '
                            'collapsed_slice_dims = [0], start_index_map = [0], index_vector_dim = 1>, indices_are_sorted = false, '
                            'slice_sizes = array<i64: 1, %d>}> : (%s, %s) -> %s' % (
                                a["token_embedding_table"], idx, dim, b.ty((V, dim)), i32((T, 1)), b.ty((T, dim))))
    x = b.reshape(rows, (B, S, dim))
    tables = _rope_tables(b, S, dim // H, theta, dtype)

    def layer_slice(w, i):
        shape = b.types[w]
        s = b.slice(w, [i] + [0] * (len(shape) - 1), [i + 1] + list(shape[1:]))
        return b.reshape(s, shape[1:])

    for l in range(L):
        x = _layer_rows(b, x, {k: layer_slice(a[k], l) for k in LAYER_ORDER}, H, hidden, tables, eps)
    x = _rmsnorm_rows(b, x, a["rms_final_weight"], eps)
    logits = _linear_rows(b, x, a["wcls"])                                    # [B, S, V]
    order = ["tokens"] + MODEL_ORDER
    sig = ["%%tokens: %s" % i32((B, S))] + ["%s: %s" % (a[n], b.ty(shapes[n])) for n in MODEL_ORDER]
    if loss is None:
        out, out_shape = logits, (B, S, V)
    else:
        order.append("targets")
        sig.append("%%targets: %s" % i32((B, S)))
        full = (B, S, V)
        mx = b.reduce(logits, "maximum", [2])
        shifted = b.binary("subtract", logits, b.bcast(b.bcast(mx, (B, S, 1), (0, 1)), full, (0, 1, 2)))
        se = b.reduce(b.unary("exponential", shifted), "add", [2])
        lg = b.unary("log", b.bcast(se, (B, S, 1), (0, 1)))
        logp = b.binary("subtract", shifted, b.bcast(lg, full, (0, 1, 2)))
        if loss == "onehot":
            t1 = raw((B, S, 1), "stablehlo.broadcast_in_dim %%targets, dims = [0, 1] : (%s) -> %s" % (i32((B, S)), i32((B, S, 1))))
            t2 = raw(full, "stablehlo.broadcast_in_dim %s, dims = [0, 1, 2] : (%s) -> %s" % (t1, i32((B, S, 1)), i32(full)))
            io = raw((1, 1, V), "stablehlo.iota dim = 2 : %s" % i32((1, 1, V)))
            io2 = raw(full, "stablehlo.broadcast_in_dim %s, dims = [0, 1, 2] : (%s) -> %s" % (io, i32((1, 1, V)), i32(full)))
            i1 = "tensor<%s>" % "x".join([str(s_) for s_ in full] + ["i1"])
            eq = raw(full, "stablehlo.compare  EQ, %s, %s,  SIGNED : (%s, %s) -> %s" % (t2, io2, i32(full), i32(full), i1))
            oh = b.emit(full, "stablehlo.convert %s : (%s) -> %s" % (eq, i1, b.ty(full)))
            picked = b.reduce(b.binary("multiply", oh, logp), "add", [2])                     # [B, S]
        else:
            t1 = raw((B, S, 1), "stablehlo.reshape %%targets : (%s) -> %s" % (i32((B, S)), i32((B, S, 1))))
            picked = b.emit((B, S), '"stablehlo.gather"(%s, %s) <{dimension_numbers = #stablehlo.gather<collapsed_slice_dims = [2], '
                                    'operand_batching_dims = [0, 1], start_indices_batching_dims = [0, 1], start_index_map = [2], '
                                    'index_vector_dim = 2>, indices_are_sorted = false, slice_sizes = array<i64: 1, 1, 1>}> : (%s, %s) -> %s' % (
                                        logp, t1, b.ty(full), i32((B, S, 1)), b.ty((B, S))))
        total = b.reduce(picked, "add", [0, 1])
        out = b.unary("negate", b.binary("divide", total, b.const(float(T))))
        out_shape = ()
    head = "module @jit_model {\n  func.func public @main(%s) -> (%s {jax.result_info = \"\"}) {\n" % (", ".join(sig), b.ty(out_shape))
    return head + "\n".join(b.lines) + "\n    return %s : %s\n  }\n}\n" % (out, b.ty(out_shape)), order
