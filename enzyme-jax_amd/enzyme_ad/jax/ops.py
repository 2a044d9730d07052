"""Device operators of the llama path and their reverse-mode rules.

This is the lowering table of the MI355X build: where the reference lowers an
`enzyme_jax_ir`-decorated function to optimized StableHLO and lets XLA generate
code (src/enzyme_ad/jax/primitives.py:626-692), each operator here is one
custom-call target (`emi_<op>`) served by a hand-written gfx950 kernel through
the C ABI in include/emi.h.  Tensors are torch CUDA tensors (device memory and
streams only; no torch arithmetic happens on this path).

Every operator records, on the active `Tape`, a rule that maps the cotangent
of its result to the cotangents of its operands.  The rules restate the
reference's StableHLO adjoints for the op clusters test/llama.py traces
(Implementations/HLODerivatives.td: DotGeneral :1166, Mul :1221, Div :1133,
Exp :1182, Sqrt :1320, Add :964; StableHLOAutoDiffOpInterfaceImpl.cpp: Reduce
:1833).  A rule receives the cotangent already accumulated for each operand so
that fan-in sums (Add rule) are fused into the producing kernel's epilogue
instead of costing an extra pass over HBM.
"""
import math

import ctypes
import threading

import torch

from . import _native as N

FFI_TARGETS = {
    # operator        -> (forward target, adjoint target(s))
    "rmsnorm":   ("emi_rmsnorm_fwd", ("emi_rmsnorm_bwd",)),
    "rope":      ("emi_rope", ("emi_rope",)),                    # adjoint = inverse rotation
    "matmul_nt": ("emi_gemm", ("emi_gemm", "emi_gemm")),         # dX (NN) and dW (TN)
    "swiglu":    ("emi_swiglu_fwd", ("emi_swiglu_bwd",)),
    "ffn":       ("emi_gemm_swiglu_fwd", ("emi_gemm_swiglu_bwd", "emi_gemm_grouped", "emi_gemm")),   # between two emi_gemm
    "attention": ("emi_attn_fwd", ("emi_attn_bwd",)),
    "attention_block": ("emi_gemm_rope", ("emi_attn_bwd_rope", "emi_gemm_grouped", "emi_gemm")),  # + emi_gemm (v), emi_attn_fwd
    "attention_step": ("emi_attn_step_fwd", ("emi_attn_step_bwd",)),
    "add":       ("emi_add", ()),
    "embedding": ("emi_embedding_fwd", ("emi_embedding_bwd",)),
    "cross_entropy": ("emi_cross_entropy_fwd", ("emi_cross_entropy_bwd",)),
}

# operator -> tangent target(s); linear operators push tangents through their forward target
FFI_TANGENT_TARGETS = {
    "rmsnorm": ("emi_rmsnorm_jvp",), "rope": ("emi_rope",), "matmul_nt": ("emi_gemm", "emi_gemm"),
    "swiglu": ("emi_swiglu_jvp",), "attention": ("emi_attn_jvp",), "attention_step": ("emi_attn_step_jvp",),
    "add": ("emi_add",), "embedding": ("emi_embedding_fwd",), "cross_entropy": ("emi_cross_entropy_jvp",),
}

_DTYPES = {torch.float32: N.EMI_F32, torch.bfloat16: N.EMI_BF16}


def _code(t):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError("unsupported dtype %s (float32 and bfloat16 only)" % t.dtype) from None


def _dev(*ts):
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("operand is not in device memory: the HIP path has no CPU fallback")
        if not t.is_contiguous():
            raise ValueError("operand must be contiguous")


def _p(t):
    return None if t is None else t.data_ptr()


def _stream():
    # the raw handle of torch's current stream on the current device (torch.cuda.current_stream() builds a Stream
    # object per call: a fifth of the host time of a launch-bound step)
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _same_dtype(*ts):
    d = ts[0].dtype
    for t in ts[1:]:
        if t is not None and t.dtype != d:
            raise TypeError("mixed dtypes: %s vs %s" % (d, t.dtype))


# ---------------------------------------------------------------------------
# tape
# ---------------------------------------------------------------------------

_tls = threading.local()      # the active Tape / Forward context and the running reverse passes of this thread


class _PerThread(type):
    """`Tape._active` / `Forward._active` are per thread: executor threads that differentiate different functions at
    the same time (the reference guards its registries for the same reason, enzyme_call.cc:173,263) never see each
    other's context."""

    @property
    def _active(cls):
        return getattr(_tls, cls.__name__, None)

    @_active.setter
    def _active(cls, value):
        setattr(_tls, cls.__name__, value)


class _Pass:
    """What one Tape.backward call shares between its rules: the in-place gradient buffers of stacked weights, the
    deferred weight-gradient products and the weight transposes.  One object per call, kept on a per-thread stack, so
    that a reverse pass started inside a rule of another one (or on another thread) has its own."""

    def __init__(self, tape):
        ok, other, seen, twice, uses, selects = set(), set(), set(), set(), {}, {}
        for inputs, _, rule in tape.nodes:
            sel = getattr(rule, "_emi_select", None)
            for t in inputs:
                if isinstance(t, torch.Tensor):
                    uses[id(t)] = uses.get(id(t), 0) + 1
                    if sel is None:
                        other.add(id(t))
                    else:
                        ok.add(id(t))
                        selects[id(t)] = selects.get(id(t), 0) + 1
                        if (id(t), sel) in seen:
                            twice.add(id(t))
                        seen.add((id(t), sel))
        # a stacked tensor that an operator on this tape produced (a converted or scaled copy of master weights) is
        # not eligible: its producer's rule runs before the deferred products have written the buffer
        self.ok = ok - other - twice - tape.produced
        self.buf = {}
        self.handed = set()
        self.uses = uses
        self.selects = selects           # id(stack) -> number of slices selected on this tape
        self.pending_dw = []
        self.pending_dw_bytes = 0
        self.transposed = {}             # (data_ptr, shape, dtype) -> (a^T, a)


def _pass():
    stack = getattr(_tls, "passes", None)
    return stack[-1] if stack else None


class Tape(metaclass=_PerThread):
    """Linear record of operator applications for reverse mode."""

    def __init__(self):
        self.nodes = []          # (inputs, output, rule)
        self.produced = set()    # ids of operator results (everything else is a leaf)

    def __enter__(self):
        self._prev = Tape._active
        Tape._active = self
        return self

    def __exit__(self, *exc):
        Tape._active = self._prev
        return False

    @staticmethod
    def record(inputs, output, rule):
        t = Tape._active
        if t is not None:
            t.nodes.append((inputs, output, rule))       # output: a tensor, or a tuple of tensors (one rule for all of them)
            for o in (output if isinstance(output, tuple) else (output,)):
                t.produced.add(id(o))

    def backward(self, outputs, cotangents, wrt):
        """Cotangents of `wrt` (list of tensors) given cotangents of `outputs`."""
        if not hasattr(_tls, "passes"):
            _tls.passes = []
        _tls.passes.append(_Pass(self))
        try:
            return self._backward(outputs, cotangents, wrt)
        finally:
            _tls.passes.pop()            # also on an exception: nothing of the pass outlives it

    def _backward(self, outputs, cotangents, wrt):
        ct = {}
        for o, c in zip(outputs, cotangents):
            if c is None:
                continue
            if c.shape != o.shape or c.dtype != o.dtype:
                raise ValueError("cotangent %s/%s does not match output %s/%s" % (tuple(c.shape), c.dtype, tuple(o.shape), o.dtype))
            ct[id(o)] = c if id(o) not in ct else add(ct[id(o)], c)
        for inputs, output, rule in reversed(self.nodes):
            if isinstance(output, tuple):                # the rule takes the tuple of cotangents (None = zero)
                c = tuple(ct.pop(id(o), None) for o in output)
                if all(x is None for x in c):
                    continue
            else:
                c = ct.pop(id(output), None)
                if c is None:
                    continue
            first, acc = set(), []
            for i in inputs:          # an operand that appears twice gets its fan-in summed afterwards
                fresh = isinstance(i, torch.Tensor) and id(i) not in first
                acc.append(ct.get(id(i)) if fresh else None)
                first.add(id(i))
            new = rule(c, acc)
            done = set()
            for i, g in zip(inputs, new):
                if g is None:
                    continue
                ct[id(i)] = g if id(i) not in done else add(ct[id(i)], g)
                done.add(id(i))
        _flush_dw()
        return [ct.get(id(w)) for w in wrt]


class Forward(metaclass=_PerThread):
    """Forward mode: tangents travel with the primal values.  While a Forward context is
    active every operator also computes the tangent of its result from the tangents of
    its operands (None = zero) with the forward kernels; linear operators reuse their own
    kernel on the tangent."""

    def __init__(self):
        self.tan = {}            # id(primal tensor) -> tangent tensor
        self.keep = []           # primal tensors kept alive so that ids stay unique

    def __enter__(self):
        self._prev = Forward._active
        Forward._active = self
        return self

    def __exit__(self, *exc):
        Forward._active = self._prev
        return False

    def seed(self, primal, tangent):
        if tangent is None:
            return
        if tangent.shape != primal.shape or tangent.dtype != primal.dtype:
            raise ValueError("tangent %s/%s does not match primal %s/%s" %
                             (tuple(tangent.shape), tangent.dtype, tuple(primal.shape), primal.dtype))
        self.tan[id(primal)] = tangent
        self.keep.append(primal)

    def get(self, primal):
        return self.tan.get(id(primal))


def _tan(*ts):
    """Tangents of the operands (None each without an active Forward context)."""
    f = Forward._active
    return None if f is None else tuple(None if t is None else f.get(t) for t in ts)


def _quiet(fn):
    """Runs fn() without recording on the tape and without tangent propagation: used for
    the kernel calls that compute a tangent."""
    tape, fwd = Tape._active, Forward._active
    Tape._active, Forward._active = None, None
    try:
        return fn()
    finally:
        Tape._active, Forward._active = tape, fwd


def _set_tan(y, t):
    if t is not None:
        Forward._active.seed(y, t)


def _accumulate(acc, g):
    return g if acc is None else add(acc, g)


# ---------------------------------------------------------------------------
# operators
# ---------------------------------------------------------------------------

def add(a, b):
    """a + b (test/llama.py:215,233; Add rule HLODerivatives.td:964)."""
    _dev(a, b)
    _same_dtype(a, b)
    if a.shape != b.shape:
        raise ValueError("add: shape mismatch %s vs %s" % (tuple(a.shape), tuple(b.shape)))
    y = torch.empty_like(a)
    N.check(N.lib().emi_add(_stream(), _p(a), _p(b), _p(y), a.numel(), _code(a)))
    Tape.record((a, b), y, lambda c, acc: (_accumulate(acc[0], c), _accumulate(acc[1], c)))
    tans = _tan(a, b)
    if tans is not None and (tans[0] is not None or tans[1] is not None):
        ta, tb = tans
        _set_tan(y, tb if ta is None else ta if tb is None else _quiet(lambda: add(ta, tb)))
    return y


def rmsnorm(x, gamma, eps=1e-5):
    """gamma * x * rsqrt(mean(x^2) + eps) over the last dim (test/llama.py:6-10)."""
    _dev(x, gamma)
    _same_dtype(x, gamma)
    D = x.shape[-1]
    if gamma.shape != (D,):
        raise ValueError("rmsnorm: gamma shape %s != (%d,)" % (tuple(gamma.shape), D))
    rows = x.numel() // D
    y = torch.empty_like(x)
    N.check(N.lib().emi_rmsnorm_fwd(_stream(), _p(x), _p(gamma), _p(y), rows, D, eps, _code(x)))

    def rule(c, acc):
        dx = torch.empty_like(x)
        dgamma = _grad_target(gamma, acc[1])
        if dgamma is None:
            dgamma = torch.empty_like(gamma)
        nbytes = N.lib().emi_rmsnorm_bwd_workspace_bytes(rows, D)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        N.check(N.lib().emi_rmsnorm_bwd(_stream(), _p(x), _p(gamma), _p(c), _p(acc[0]), _p(dx), _p(dgamma), _p(ws),
                                        nbytes, rows, D, eps, _code(x)))
        return dx, _accumulate(acc[1], dgamma)

    Tape.record((x, gamma), y, rule)
    tans = _tan(x, gamma)
    if tans is not None and (tans[0] is not None or tans[1] is not None):
        ty = torch.empty_like(x)
        N.check(N.lib().emi_rmsnorm_jvp(_stream(), _p(x), _p(gamma), _p(tans[0]), _p(tans[1]), _p(ty), rows, D, eps, _code(x)))
        _set_tan(y, ty)
    return y


_rope_tables = {}
_rope_tables_lock = threading.Lock()


def rope_table(seq, head_dim, theta=10000.0, pos0=0, device=None):
    """fp32 (cos, sin) table [seq, head_dim/2, 2]; trace-time constants in the
    reference (test/llama.py:127-140).  Cached per (device, shape, theta, pos0)."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else device
    key = (str(device), seq, head_dim, float(theta), pos0)
    t = _rope_tables.get(key)
    if t is None:
        with _rope_tables_lock:
            t = _rope_tables.get(key)
            if t is None:
                t = torch.empty((seq, head_dim // 2, 2), dtype=torch.float32, device=device)
                N.check(N.lib().emi_rope_table(_stream(), _p(t), seq, head_dim, float(theta), pos0))
                # the table is shared by every stream of the process: it is complete before anyone else can find it
                # (a one-time wait at what is trace time in the reference; never reached under graph capture, whose
                # eager warm-up run has filled the cache)
                if not torch.cuda.is_current_stream_capturing():
                    torch.cuda.current_stream().synchronize()
                _rope_tables[key] = t
    return t


def rope(x, n_heads, theta=10000.0, pos0=0, inverse=False):
    """Rotate adjacent pairs of every head of x [B, S, n_heads*head_dim] by the
    position angle (test/llama.py:161-168)."""
    _dev(x)
    B, S, D = x.shape
    d = D // n_heads
    if d * n_heads != D or d % 2:
        raise ValueError("rope: dim %d is not n_heads=%d x even head_dim" % (D, n_heads))
    table = rope_table(S, d, theta, pos0, x.device)
    y = torch.empty_like(x)
    N.check(N.lib().emi_rope(_stream(), _p(x), _p(table), _p(y), B, S, n_heads, d, int(inverse), _code(x)))

    def rule(c, acc):
        g = torch.empty_like(c)
        N.check(N.lib().emi_rope(_stream(), _p(c), _p(table), _p(g), B, S, n_heads, d, int(not inverse), _code(c)))
        return (_accumulate(acc[0], g),)

    Tape.record((x,), y, rule)
    tans = _tan(x)
    if tans is not None and tans[0] is not None:
        tx = tans[0]
        _set_tan(y, _quiet(lambda: rope(tx, n_heads, theta, pos0, inverse)))     # linear in x
    return y


_STACK_SMALL = 1 << 25        # elements: groups of results up to this size are laid out side by side so that a pair can share a launch


def _adjacent(a, b):
    """b starts where a ends (same shape, dtype, both contiguous): the two are one [2, ...] tensor in memory."""
    return (a.shape == b.shape and a.dtype == b.dtype and a.is_contiguous() and b.is_contiguous()
            and b.data_ptr() == a.data_ptr() + a.numel() * a.element_size())


def rope_pair(q, k, n_heads, theta=10000.0, pos0=0):
    """(rope(q), rope(k)) of test/llama.py:161-168.  When k lies right behind q in memory (the grouped projection lays
    small results out that way) both are rotated by one launch, and so are their cotangents when the attention
    adjoint hands them over the same way: for a small model a launch costs more than the rotation."""
    if not _adjacent(q, k) or q.dim() != 3:
        return rope(q, n_heads, theta, pos0), rope(k, n_heads, theta, pos0)
    _dev(q, k)
    B, S, D = q.shape
    d = D // n_heads
    if d * n_heads != D or d % 2:
        raise ValueError("rope: dim %d is not n_heads=%d x even head_dim" % (D, n_heads))
    table = rope_table(S, d, theta, pos0, q.device)
    ybuf = torch.empty((2, B, S, D), dtype=q.dtype, device=q.device)
    N.check(N.lib().emi_rope(_stream(), _p(q), _p(table), _p(ybuf), 2 * B, S, n_heads, d, 0, _code(q)))
    yq, yk = ybuf[0], ybuf[1]

    def rule(cs, acc):
        cq, ck = cs
        if cq is not None and ck is not None and _adjacent(cq, ck):
            gbuf = torch.empty((2, B, S, D), dtype=cq.dtype, device=cq.device)
            N.check(N.lib().emi_rope(_stream(), _p(cq), _p(table), _p(gbuf), 2 * B, S, n_heads, d, 1, _code(cq)))
            gs = [gbuf[0], gbuf[1]]
        else:
            gs = []
            for c in (cq, ck):
                g = None
                if c is not None:
                    c = c.contiguous()
                    g = torch.empty_like(c)
                    N.check(N.lib().emi_rope(_stream(), _p(c), _p(table), _p(g), B, S, n_heads, d, 1, _code(c)))
                gs.append(g)
        return [None if g is None else _accumulate(a, g) for g, a in zip(gs, acc)]

    Tape.record((q, k), (yq, yk), rule)
    tans = _tan(q, k)
    if tans is not None:
        for y, t in zip((yq, yk), tans):
            if t is not None:
                _set_tan(y, _quiet(lambda t=t: rope(t, n_heads, theta, pos0)))          # linear
    return yq, yk


def rotate_pairs(x, table, inverse=False):
    """Rotate the adjacent pairs (2p, 2p+1) of the last dimension of x by the angles of an
    explicit fp32 (cos, sin) table [pairs, 2]: the batched 2x2 products of
    test/llama.py:161-168 with their constant rotation matrices, as the StableHLO front end
    finds them in a traced module.  Adjoint = rotation by the negated angles."""
    _dev(x, table)
    D = x.shape[-1]
    if table.dtype != torch.float32 or tuple(table.shape) != (D // 2, 2) or D % 2:
        raise ValueError("rotate_pairs: table %s/%s for a last dimension of %d" % (tuple(table.shape), table.dtype, D))
    rows = x.numel() // D
    y = torch.empty_like(x)
    N.check(N.lib().emi_rope(_stream(), _p(x), _p(table), _p(y), rows, 1, 1, D, int(inverse), _code(x)))

    def rule(c, acc):
        g = torch.empty_like(c)
        N.check(N.lib().emi_rope(_stream(), _p(c), _p(table), _p(g), rows, 1, 1, D, int(not inverse), _code(c)))
        return (_accumulate(acc[0], g), None)

    Tape.record((x, table), y, rule)
    tans = _tan(x)
    if tans is not None and tans[0] is not None:
        tx = tans[0]
        _set_tan(y, _quiet(lambda: rotate_pairs(tx, table, inverse)))      # linear in x
    return y


def rope_rows(x, n_heads, table, inverse=False):
    """RoPE over a batch of sequences with an explicit fp32 (cos, sin) table [S, head_dim/2, 2]
    (what the StableHLO front end recovers from a traced module's constants): x is
    [B, S, n_heads*head_dim], position = index along S.  Adjoint = inverse rotation."""
    _dev(x, table)
    B, S, D = x.shape
    d = D // n_heads
    if table.dtype != torch.float32 or tuple(table.shape) != (S, d // 2, 2) or d * n_heads != D or d % 2:
        raise ValueError("rope_rows: table %s for x %s with %d heads" % (tuple(table.shape), tuple(x.shape), n_heads))
    y = torch.empty_like(x)
    N.check(N.lib().emi_rope(_stream(), _p(x), _p(table), _p(y), B, S, n_heads, d, int(inverse), _code(x)))

    def rule(c, acc):
        g = torch.empty_like(c)
        N.check(N.lib().emi_rope(_stream(), _p(c), _p(table), _p(g), B, S, n_heads, d, int(not inverse), _code(c)))
        return (_accumulate(acc[0], g), None)

    Tape.record((x, table), y, rule)
    tans = _tan(x)
    if tans is not None and tans[0] is not None:
        tx = tans[0]
        _set_tan(y, _quiet(lambda: rope_rows(tx, n_heads, table, inverse)))
    return y


def transpose(a):
    """a^T for a 2-D operand (a fresh buffer; Transpose rule HLODerivatives.td:1334)."""
    _dev(a)
    rows, cols = a.shape
    out = torch.empty((cols, rows), dtype=a.dtype, device=a.device)
    N.check(N.lib().emi_transpose(_stream(), _p(a), _p(out), rows, cols, _code(a)))
    Tape.record((a,), out, lambda c, acc: (_accumulate(acc[0], transpose(c)),))
    tans = _tan(a)
    if tans is not None and tans[0] is not None:
        _set_tan(out, _quiet(lambda: transpose(tans[0])))      # linear: the tangent is transposed
    return out


# Gradients of the slices of a stacked per-layer weight (`wq[l]`): when every use of the stacked tensor on the tape is
# a `select`, no slice is selected twice and the stack is a leaf, the kernel that produces a slice's gradient writes it
# straight into slice l of one zero-filled buffer shaped like the stacked tensor, instead of into a temporary that the
# select rule then adds in.  The buffers belong to the running reverse pass (`_Pass`).
#
# Weight gradients dW = dY^T . X whose destination is a slice of such a buffer feed nothing else in the backward
# pass, so they wait: at the end of Tape.backward the products of one shape (the same weight of every layer) run as
# one grouped launch, which fills the chip without split-K partials (12 x [768, 768] over 8192 tokens: 446 -> 173 us).
_PENDING_DW_BYTES = 6 << 30          # cotangents kept alive for the deferred products, at most


def _defer_dw(c2, x2, target):
    ps = _pass()
    ps.pending_dw.append((c2, x2, target))
    ps.pending_dw_bytes += c2.numel() * c2.element_size()
    if ps.pending_dw_bytes > _PENDING_DW_BYTES:
        _flush_dw()


def _flush_dw():
    ps = _pass()
    todo, ps.pending_dw = ps.pending_dw, []
    ps.pending_dw_bytes = 0
    by_shape = {}
    for c2, x2, target in todo:
        by_shape.setdefault((tuple(c2.shape), tuple(x2.shape), c2.dtype), []).append((c2, x2, target))
    for items in by_shape.values():
        for k in range(0, len(items), 48):
            part = items[k:k + 48]
            gemm_grouped([c for c, _, _ in part], [x for _, x, _ in part], True, False, outs=[t for _, _, t in part])


def _stack_buffer(ps, w):
    buf = ps.buf.get(id(w))
    if buf is None:
        buf = ps.buf[id(w)] = torch.zeros_like(w)        # device memset
    return buf


def _grad_target(t, acc):
    """The place the gradient of `t` is to be written to directly, or None (then the producer allocates): `t` is a
    slice of an eligible stacked tensor and the caller is its only consumer (with two, the second would read the first
    one's gradient as its residual before a deferred product has written it)."""
    st = getattr(t, "_emi_stack", None)
    ps = _pass()
    if acc is not None or st is None or ps is None or id(st[0]) not in ps.ok or id(t) in ps.handed or \
            ps.uses.get(id(t), 0) != 1:
        return None
    ps.handed.add(id(t))
    return _stack_buffer(ps, st[0])[st[1]]


def _transpose_shared(a):
    """a^T, computed once per reverse pass however many adjoint GEMMs read it.  A slice of a stacked per-layer
    weight takes its transpose from one batched transpose of the whole stack (one launch for all layers) when at
    least half of the stack's slices are selected on the tape; a pass over one layer of a deep stack transposes
    that slice alone."""
    ps = _pass()
    cache = ps.transposed if ps is not None else {}
    st = getattr(a, "_emi_stack", None)
    if st is not None and st[0].dim() == 3 and st[0].is_contiguous() and ps is not None and \
            2 * ps.selects.get(id(st[0]), 0) >= st[0].shape[0]:
        w, i = st
        skey = ("stack", w.data_ptr(), tuple(w.shape), w.dtype)
        hit = cache.get(skey)
        if hit is None:
            L_, rows, cols = w.shape
            out = torch.empty((L_, cols, rows), dtype=w.dtype, device=w.device)
            i64 = lambda v: (ctypes.c_int64 * len(v))(*v)
            N.check(N.lib().emi_strided_copy(_stream(), _p(w), _p(out), 3, i64([L_, cols, rows]), i64([rows * cols, 1, cols]), 0,
                                             i64([rows * cols, rows, 1]), 0, w.element_size()))
            hit = cache[skey] = (out, w)
        return hit[0][i]
    key = (a.data_ptr(), tuple(a.shape), a.dtype)
    hit = cache.get(key)
    if hit is None:
        rows, cols = a.shape
        out = torch.empty((cols, rows), dtype=a.dtype, device=a.device)
        N.check(N.lib().emi_transpose(_stream(), _p(a), _p(out), rows, cols, _code(a)))
        hit = cache[key] = (out, a)       # keeps `a` alive so the pointer cannot be reused
    return hit[0]


def gemm(a, b, trans_a=False, trans_b=False, residual=None, out=None):
    """op(a) . op(b) [+ residual] on 2-D operands; fp32 accumulate.  out: a contiguous [M, N] tensor to write to."""
    _dev(a, b, residual)
    _same_dtype(a, b, residual)
    M, K = (a.shape[1], a.shape[0]) if trans_a else a.shape
    Kb, Nn = (b.shape[1], b.shape[0]) if trans_b else b.shape
    if K != Kb:
        raise ValueError("gemm: contraction mismatch %d vs %d" % (K, Kb))
    if residual is not None and residual.shape != (M, Nn):
        raise ValueError("gemm: residual shape %s != (%d, %d)" % (tuple(residual.shape), M, Nn))
    if out is not None and (tuple(out.shape) != (M, Nn) or out.dtype != a.dtype or not out.is_contiguous()):
        raise ValueError("gemm: out must be a contiguous [%d, %d] tensor of the operands' dtype" % (M, Nn))
    c = torch.empty((M, Nn), dtype=a.dtype, device=a.device) if out is None else out
    nbytes = N.lib().emi_gemm_workspace_bytes(M, Nn, K, int(trans_a), int(trans_b), _code(a))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=a.device) if nbytes else None
    N.check(N.lib().emi_gemm_ws(_stream(), _p(a), _p(b), _p(residual), _p(c), _p(ws), nbytes, M, Nn, K, a.shape[1],
                                b.shape[1], Nn, Nn, int(trans_a), int(trans_b), _code(a)))
    return c


def _weight_in_place(rows2d, w):
    """dX = dY . W reads W as stored (k-major) rather than through a transposed copy."""
    return rows2d.shape[0] <= 8 or rows2d.dtype == torch.float32


def _ptr_table(ts):
    return (ctypes.c_void_p * len(ts))(*[None if t is None else t.data_ptr() for t in ts])


def gemm_grouped(As, Bs, trans_a=False, trans_b=False, residuals=None, sum_into_one=False, outs=None):
    """Up to 48 products of one shape in one launch (emi_gemm_grouped): the list of op(a_i) . op(b_i) [+ r_i], or, with
    sum_into_one, the single tensor sum_i op(a_i) . op(b_i) [+ r_0]."""
    n = len(As)
    if n != len(Bs) or not 1 <= n <= 48:
        raise ValueError("gemm_grouped: %d / %d operands (1 to 48 pairs wanted)" % (len(As), len(Bs)))
    rs = list(residuals) if residuals is not None else [None] * (1 if sum_into_one else n)
    _dev(*As, *Bs, *rs)
    _same_dtype(*As, *Bs, *rs)
    a, b = As[0], Bs[0]
    if any(t.shape != a.shape for t in As) or any(t.shape != b.shape for t in Bs):
        raise ValueError("gemm_grouped: the products must have one shape")
    M, K = (a.shape[1], a.shape[0]) if trans_a else a.shape
    Kb, Nn = (b.shape[1], b.shape[0]) if trans_b else b.shape
    if K != Kb:
        raise ValueError("gemm_grouped: contraction mismatch %d vs %d" % (K, Kb))
    if any(r is not None and r.shape != (M, Nn) for r in rs):
        raise ValueError("gemm_grouped: residual shape")
    if any(r is None for r in rs) and any(r is not None for r in rs):
        raise ValueError("gemm_grouped: residuals for all results or for none")
    given = list(outs) if outs is not None else [None] * len(rs)
    if len(given) != len(rs) or any(o is not None and (tuple(o.shape) != (M, Nn) or o.dtype != a.dtype or not o.is_contiguous())
                                    for o in given):
        raise ValueError("gemm_grouped: outs must be contiguous [%d, %d] tensors of the operands' dtype, one per result" % (M, Nn))
    if all(o is None for o in given) and 1 < len(given) and len(given) * M * Nn <= _STACK_SMALL:
        given = list(torch.empty((len(given), M, Nn), dtype=a.dtype, device=a.device).unbind(0))     # side by side: see rope_pair
    outs = [torch.empty((M, Nn), dtype=a.dtype, device=a.device) if o is None else o for o in given]
    lib = N.lib()
    nbytes = lib.emi_gemm_grouped_workspace_bytes(n, M, Nn, K, int(trans_a), int(trans_b), int(sum_into_one), _code(a))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=a.device) if nbytes else None
    N.check(lib.emi_gemm_grouped(_stream(), n, _ptr_table(As), _ptr_table(Bs), _ptr_table(rs) if rs[0] is not None else None,
                                 _ptr_table(outs), _p(ws), nbytes, M, Nn, K, a.shape[1], b.shape[1], Nn, Nn, int(trans_a),
                                 int(trans_b), int(sum_into_one), _code(a)))
    return outs[0] if sum_into_one else outs


def _group_rule(x, ws, cs, acc):
    """Reverse rule of (x . w^T for w in ws) for cotangents cs (None = zero) and accumulated cotangents acc of
    (x, *ws): dX as one summed launch, the dW_i grouped, or deferred into their stacked gradients."""
    K, Nout = x.shape[-1], ws[0].shape[0]
    x2 = x.reshape(-1, K)
    live = [i for i, c in enumerate(cs) if c is not None]
    c2 = [cs[i].reshape(-1, Nout) for i in live]
    ax = None if acc[0] is None else acc[0].reshape(-1, K)
    few = _weight_in_place(x2, ws[0])                              # as in matmul_nt
    wb = [ws[i] if few else _transpose_shared(ws[i]) for i in live]
    dx = gemm_grouped(c2, wb, False, not few, None if ax is None else [ax], sum_into_one=True).reshape(x.shape)
    racc = [acc[1 + i] for i in live]
    targets = [_grad_target(ws[i], acc[1 + i]) for i in live]
    if all(t is not None for t in targets):
        for c, t in zip(c2, targets):
            _defer_dw(c, x2, t)
        dws = targets
    elif any(t is not None for t in targets) or (any(r is None for r in racc) and any(r is not None for r in racc)):
        dws = [gemm(c, x2, True, False, r, out=t) for c, r, t in zip(c2, racc, targets)]     # (a target implies r is None)
    else:
        dws = gemm_grouped(c2, [x2] * len(live), True, False, None if racc[0] is None else racc)
    out = [dx] + [None] * len(ws)
    for i, dw in zip(live, dws):
        out[1 + i] = dw
    return out


def matmul_nt_group(x, ws):
    """(x . w^T for w in ws) for two to four weights of one shape applied to the same activation: q, k, v of
    test/llama.py:149-157 and w1, w3 of :224-227 as one launch.  Reverse mode is one rule for the group: the weight
    gradients dW_i = dY_i^T . X as one launch and dX = sum_i dY_i . W_i as one accumulation (the fan-in the Add rule
    would build from three separate adjoints)."""
    ws = list(ws)
    if not 2 <= len(ws) <= 4 or any(w.shape != ws[0].shape or w.dtype != x.dtype for w in ws):
        return tuple(matmul_nt(x, w) for w in ws)
    lead, K, Nout = x.shape[:-1], x.shape[-1], ws[0].shape[0]
    x2 = x.reshape(-1, K)
    ys = tuple(y.reshape(*lead, Nout) for y in gemm_grouped([x2] * len(ws), ws, False, True))

    def rule(cs, acc):
        return _group_rule(x, ws, cs, acc)

    Tape.record((x, *ws), ys, rule)
    tans = _tan(x, *ws)
    if tans is not None and any(t is not None for t in tans):
        tx = tans[0]
        for y, w, tw in zip(ys, ws, tans[1:]):                  # ty = tx W^T + x tW^T
            t = None
            if tx is not None:
                t = gemm(tx.reshape(-1, K), w, False, True, t)
            if tw is not None:
                t = gemm(x2, tw, False, True, t)
            if t is not None:
                _set_tan(y, t.reshape(*lead, Nout))
    return ys


def matmul_nt(x, w, residual=None):
    """Y[..., out] = X[..., in] . W[out, in]^T [+ residual]  (`w @ x` of
    test/llama.py:149-157,211,224-233, batched over tokens)."""
    lead = x.shape[:-1]
    K = x.shape[-1]
    Nout = w.shape[0]
    x2 = x.reshape(-1, K)
    r2 = None if residual is None else residual.reshape(-1, Nout)
    y = gemm(x2, w, False, True, r2).reshape(*lead, Nout)

    def rule(c, acc):
        c2 = c.reshape(-1, Nout)
        ax = None if acc[0] is None else acc[0].reshape(-1, K)
        # dX = dY . W: W is transposed first (2|W| bytes of HBM traffic, shared by nothing
        # else) so that the contraction index is innermost in both operands: the
        # k-contiguous kernel beats the k-major one by more than the transpose costs.
        # With a handful of tokens (the single-token step) W is read in place, once; so it is in fp32, whose
        # kernels read either layout at the same speed.  (Reading small bf16 weights in place was tried for the
        # 768-wide model: the whole step came out 1.4 % slower than with the transposes.)
        if _weight_in_place(c2, w):
            dx = gemm(c2, w, False, False, ax).reshape(x.shape)
        else:
            dx = gemm(c2, _transpose_shared(w), False, True, ax).reshape(x.shape)
        # dW = dY^T . X contracts over tokens, the slow index of both operands: the
        # k-major form of the GEMM kernel reads them in place (transposing LDS loads),
        # 3-7% slower than the k-contiguous form but without two activation-sized
        # transposes per projection.
        target = _grad_target(w, acc[1])
        if target is not None:
            _defer_dw(c2, x2, target)
            dw = target
        else:
            dw = gemm(c2, x2, True, False, acc[1])
        out = [dx, dw]
        if residual is not None:
            out.append(_accumulate(acc[2], c))
        return out

    Tape.record((x, w) if residual is None else (x, w, residual), y, rule)
    tans = _tan(x, w, residual)
    if tans is not None and any(t is not None for t in tans):
        tx, tw, tr = tans                                   # ty = tx W^T + x tW^T + tr
        t = None if tr is None else tr.reshape(-1, Nout)
        if tx is not None:
            t = gemm(tx.reshape(-1, K), w, False, True, t)
        if tw is not None:
            t = gemm(x2, tw, False, True, t)
        _set_tan(y, t.reshape(*lead, Nout))
    return y


def swiglu(a, b):
    """a * sigmoid(a) * b (test/llama.py:21-28,229-231)."""
    _dev(a, b)
    _same_dtype(a, b)
    if a.shape != b.shape:
        raise ValueError("swiglu: shape mismatch")
    g = torch.empty_like(a)
    N.check(N.lib().emi_swiglu_fwd(_stream(), _p(a), _p(b), _p(g), a.numel(), _code(a)))

    def rule(c, acc):
        da, db = torch.empty_like(a), torch.empty_like(b)
        N.check(N.lib().emi_swiglu_bwd(_stream(), _p(a), _p(b), _p(c), _p(da), _p(db), a.numel(), _code(a)))
        return _accumulate(acc[0], da), _accumulate(acc[1], db)

    Tape.record((a, b), g, rule)
    tans = _tan(a, b)
    if tans is not None and (tans[0] is not None or tans[1] is not None):
        tg = torch.empty_like(a)
        N.check(N.lib().emi_swiglu_jvp(_stream(), _p(a), _p(b), _p(tans[0]), _p(tans[1]), _p(tg), a.numel(), _code(a)))
        _set_tan(g, tg)
    return g


def ffn(xb, w1, w3, w2, residual=None):
    """The SwiGLU FFN of test/llama.py:224-233 as one operator: w2 @ (silu(w1 @ xb) * (w3 @ xb)) [+ residual], with the
    elementwise part applied in GEMM epilogues (emi_gemm_swiglu_fwd / _bwd) instead of in passes of their own over
    [tokens, hidden].  The same values and gradients as matmul_nt_group + swiglu + matmul_nt, whose rules it chains:
    h1, h3 = x W1^T, x W3^T;  g = swiglu(h1, h3);  y = g W2^T + r.  Reverse: dW2 = dY^T g; (dh1, dh3) from dY . W2 through
    the SwiGLU adjoint in the product's epilogue; dX = dh1 . W1 + dh3 . W3 as one summed launch; dW1, dW3 grouped.
    Shapes the fused kernels do not serve, fp32, and forward mode take the three separate operators."""
    lead, K = xb.shape[:-1], xb.shape[-1]
    Hn = w1.shape[0]
    fused = (xb.dtype == torch.bfloat16 and Forward._active is None and w1.shape == w3.shape and w2.shape == (K, Hn)
             and w1.dtype == xb.dtype and w3.dtype == xb.dtype and w2.dtype == xb.dtype
             and xb.numel() // K >= 256 and (residual is None or residual.shape == xb.shape))
    if not fused:
        h1, h3 = matmul_nt_group(xb, (w1, w3))
        return matmul_nt(swiglu(h1, h3), w2, residual=residual)
    _dev(xb, w1, w3, w2, residual)
    x2 = xb.reshape(-1, K)
    T = x2.shape[0]
    lib = N.lib()
    h1 = gemm(x2, w1, False, True)
    h3 = torch.empty_like(h1)
    g = torch.empty_like(h1)
    N.check(lib.emi_gemm_swiglu_fwd(_stream(), _p(x2), _p(w3), _p(h1), _p(h3), _p(g), T, Hn, K, _code(x2)))
    r2 = None if residual is None else residual.reshape(-1, K)
    y = gemm(g, w2, False, True, r2).reshape(*lead, K)

    def rule(c, acc):
        c2 = c.reshape(-1, K)
        # w2: dW2 = dY^T . g (deferred when its destination is a slice of a stacked gradient)
        target = _grad_target(w2, acc[3])
        if target is not None:
            _defer_dw(c2, g, target)
            dw2 = target
        else:
            dw2 = gemm(c2, g, True, False, acc[3])
        # (dh1, dh3) = SwiGLU adjoint of dY . W2, in the epilogue of that product
        dh1, dh3 = torch.empty_like(h1), torch.empty_like(h3)
        nbytes = lib.emi_gemm_swiglu_bwd_workspace_bytes(T, Hn, K, _code(c2))
        one_launch = T % 256 == 0 and Hn % 256 == 0 and (T // 256) * (Hn // 256) >= 192      # else dY . W2 goes through a workspace
        ws = None if one_launch else torch.empty(nbytes, dtype=torch.uint8, device=c2.device)
        N.check(lib.emi_gemm_swiglu_bwd(_stream(), _p(c2), _p(_transpose_shared(w2)), _p(h1), _p(h3), _p(dh1), _p(dh3), _p(ws),
                                        nbytes if ws is not None else 0, T, Hn, K, _code(c2)))
        # the group's rule: dX summed over the two branches, dW1 / dW3 grouped or deferred
        ax = None if acc[0] is None else acc[0].reshape(-1, K)
        dx = gemm_grouped([dh1, dh3], [_transpose_shared(w1), _transpose_shared(w3)], False, True, None if ax is None else [ax],
                          sum_into_one=True).reshape(xb.shape)
        t1, t3 = _grad_target(w1, acc[1]), _grad_target(w3, acc[2])
        if t1 is not None and t3 is not None:
            _defer_dw(dh1, x2, t1)
            _defer_dw(dh3, x2, t3)
            dw1, dw3 = t1, t3
        elif t1 is not None or t3 is not None or (acc[1] is None) != (acc[2] is None):
            dw1 = gemm(dh1, x2, True, False, acc[1], out=t1)
            dw3 = gemm(dh3, x2, True, False, acc[2], out=t3)
        else:
            dw1, dw3 = gemm_grouped([dh1, dh3], [x2, x2], True, False, None if acc[1] is None else [acc[1], acc[2]])
        out = [dx, dw1, dw3, dw2]
        if residual is not None:
            out.append(_accumulate(acc[4], c))
        return out

    Tape.record((xb, w1, w3, w2) if residual is None else (xb, w1, w3, w2, residual), y, rule)
    return y


def attention_raw(q, k, v, n_heads, scale, causal, strides):
    B, S = q.shape[0], q.shape[1 if strides == "bshd" else 2]
    d = q.shape[-1] if q.dim() == 4 else q.shape[-1] // n_heads
    if strides == "bshd":
        sb, sh, ss = S * n_heads * d, d, n_heads * d
    else:
        sb, sh, ss = n_heads * S * d, S * d, d
    o = torch.empty_like(q)
    lse = torch.empty((B, n_heads, S), dtype=torch.float32, device=q.device)
    nbytes = N.lib().emi_attn_fwd_workspace_bytes(B, n_heads, S, d) if q.dtype == torch.bfloat16 else 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device) if nbytes else None
    N.check(N.lib().emi_attn_fwd_ws(_stream(), _p(q), _p(k), _p(v), _p(o), _p(lse), _p(ws), nbytes, B, n_heads, S, d,
                                    sb, sh, ss, float(scale), int(causal), _code(q)))
    return o, lse, (B, S, d, sb, sh, ss)


def attention(q, k, v, n_heads, scale=None, causal=True, layout="bshd", return_lse=False):
    """Causal softmax attention (test/llama.py:178-206).  layout "bshd": operands
    are [B, S, n_heads*head_dim] (token-major, as the projections produce them);
    layout "bhsd": [B, n_heads, S, head_dim]."""
    _dev(q, k, v)
    _same_dtype(q, k, v)
    if q.shape != k.shape or q.shape != v.shape:
        raise ValueError("attention: q, k, v shapes differ")
    d = q.shape[-1] // n_heads if layout == "bshd" else q.shape[-1]
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    o, lse, (B, S, d, sb, sh, ss) = attention_raw(q, k, v, n_heads, scale, causal, layout)

    def rule(c, acc):
        if 3 * q.numel() <= _STACK_SMALL and q.is_contiguous():
            dq, dk, dv = torch.empty((3,) + tuple(q.shape), dtype=q.dtype, device=q.device).unbind(0)   # side by side: see rope_pair
        else:
            dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        nbytes = N.lib().emi_attn_bwd_workspace_bytes(B, n_heads, S, d)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
        N.check(N.lib().emi_attn_bwd(_stream(), _p(q), _p(k), _p(v), _p(o), _p(lse), _p(c), _p(dq), _p(dk), _p(dv),
                                     _p(ws), nbytes, B, n_heads, S, d, sb, sh, ss, float(scale), int(causal), _code(q)))
        return _accumulate(acc[0], dq), _accumulate(acc[1], dk), _accumulate(acc[2], dv)

    Tape.record((q, k, v), o, rule)
    tans = _tan(q, k, v)
    if tans is not None and any(t is not None for t in tans):
        to = torch.empty_like(q)
        N.check(N.lib().emi_attn_jvp(_stream(), _p(q), _p(k), _p(v), _p(lse), _p(tans[0]), _p(tans[1]), _p(tans[2]), _p(to),
                                     B, n_heads, S, d, sb, sh, ss, float(scale), int(causal), _code(q)))
        _set_tan(o, to)
    return (o, lse) if return_lse else o


def gemm_rope(x2, w, table):
    """rope(x2 . w^T) as the custom call `emi_gemm_rope` computes it: x2 [T, K] holds whole sequences of
    S = table.shape[0] positions, w [n_heads*head_dim, K], table fp32 [S, head_dim/2, 2] (test/llama.py:149-168).
    Reverse: the cotangent is turned back by the angle, then the DotGeneral rule (dX = c W, dW = c^T X)."""
    _dev(x2, w, table)
    _same_dtype(x2, w)
    if x2.dim() != 2 or w.dim() != 2 or table.dim() != 3 or table.dtype != torch.float32 or table.shape[2] != 2 or not table.is_contiguous():
        raise ValueError("gemm_rope: x %s, w %s, table %s" % (tuple(x2.shape), tuple(w.shape), tuple(table.shape)))
    T_, K = x2.shape
    D, S, d = w.shape[0], table.shape[0], 2 * table.shape[1]
    if w.shape[1] != K or T_ % S or D % d:
        raise ValueError("gemm_rope: x %s, w %s, table %s" % (tuple(x2.shape), tuple(w.shape), tuple(table.shape)))
    lib = N.lib()
    x2 = x2.contiguous()
    y = torch.empty((T_, D), dtype=x2.dtype, device=x2.device)
    N.check(lib.emi_gemm_rope(_stream(), _p(x2), _p(w), _p(y), _p(table), T_, D, K, S, d, _code(x2)))

    def turn(c, inverse):
        g = torch.empty_like(c)
        N.check(lib.emi_rope(_stream(), _p(c), _p(table), _p(g), T_ // S, S, D // d, d, int(inverse), _code(c)))
        return g

    def rule(c, acc):
        return _group_rule(x2, (w,), (turn(c.contiguous(), True),), acc[:2]) + [None]

    Tape.record((x2, w, table), y, rule)
    tans = _tan(x2, w)
    if tans is not None and any(t is not None for t in tans):          # linear in x and in w
        t = None
        if tans[0] is not None:
            t = gemm(tans[0], w, False, True, t)
        if tans[1] is not None:
            t = gemm(x2, tans[1], False, True, t)
        _set_tan(y, turn(t, False))
    return y


def gemm_swiglu(x2, w3, a):
    """(b, g) = (x2 . w3^T, a * sigmoid(a) * b) as the custom call `emi_gemm_swiglu_fwd` computes them (test/llama.py:
    224-231 with a = x2 . w1^T given).  Reverse: (da, db) from the cotangent of g through the SwiGLU adjoint, then the
    DotGeneral rule on the total cotangent of b."""
    _dev(x2, w3, a)
    _same_dtype(x2, w3, a)
    if x2.dim() != 2 or w3.dim() != 2 or w3.shape[1] != x2.shape[1] or tuple(a.shape) != (x2.shape[0], w3.shape[0]):
        raise ValueError("gemm_swiglu: x %s, w3 %s, a %s" % (tuple(x2.shape), tuple(w3.shape), tuple(a.shape)))
    lib = N.lib()
    x2, a = x2.contiguous(), a.contiguous()
    T_, K = x2.shape
    Hn = w3.shape[0]
    b, g = torch.empty_like(a), torch.empty_like(a)
    N.check(lib.emi_gemm_swiglu_fwd(_stream(), _p(x2), _p(w3), _p(a), _p(b), _p(g), T_, Hn, K, _code(x2)))

    def rule(cs, acc):
        cb, cg = cs
        da = None
        if cg is not None:
            da, db = torch.empty_like(a), torch.empty_like(a)
            N.check(lib.emi_swiglu_bwd(_stream(), _p(a), _p(b), _p(cg.contiguous()), _p(da), _p(db), a.numel(), _code(a)))
            cb = db if cb is None else _quiet(lambda: add(cb, db))
        out = _group_rule(x2, (w3,), (cb,), acc[:2]) if cb is not None else [None, None]
        return out + [None if da is None else _accumulate(acc[2], da)]

    Tape.record((x2, w3, a), (b, g), rule)
    tans = _tan(x2, w3, a)
    if tans is not None and any(t is not None for t in tans):
        tx, tw, ta = tans
        tb = None
        if tx is not None:
            tb = gemm(tx, w3, False, True, tb)
        if tw is not None:
            tb = gemm(x2, tw, False, True, tb)
        if tb is not None:
            _set_tan(b, tb)
        tg = torch.empty_like(a)
        N.check(lib.emi_swiglu_jvp(_stream(), _p(a), _p(b), _p(ta), _p(tb), _p(tg), a.numel(), _code(a)))
        _set_tan(g, tg)
    return b, g


def attention_block(xb, wq, wk, wv, n_heads, theta=10000.0, scale=None, causal=True, table=None):
    """The attention sub-block of test/llama.py:149-209 as one operator: q, k, v = xb Wq^T, xb Wk^T, xb Wv^T;
    q, k = rope(q), rope(k); softmax attention.  xb: [B, S, dim]; returns [B, S, n_heads*head_dim].  The rotation of
    q and k is applied in the epilogue of their projections (emi_gemm_rope) and its adjoint where the attention
    adjoint stores dq and dk (emi_attn_bwd_rope), so that the four passes over [tokens, dim] that rope and its
    adjoint would make disappear.  Same values and gradients as matmul_nt_group + rope_pair + attention up to the
    rounding of the unrotated q, k, dq, dk, which here never exist in bf16.  Small shapes, fp32 and forward mode take
    the three separate operators.  `table`: an explicit fp32 (cos, sin) table [S, head_dim/2, 2] instead of the angles
    of `theta` (what the StableHLO front end recovers from a module's constants)."""
    D = wq.shape[0]
    d = D // max(n_heads, 1)
    fused = (xb.dim() == 3 and xb.dtype == torch.bfloat16 and Forward._active is None and wq.shape == wk.shape == wv.shape
             and wq.dtype == wk.dtype == wv.dtype == xb.dtype and wq.dim() == 2 and wq.shape[1] == xb.shape[-1]
             and d * n_heads == D and d in (64, 128))
    proj_fused = False
    if fused:
        T = xb.shape[0] * xb.shape[1]
        proj_fused = T % 256 == 0 and D % 256 == 0 and (T // 256) * (D // 256) >= 192 and xb.shape[1] >= 128
        # smaller projections (one grouped launch, then q and k rotated in place by one launch) still take the
        # attention adjoint that turns dq and dk back as it stores them
        fused = proj_fused or (xb.shape[1] >= 128 and D % 8 == 0 and xb.shape[-1] % 8 == 0)
    if table is not None and (table.dtype != torch.float32 or xb.dim() != 3 or tuple(table.shape) != (xb.shape[1], d // 2, 2)
                              or not table.is_contiguous()):
        raise ValueError("attention_block: table %s for x %s with %d heads" % (tuple(table.shape), tuple(xb.shape), n_heads))
    if not fused:
        q, k, v = matmul_nt_group(xb, (wq, wk, wv))
        if table is None:
            q, k = rope_pair(q, k, n_heads, theta)
        else:
            q, k = rope_rows(q, n_heads, table), rope_rows(k, n_heads, table)
        return attention(q, k, v, n_heads, scale=scale, causal=causal)
    _dev(xb, wq, wk, wv, table)
    B, S, K = xb.shape
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    lib = N.lib()
    x2 = xb.reshape(-1, K)
    if table is None:
        table = rope_table(S, d, theta, 0, xb.device)
    if proj_fused:
        q = torch.empty((B, S, D), dtype=xb.dtype, device=xb.device)
        k = torch.empty_like(q)
        N.check(lib.emi_gemm_rope(_stream(), _p(x2), _p(wq), _p(q), _p(table), T, D, K, S, d, _code(x2)))
        N.check(lib.emi_gemm_rope(_stream(), _p(x2), _p(wk), _p(k), _p(table), T, D, K, S, d, _code(x2)))
        v = gemm(x2, wv, False, True).reshape(B, S, D)
    else:
        q, k, v = (t.reshape(B, S, D) for t in gemm_grouped([x2] * 3, [wq, wk, wv], False, True))
        if _adjacent(q, k):
            N.check(lib.emi_rope(_stream(), _p(q), _p(table), _p(q), 2 * B, S, n_heads, d, 0, _code(q)))
        else:
            for t in (q, k):
                N.check(lib.emi_rope(_stream(), _p(t), _p(table), _p(t), B, S, n_heads, d, 0, _code(t)))
    o, lse, (_, _, _, sb, sh, ss) = attention_raw(q, k, v, n_heads, scale, causal, "bshd")

    def rule(c, acc):
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        nbytes = lib.emi_attn_bwd_workspace_bytes(B, n_heads, S, d)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
        N.check(lib.emi_attn_bwd_rope(_stream(), _p(q), _p(k), _p(v), _p(o), _p(lse), _p(c.contiguous()), _p(dq), _p(dk), _p(dv),
                                      _p(table), _p(ws), nbytes, B, n_heads, S, d, sb, sh, ss, float(scale), int(causal),
                                      _code(q)))
        return _group_rule(xb, (wq, wk, wv), (dq, dk, dv), acc)

    Tape.record((xb, wq, wk, wv), o, rule)
    return o


def reshape(x, shape):
    """x viewed with another shape (Reshape rule, HLODerivatives.td:1271: the cotangent is
    reshaped back)."""
    y = x.reshape(shape)
    Tape.record((x,), y, lambda c, acc: (_accumulate(acc[0], c.reshape(x.shape)),))
    tans = _tan(x)
    if tans is not None and tans[0] is not None:
        _set_tan(y, tans[0].reshape(shape))
    return y


def append_row(cache, row):
    """[cache; row]: the key / value cache of one layer with the current token's row
    appended (`jnp.append`, test/llama.py:170-175).  Adjoint: the cotangent is sliced
    (Concatenate rule, StableHLOAutoDiffOpInterfaceImpl.cpp:2015-2059)."""
    _dev(cache, row)
    _same_dtype(cache, row)
    if cache.dim() != 2 or row.shape != (cache.shape[1],):
        raise ValueError("append_row: cache %s, row %s" % (tuple(cache.shape), tuple(row.shape)))
    out = torch.cat([cache, row[None, :]], dim=0)          # device-to-device copies

    def rule(c, acc):
        n = cache.shape[0]
        return _accumulate(acc[0], c[:n].contiguous()), _accumulate(acc[1], c[n].contiguous())

    Tape.record((cache, row), out, rule)
    tans = _tan(cache, row)
    if tans is not None and (tans[0] is not None or tans[1] is not None):
        tc = torch.zeros_like(cache) if tans[0] is None else tans[0]
        tr = torch.zeros_like(row) if tans[1] is None else tans[1]
        _set_tan(out, torch.cat([tc, tr[None, :]], dim=0))
    return out


def attention_step(q, k_cache, v_cache, n_heads, scale=None, return_lse=False):
    """Attention of one token against its layer's cache (test/llama.py:178-209): q is
    [n_heads*head_dim], the caches are [seq_kv, n_heads*head_dim] and already hold the
    token's own row.  Returns the concatenated per-head outputs [n_heads*head_dim] (with
    return_lse also the fp32 log-sum-exp per head, [1, n_heads], which the adjoint reads)."""
    _dev(q, k_cache, v_cache)
    _same_dtype(q, k_cache, v_cache)
    D = q.shape[-1]
    if q.dim() != 1 or k_cache.dim() != 2 or k_cache.shape != v_cache.shape or k_cache.shape[1] != D or D % n_heads:
        raise ValueError("attention_step: q %s, caches %s / %s, %d heads" %
                         (tuple(q.shape), tuple(k_cache.shape), tuple(v_cache.shape), n_heads))
    S, d = k_cache.shape[0], D // n_heads
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    k_cache, v_cache = k_cache.contiguous(), v_cache.contiguous()
    o = torch.empty_like(q)
    lse = torch.empty((1, n_heads), dtype=torch.float32, device=q.device)
    strides = (D, d, S * D, d, D)              # q: batch, head; cache: batch, head, row
    nbytes = N.lib().emi_attn_step_workspace_bytes(1, n_heads, S, d)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
    N.check(N.lib().emi_attn_step_fwd(_stream(), _p(q), _p(k_cache), _p(v_cache), _p(o), _p(lse), _p(ws), nbytes, 1,
                                      n_heads, S, d, *strides, float(scale), _code(q)))

    def rule(c, acc):
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k_cache), torch.empty_like(v_cache)
        N.check(N.lib().emi_attn_step_bwd(_stream(), _p(q), _p(k_cache), _p(v_cache), _p(o), _p(lse), _p(c), _p(dq),
                                          _p(dk), _p(dv), _p(ws), nbytes, 1, n_heads, S, d, *strides, float(scale),
                                          _code(q)))
        return _accumulate(acc[0], dq), _accumulate(acc[1], dk), _accumulate(acc[2], dv)

    Tape.record((q, k_cache, v_cache), o, rule)
    tans = _tan(q, k_cache, v_cache)
    if tans is not None and any(t is not None for t in tans):
        tq, tk, tv = (None if t is None else t.contiguous() for t in tans)
        to = torch.empty_like(q)
        N.check(N.lib().emi_attn_step_jvp(_stream(), _p(q), _p(k_cache), _p(v_cache), _p(o), _p(lse), _p(tq), _p(tk), _p(tv),
                                          _p(to), _p(ws), nbytes, 1, n_heads, S, d, *strides, float(scale), _code(q)))
        _set_tan(o, to)
    return (o, lse) if return_lse else o


def embedding(tokens, table):
    """table[tokens] (the lookup commented out at test/llama.py:109-113)."""
    _dev(tokens, table)
    if tokens.dtype != torch.int32:
        raise TypeError("embedding: tokens must be int32")
    V, D = table.shape
    x = torch.empty(tuple(tokens.shape) + (D,), dtype=table.dtype, device=table.device)
    N.check(N.lib().emi_embedding_fwd(_stream(), _p(tokens), _p(table), _p(x), tokens.numel(), V, D, _code(table)))

    def rule(c, acc):
        dt = torch.empty_like(table)
        nbytes = N.lib().emi_embedding_bwd_workspace_bytes(V, D, _code(table))
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=table.device)
        N.check(N.lib().emi_embedding_bwd(_stream(), _p(tokens), _p(c), _p(dt), _p(ws), nbytes, tokens.numel(), V, D,
                                          _code(table)))
        return None, _accumulate(acc[1], dt)

    Tape.record((tokens, table), x, rule)
    tans = _tan(table)
    if tans is not None and tans[0] is not None:
        tt = tans[0]
        _set_tan(x, _quiet(lambda: embedding(tokens, tt)))                 # linear in the table
    return x


def cross_entropy(logits, targets, return_lse=False):
    """Per-token softmax cross-entropy `logsumexp(z) - z[target]` of logits `[..., vocab]` against int32 targets
    `[...]`; the losses are fp32 whatever the logits' dtype.  The loss that follows the classifier commented out at
    test/llama.py:236.  Adjoint: `(softmax(z) - onehot) * dloss` from the saved logsumexp; a target outside
    `[0, vocab)` masks its token (zero loss and gradient)."""
    _dev(logits, targets)
    if targets.dtype != torch.int32:
        raise TypeError("cross_entropy: targets must be int32")
    if tuple(targets.shape) != tuple(logits.shape[:-1]):
        raise ValueError("cross_entropy: targets %s do not match logits %s" % (tuple(targets.shape), tuple(logits.shape)))
    V = logits.shape[-1]
    T = targets.numel()
    loss = torch.empty(targets.shape, dtype=torch.float32, device=logits.device)
    lse = torch.empty(targets.shape, dtype=torch.float32, device=logits.device)
    N.check(N.lib().emi_cross_entropy_fwd(_stream(), _p(logits), _p(targets), _p(loss), _p(lse), T, V, _code(logits)))

    def rule(c, acc):
        if c.dtype != torch.float32 or not c.is_contiguous():
            raise TypeError("cross_entropy: the cotangent of the losses must be contiguous float32")
        dz = torch.empty_like(logits)
        N.check(N.lib().emi_cross_entropy_bwd(_stream(), _p(logits), _p(targets), _p(lse), _p(c), _p(dz), T, V,
                                              _code(logits)))
        return _accumulate(acc[0], dz), None

    Tape.record((logits, targets), loss, rule)
    tans = _tan(logits)
    if tans is not None and tans[0] is not None:
        tl = torch.empty_like(loss)
        N.check(N.lib().emi_cross_entropy_jvp(_stream(), _p(logits), _p(targets), _p(lse), _p(tans[0]), _p(tl), T, V,
                                              _code(logits)))
        _set_tan(loss, tl)
    return (loss, lse) if return_lse else loss


def select(w, i):
    """w[i] for a stacked per-layer weight (`wq[i, :, :]`, test/llama.py:149).
    Adjoint (Slice rule, StableHLOAutoDiffOpInterfaceImpl.cpp:1586-1620): the
    cotangent is placed into slice i of a zero tensor shaped like w."""
    _dev(w)
    i = int(i) % w.shape[0]             # w[-1] and w[L-1] are one slice
    y = w[i]
    y._emi_stack = (w, i)

    def rule(c, acc):
        g = acc[0]
        ps = _pass()
        if ps is not None and id(w) in ps.ok:
            # every cotangent of w comes from select rules, one per slice: slice i of the shared buffer is either
            # already written (the producer was handed it) or still zero
            buf = _stack_buffer(ps, w)
            if c.data_ptr() != buf[i].data_ptr():
                buf[i].copy_(c)              # device-to-device copy
            return (buf,)
        if g is not None and getattr(g, "_emi_select_owned", False):
            # a buffer an earlier select rule zero-filled and nobody else holds: add slice i in place
            N.check(N.lib().emi_add(_stream(), _p(g[i]), _p(c), _p(g[i]), c.numel(), _code(c)))
            return (g,)
        fresh = torch.zeros_like(w)          # device memset
        fresh[i].copy_(c)                    # device-to-device copy
        if g is None:
            fresh._emi_select_owned = True
            return (fresh,)
        # the accumulated cotangent came from another rule (it may be shared with another operand or be the
        # caller's own tensor): never written in place
        return (add(g, fresh),)

    rule._emi_select = i
    Tape.record((w,), y, rule)
    tans = _tan(w)
    if tans is not None and tans[0] is not None:
        _set_tan(y, tans[0][i])
    return y
