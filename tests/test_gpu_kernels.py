"""GPU parity: every kernel, through the C ABI, against the CPU oracle on the
same seeded inputs.  Tolerances are the contract's: max relative error
(max|got-ref| / max|ref|) 1e-4 for fp32 and 2e-2 for bf16."""
import numpy as np
import pytest
import torch

from oracle import llama_ref as L

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a GPU (run with -m 'not gpu' on CPU)")
    from enzyme_ad.jax import ops as o
    return o


from gpu_util import dev, host, check, rel_err  # noqa: E402


def _say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("rows,dim", [(37, 288), (5, 768), (9, 4096), (3, 8192), (7, 100), (3, 10000), (1, 8)])
def test_rmsnorm_fwd_bwd(ops, dt, rows, dim):
    _say("rmsnorm", dt, rows, dim)
    rng = np.random.default_rng(rows * 1000 + dim)
    x, xr = dev(rng.standard_normal((rows, dim)), dt)
    g, gr = dev(rng.uniform(0.5, 1.5, dim), dt)
    dy, dyr = dev(rng.standard_normal((rows, dim)), dt)
    add, addr = dev(rng.standard_normal((rows, dim)), dt)
    y = ops.rmsnorm(x, g)
    check(y, L.rmsnorm_fwd(xr, gr), dt, "rmsnorm fwd")
    with ops.Tape() as tape:
        y = ops.rmsnorm(x, g)
    dx, dg = tape.backward([y], [dy], [x, g])
    rdx, rdg = L.rmsnorm_bwd(xr, gr, dyr)
    check(dx, rdx, dt, "rmsnorm dx")
    check(dg, rdg, dt, "rmsnorm dgamma")
    # fused residual-cotangent add
    with ops.Tape() as tape:
        y = ops.rmsnorm(x, g)
        z = ops.add(y, x)
    dx2, _ = tape.backward([z], [dy], [x, g])
    check(dx2, rdx + dyr, dt, "rmsnorm dx + residual")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("B,S,h,d", [(2, 33, 6, 48), (1, 128, 4, 128), (2, 17, 3, 64), (1, 9, 2, 6)])
def test_rope_fwd_bwd(ops, dt, B, S, h, d):
    _say("rope", dt, B, S, h, d)
    rng = np.random.default_rng(S * 100 + d)
    x, xr = dev(rng.standard_normal((B, S, h * d)), dt)
    cos, sin = L.rope_angles(S, d)
    y = ops.rope(x, h)
    check(y, L.rope_fwd(xr.reshape(B, S, h, d), cos, sin).reshape(B, S, h * d), dt, "rope fwd")
    dy, dyr = dev(rng.standard_normal((B, S, h * d)), dt)
    with ops.Tape() as tape:
        y = ops.rope(x, h)
    (dx,) = tape.backward([y], [dy], [x])
    check(dx, L.rope_bwd(dyr.reshape(B, S, h, d), cos, sin).reshape(B, S, h * d), dt, "rope bwd")
    # the table itself: float64 angles rounded to fp32
    tab = host(ops.rope_table(S, d))
    assert np.max(np.abs(tab[..., 0] - cos)) < 1e-7 and np.max(np.abs(tab[..., 1] - sin)) < 1e-7


def test_rope_large_positions_fp32(ops):
    """Angles up to ~4095 rad: fp32 angle arithmetic would lose 1e-4; the table is made in float64."""
    B, S, h, d = 1, 4096, 1, 128
    rng = np.random.default_rng(0)
    x, xr = dev(rng.standard_normal((B, S, h * d)), "f32")
    cos, sin = L.rope_angles(S, d)
    check(ops.rope(x, h), L.rope_fwd(xr.reshape(B, S, h, d), cos, sin).reshape(B, S, h * d), "f32", "rope S=4096", 0.1)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("n", [8, 1003, 4096 * 3 + 5])
def test_swiglu_and_add(ops, dt, n):
    _say("swiglu", dt, n)
    rng = np.random.default_rng(n)
    a, ar = dev(rng.standard_normal(n) * 3, dt)
    b, br = dev(rng.standard_normal(n), dt)
    dg, dgr = dev(rng.standard_normal(n), dt)
    check(ops.swiglu(a, b), L.swiglu_fwd(ar, br), dt, "swiglu fwd")
    with ops.Tape() as tape:
        g = ops.swiglu(a, b)
    da, db = tape.backward([g], [dg], [a, b])
    rda, rdb = L.swiglu_bwd(ar, br, dgr)
    check(da, rda, dt, "swiglu da")
    check(db, rdb, dt, "swiglu db")
    check(ops.add(a, b), ar + br, dt, "add")


GEMM_SHAPES = [
    (37, 29, 19),        # generic path (nothing aligned)
    (256, 384, 320),     # fast path, 128-tiles, K not a multiple of 64
    (200, 136, 72),      # fast path, ragged tiles
    (64, 288, 288),      # C1 projection
    (4096, 3072, 264),   # fast path, 256-tiles (192 tiles)
    (4000, 3080, 128),   # 256-tiles, ragged M and N
    (264, 136, 4104),    # few tiles, long contraction: split-K with fp32 partials (bf16 128-tile kernel and fp32 kernel)
    (100, 200, 2600),    # split-K on the generic kernel for both dtypes where M is not a multiple of 8
    (64, 101, 4096),     # split-K with rows of the partials that are not 16-byte aligned (scalar partial stores)
    (256, 288, 32000),   # the logits adjoint dX = dY . Wcls of the 15M model: 50 planes of K
    (2300, 1000, 8264),  # more than 128 tiles of 128, fewer than 192 of 256, long contraction: in the NT bf16 form split-K
                         # on the 256-tile kernel (36 tiles x 4 splits, ragged rows and columns, a ragged last k-tile)
]


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_layouts(ops, dt, ta, tb, M, N, K):
    _say("gemm", dt, ta, tb, M, N, K)
    rng = np.random.default_rng(M + N + K + ta * 2 + tb)
    A = rng.standard_normal((K, M) if ta else (M, K))
    B = rng.standard_normal((N, K) if tb else (K, N))
    R = rng.standard_normal((M, N))
    a, ar = dev(A, dt)
    b, br = dev(B, dt)
    r, rr = dev(R, dt)
    ref = (ar.T if ta else ar) @ (br.T if tb else br)
    check(ops.gemm(a, b, bool(ta), bool(tb)), ref, dt, "gemm")
    check(ops.gemm(a, b, bool(ta), bool(tb), r), ref + rr, dt, "gemm + residual")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,K,pad", [(2049, 1537, 262, 8), (259, 290, 20011, 8)])
def test_gemm_padded_leading_dimensions(ops, dt, ta, tb, M, N, K, pad):
    """emi_gemm_ws through the C ABI on operands that are windows of larger buffers: leading dimensions longer than
    the rows (16-byte aligned rows, so the chunked kernels are taken), sizes that are multiples of nothing: the tiled
    kernels' edge handling in every layout (many tiles; few tiles with planes of K)."""
    import torch
    from enzyme_ad.jax import _native as nat
    _say("gemm padded", dt, ta, tb, M, N, K)
    rng = np.random.default_rng(M + N + K + 5 * ta + 3 * tb)
    ar, ac = (K, M) if ta else (M, K)
    br, bc = (N, K) if tb else (K, N)
    A, Ar = dev(rng.standard_normal((ar, ac + pad)), dt)
    B, Br = dev(rng.standard_normal((br, bc + pad)), dt)
    R, Rr = dev(rng.standard_normal((M, N + pad)), dt)
    C = torch.full((M, N + pad), 7.0, dtype=A.dtype, device="cuda")
    a2, b2 = Ar[:, :ac], Br[:, :bc]
    ref = (a2.T if ta else a2) @ (b2.T if tb else b2) + Rr[:, :N]
    lib = nat.lib()
    code = nat.EMI_F32 if dt == "f32" else nat.EMI_BF16
    nbytes = lib.emi_gemm_workspace_bytes(M, N, K, ta, tb, code)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    nat.check(lib.emi_gemm_ws(torch.cuda.current_stream().cuda_stream, A.data_ptr(), B.data_ptr(), R.data_ptr(), C.data_ptr(),
                            ws.data_ptr(), nbytes, M, N, K, ac + pad, bc + pad, N + pad, N + pad, ta, tb, code))
    check(C[:, :N], ref, dt, "gemm on windows")
    assert bool((C[:, N:] == 7.0).all()), "wrote outside the window"


GROUPED_SHAPES = [
    (256, 384, 320),     # one launch of the 128-tile kernel, K not a multiple of 64
    (200, 136, 72),      # ragged tiles
    (264, 136, 4104),    # few tiles, long contraction: split-K partials per product
    (37, 29, 19),        # nothing aligned: product after product
    (4096, 3072, 264),   # each product fills the chip with 256-tiles on its own: product after product
]


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,K", GROUPED_SHAPES)
def test_gemm_grouped(ops, dt, ta, tb, M, N, K):
    """emi_gemm_grouped: three products of one shape, independent (with a shared A, as q/k/v share the activation)
    and summed into one result, with and without residuals, against fp64 matmul."""
    _say("gemm_grouped", dt, ta, tb, M, N, K)
    rng = np.random.default_rng(M + 3 * N + K + ta * 2 + tb)
    a0, a0r = dev(rng.standard_normal((K, M) if ta else (M, K)), dt)
    As, Ars = [a0, a0], [a0r, a0r]                                     # two products share their A operand
    a2, a2r = dev(rng.standard_normal((K, M) if ta else (M, K)), dt)
    As.append(a2)
    Ars.append(a2r)
    Bs, Brs = zip(*[dev(rng.standard_normal((N, K) if tb else (K, N)), dt) for _ in range(3)])
    Rs, Rrs = zip(*[dev(rng.standard_normal((M, N)), dt) for _ in range(3)])
    prods = [(ar.T if ta else ar) @ (br.T if tb else br) for ar, br in zip(Ars, Brs)]
    outs = ops.gemm_grouped(As, list(Bs), bool(ta), bool(tb))
    for o, ref in zip(outs, prods):
        check(o, ref, dt, "grouped")
    outs = ops.gemm_grouped(As, list(Bs), bool(ta), bool(tb), list(Rs))
    for o, ref, rr in zip(outs, prods, Rrs):
        check(o, ref + rr, dt, "grouped + residual")
    total = sum(prods)
    check(ops.gemm_grouped(As, list(Bs), bool(ta), bool(tb), sum_into_one=True), total, dt, "grouped sum")
    check(ops.gemm_grouped(As, list(Bs), bool(ta), bool(tb), [Rs[0]], sum_into_one=True), total + Rrs[0], dt, "grouped sum + residual")
    # run-to-run identical bits (fixed summation order)
    again = ops.gemm_grouped(As, list(Bs), bool(ta), bool(tb), sum_into_one=True)
    assert torch.equal(again, ops.gemm_grouped(As, list(Bs), bool(ta), bool(tb), sum_into_one=True))


@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("count,M,N,K", [(24, 520, 768, 136), (48, 256, 256, 72), (12, 768, 768, 1032)])
def test_gemm_grouped_many_products(ops, ta, tb, count, M, N, K):
    """Groups large enough to fill the chip with 256 x 256 tiles (the same weight gradient of every layer of a model):
    every product against fp64 matmul, with and without residuals, ragged M."""
    _say("gemm_grouped_many", ta, tb, count, M, N, K)
    rng = np.random.default_rng(count + M + ta * 2 + tb)
    As, Ars = zip(*[dev(rng.standard_normal((K, M) if ta else (M, K)), "bf16") for _ in range(count)])
    Bs, Brs = zip(*[dev(rng.standard_normal((N, K) if tb else (K, N)), "bf16") for _ in range(count)])
    Rs, Rrs = zip(*[dev(rng.standard_normal((M, N)), "bf16") for _ in range(count)])
    prods = [(ar.T if ta else ar) @ (br.T if tb else br) for ar, br in zip(Ars, Brs)]
    for o, ref in zip(ops.gemm_grouped(list(As), list(Bs), bool(ta), bool(tb)), prods):
        check(o, ref, "bf16", "grouped (many)")
    for o, ref, rr in zip(ops.gemm_grouped(list(As), list(Bs), bool(ta), bool(tb), list(Rs)), prods, Rrs):
        check(o, ref + rr, "bf16", "grouped (many) + residual")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_matmul_nt_group_matches_separate_projections(ops, dt):
    """q, k, v = x W^T for three weights of one shape: values, the gradients of x and of every weight, with one of the
    three cotangents missing, and the tangent, against the oracle's linear rule applied three times."""
    rng = np.random.default_rng(8)
    x, xr = dev(rng.standard_normal((2, 130, 136)), dt)
    ws, wrs = zip(*[dev(rng.standard_normal((200, 136)) * 0.1, dt) for _ in range(3)])
    dys, dyrs = zip(*[dev(rng.standard_normal((2, 130, 200)), dt) for _ in range(3)])
    with ops.Tape() as tape:
        ys = ops.matmul_nt_group(x, ws)
    for y, wr in zip(ys, wrs):
        check(y, L.linear_fwd(xr, wr), dt, "group fwd")
    grads = tape.backward(list(ys), list(dys), [x, *ws])
    rdx = sum(L.linear_bwd(xr, wr, dyr)[0] for wr, dyr in zip(wrs, dyrs))
    check(grads[0], rdx, dt, "group dX")
    for g, wr, dyr in zip(grads[1:], wrs, dyrs):
        check(g, L.linear_bwd(xr, wr, dyr)[1], dt, "group dW")
    # the cotangent of k missing: its weight gets no gradient, dX is the sum of the other two
    with ops.Tape() as tape:
        ys = ops.matmul_nt_group(x, ws)
    grads = tape.backward([ys[0], ys[2]], [dys[0], dys[2]], [x, *ws])
    check(grads[0], L.linear_bwd(xr, wrs[0], dyrs[0])[0] + L.linear_bwd(xr, wrs[2], dyrs[2])[0], dt, "group dX, two of three")
    assert grads[2] is None
    check(grads[3], L.linear_bwd(xr, wrs[2], dyrs[2])[1], dt, "group dW, two of three")
    # forward mode
    from enzyme_ad.jax import jvp
    tx, txr = dev(rng.standard_normal((2, 130, 136)), dt)
    tw, twr = dev(rng.standard_normal((200, 136)) * 0.1, dt)
    zero = torch.zeros_like(ws[0])
    _, tans = jvp(lambda a, b, c, d: ops.matmul_nt_group(a, (b, c, d)), (x, *ws), (tx, tw, zero, zero))
    check(tans[0], L.linear_fwd(txr, wrs[0]) + L.linear_fwd(xr, twr), dt, "group tangent q")
    check(tans[1], L.linear_fwd(txr, wrs[1]), dt, "group tangent k")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_matmul_nt_vjp(ops, dt):
    rng = np.random.default_rng(3)
    x, xr = dev(rng.standard_normal((2, 65, 136)), dt)
    w, wr = dev(rng.standard_normal((200, 136)) * 0.1, dt)
    dy, dyr = dev(rng.standard_normal((2, 65, 200)), dt)
    with ops.Tape() as tape:
        y = ops.matmul_nt(x, w)
    check(y, L.linear_fwd(xr, wr), dt, "linear fwd")
    dx, dw = tape.backward([y], [dy], [x, w])
    rdx, rdw = L.linear_bwd(xr, wr, dyr)
    check(dx, rdx, dt, "linear dX")
    check(dw, rdw, dt, "linear dW")


ATTN_CASES = [
    ("f32", 2, 6, 100, 48, "bshd"),     # C1 head shape, ragged sequence: fp32 matrix-core path
    ("f32", 1, 6, 256, 48, "bshd"),     # C1 (stories15M) attention at its own size
    ("f32", 1, 2, 64, 128, "bhsd"),     # fp32 matrix-core path, widest head
    ("f32", 2, 3, 333, 64, "bhsd"),     # several 64-key steps, ragged
    ("f32", 1, 1, 1, 16, "bhsd"),       # single position: out = v
    ("f32", 1, 2, 77, 40, "bshd"),      # head_dim not a multiple of 16: generic path
    ("f32", 2, 2, 50, 6, "bhsd"),       # generic path, rows not 16-byte aligned
    ("bf16", 1, 3, 70, 48, "bshd"),     # bf16 on the generic path
    ("bf16", 2, 2, 256, 128, "bhsd"),   # MFMA path
    ("bf16", 1, 2, 200, 128, "bshd"),   # MFMA, ragged sequence, token-major strides
    ("bf16", 2, 3, 320, 64, "bshd"),    # MFMA, head_dim 64
    ("bf16", 1, 1, 1, 128, "bhsd"),     # single position: out = v
    ("bf16", 1, 2, 130, 64, "bhsd"),
    ("bf16", 1, 2, 600, 128, "bshd"),   # ping-pong forward, several 256-query blocks, ragged
    ("bf16", 1, 2, 1030, 64, "bhsd"),   # ping-pong forward, head_dim 64
    # tile loads that run past the last row of a head (they rely on the buffer descriptor's bounds) with live data
    # of the next head / sequence right behind it
    ("bf16", 2, 2, 513, 128, "bhsd"),   # ping-pong forward just above its threshold: a last key tile of one row
    ("bf16", 2, 2, 577, 64, "bshd"),
    ("bf16", 2, 3, 65, 128, "bhsd"),    # dK/dV with two query tiles, the second of one row
    ("bf16", 2, 2, 191, 64, "bshd"),
]


@pytest.mark.parametrize("dt,B,h,S,d,layout", ATTN_CASES)
@pytest.mark.parametrize("causal", [True, False])
def test_attention_fwd_bwd(ops, dt, B, h, S, d, layout, causal):
    _say("attention", dt, B, h, S, d, layout, causal)
    rng = np.random.default_rng(S * 10 + d + B)
    shp = (B, h, S, d)
    arrs = [rng.standard_normal(shp) for _ in range(4)]

    def put(a):
        if layout == "bshd":
            t, r = dev(a.transpose(0, 2, 1, 3).reshape(B, S, h * d), dt)
            return t, r.reshape(B, S, h, d).transpose(0, 2, 1, 3)
        return dev(a, dt)

    def get(t):
        a = host(t)
        return a.reshape(B, S, h, d).transpose(0, 2, 1, 3) if layout == "bshd" else a

    (q, qr), (k, kr), (v, vr), (do, dor) = (put(a) for a in arrs)
    with ops.Tape() as tape:
        o = ops.attention(q, k, v, h, causal=causal, layout=layout)
    ro, rlse = L.attention_fwd(qr, kr, vr, causal=causal)
    check(get(o), ro, dt, "attention out")
    dq, dk, dv = tape.backward([o], [do], [q, k, v])
    rdq, rdk, rdv = L.attention_bwd(qr, kr, vr, dor, causal=causal)
    check(get(dq), rdq, dt, "attention dq")
    check(get(dk), rdk, dt, "attention dk")
    check(get(dv), rdv, dt, "attention dv")


def test_attention_forward_entry_points_agree(ops):
    """emi_attn_fwd and emi_attn_fwd_ws (which needs no scratch any more: its size query returns 0 and a scratch
    argument is ignored) give the same bits, and match the oracle."""
    from enzyme_ad.jax import _native as N
    B, h, S, d = 1, 3, 700, 128
    rng = np.random.default_rng(11)
    (q, qr), (k, kr), (v, vr) = (dev(rng.standard_normal((B, h, S, d)), "bf16") for _ in range(3))
    lib = N.lib()
    st = torch.cuda.current_stream().cuda_stream
    assert lib.emi_attn_fwd_workspace_bytes(B, h, S, d) == 0
    outs = []
    for use_ws in (False, True):
        o = torch.empty_like(q)
        lse = torch.empty((B, h, S), dtype=torch.float32, device="cuda")
        ws = torch.empty(64, dtype=torch.uint8, device="cuda")
        if use_ws:
            N.check(lib.emi_attn_fwd_ws(st, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                                        ws.data_ptr(), 64, B, h, S, d, h * S * d, S * d, d, d ** -0.5, 1, N.EMI_BF16))
        else:
            N.check(lib.emi_attn_fwd(st, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                                     B, h, S, d, h * S * d, S * d, d, d ** -0.5, 1, N.EMI_BF16))
        outs.append((host(o), host(lse)))
    ro, rlse = L.attention_fwd(qr, kr, vr)
    for o, lse in outs:
        check(o, ro, "bf16", "attention out")
        assert np.max(np.abs(lse - rlse)) < 2e-2
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])


def test_attention_lse_fp32_matrix_core_path(ops):
    """The saved log-sum-exp of the fp32 kernels, ragged sequence (test/llama.py:13-18: max-subtracted softmax)."""
    B, h, S, d = 2, 6, 201, 48
    rng = np.random.default_rng(2)
    (q, qr), (k, kr), (v, vr) = (dev(rng.standard_normal((B, h, S, d)), "f32") for _ in range(3))
    for causal in (True, False):
        o, lse, _ = ops.attention_raw(q, k, v, h, 1.0 / np.sqrt(d), causal, "bhsd")
        ro, rlse = L.attention_fwd(qr, kr, vr, causal=causal)
        assert np.max(np.abs(host(lse) - rlse)) < 1e-5
        check(host(o), ro, "f32", "attention out")


def test_attention_lse(ops):
    B, h, S, d = 1, 2, 192, 128
    rng = np.random.default_rng(1)
    (q, qr), (k, kr), (v, vr) = (dev(rng.standard_normal((B, h, S, d)), "bf16") for _ in range(3))
    o, lse, _ = ops.attention_raw(q, k, v, h, 1.0 / np.sqrt(d), True, "bhsd")
    _, rlse = L.attention_fwd(qr, kr, vr)
    assert np.max(np.abs(host(lse) - rlse)) < 2e-2


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_embedding(ops, dt):
    rng = np.random.default_rng(2)
    V, D = 50, 24
    tab, tabr = dev(rng.standard_normal((V, D)), dt)
    tok = rng.integers(0, V, size=(2, 31))
    tok[0, :5] = 7                                        # collisions
    tt = torch.from_numpy(tok.astype(np.int32)).cuda()
    dx, dxr = dev(rng.standard_normal((2, 31, D)), dt)
    with ops.Tape() as tape:
        x = ops.embedding(tt, tab)
    assert np.array_equal(host(x), tabr[tok])              # a gather is exact
    (dtab,) = tape.backward([x], [dx], [tab])
    ref = np.zeros((V, D))
    np.add.at(ref, tok.reshape(-1), dxr.reshape(-1, D))
    check(dtab, ref, dt, "embedding scatter-add")


def test_error_paths_do_not_launch(ops):
    from enzyme_ad.jax import _native as N
    lib = N.lib()
    x = torch.zeros(16, device="cuda")
    assert lib.emi_rmsnorm_fwd(None, x.data_ptr(), x.data_ptr(), x.data_ptr(), 2, 8, 1e-5, 99) == 3
    assert b"dtype" in lib.emi_last_error()
    assert lib.emi_gemm(None, x.data_ptr(), x.data_ptr(), None, x.data_ptr(), 2, 2, 4, 1, 2, 2, 2, 0, 0, 11) == 3
    assert b"leading dimension" in lib.emi_last_error()
    assert lib.emi_attn_bwd(None, *([x.data_ptr()] * 9), None, 0, 1, 1, 4, 4, 16, 16, 4, 1.0, 1, 11) == 3
    assert b"workspace" in lib.emi_last_error()
    with pytest.raises(RuntimeError):
        ops.add(torch.zeros(4), torch.zeros(4))            # host memory is refused, never computed on CPU
    torch.cuda.synchronize()


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("rows,cols", [(64, 64), (128, 192), (70, 33), (1, 5), (4096, 1032)])
def test_transpose(ops, dt, rows, cols):
    rng = np.random.default_rng(rows + cols)
    a, ar = dev(rng.standard_normal((rows, cols)), dt)
    assert np.array_equal(host(ops.transpose(a)), ar.T)      # a pure permutation is exact


@pytest.mark.parametrize("T,D,Hd,dt", [(2048, 512, 6144, "bf16"),      # one launch each way: 8 x 24 = 192 tiles of 256 x 256
                                       (520, 256, 704, "bf16"),        # ragged: product followed by the elementwise kernel
                                       (300, 128, 352, "f32")])
def test_gemm_swiglu_epilogues(ops, T, D, Hd, dt):
    """emi_gemm_swiglu_fwd / _bwd (the SwiGLU of test/llama.py:224-231 in the epilogue of the product next to it) through
    the C ABI and through their XLA-FFI handlers, against the oracle's linear and SwiGLU rules; and the `ffn` operator
    built on them (value and every gradient) against matmul_nt_group + swiglu + matmul_nt."""
    import ctypes as C
    import ffi_frames as F
    from enzyme_ad.jax import _native as N, vjp
    lib = N.lib()
    st = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(T + Hd)
    x, xr = dev(rng.standard_normal((T, D)), dt)
    w1, w1r = dev(rng.standard_normal((Hd, D)) * 0.1, dt)
    w3, w3r = dev(rng.standard_normal((Hd, D)) * 0.1, dt)
    w2, w2r = dev(rng.standard_normal((D, Hd)) * 0.1, dt)
    dy, dyr = dev(rng.standard_normal((T, D)), dt)
    code = N.EMI_BF16 if dt == "bf16" else N.EMI_F32
    a = ops.gemm(x, w1, False, True)
    b, g = torch.empty_like(a), torch.empty_like(a)
    N.check(lib.emi_gemm_swiglu_fwd(st, x.data_ptr(), w3.data_ptr(), a.data_ptr(), b.data_ptr(), g.data_ptr(), T, Hd, D, code))
    ar_, br_ = host(a), L.linear_fwd(xr, w3r)
    check(b, br_, dt, "b = x w3^T")
    check(g, L.swiglu_fwd(ar_, host(b)), dt, "g = swiglu(a, b)")
    assert torch.equal(b, ops.gemm(x, w3, False, True)) and torch.equal(g, ops.swiglu(a, b))
    w2t = w2.t().contiguous()
    da, db = torch.empty_like(a), torch.empty_like(a)
    nb = lib.emi_gemm_swiglu_bwd_workspace_bytes(T, Hd, D, code)
    ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
    N.check(lib.emi_gemm_swiglu_bwd(st, dy.data_ptr(), w2t.data_ptr(), a.data_ptr(), b.data_ptr(), da.data_ptr(), db.data_ptr(),
                                    ws.data_ptr(), nb, T, Hd, D, code))
    dg = ops.gemm(dy, w2t, False, True)
    rda, rdb = L.swiglu_bwd(host(a), host(b), host(dg))
    check(da, rda, dt, "da")
    check(db, rdb, dt, "db")
    # the handlers
    xla = F.FakeXla(stream=st)
    codes = {torch.float32: F.F32, torch.bfloat16: F.BF16, torch.uint8: F.U8}
    buf = lambda t: xla.buffer(codes[t.dtype], list(t.shape), t.data_ptr())

    def call(name, args, rets):
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = C.c_void_p, [C.POINTER(F.CallFrame)]
        cf = xla.frame(args, rets, {})
        assert fn(C.byref(cf)) is None, (name, xla.errors)

    b2, g2, da2, db2 = (torch.empty_like(a) for _ in range(4))
    call("emi_gemm_swiglu_fwd_ffi", [buf(x), buf(w3), buf(a)], [buf(b2), buf(g2)])
    call("emi_gemm_swiglu_bwd_ffi", [buf(dy), buf(w2t), buf(a), buf(b)], [buf(da2), buf(db2), buf(ws)])
    torch.cuda.synchronize()
    assert torch.equal(b2, b) and torch.equal(g2, g) and torch.equal(da2, da) and torch.equal(db2, db)
    # the operator
    r, rr = dev(rng.standard_normal((T, D)), dt)

    def unfused(x, w1, w3, w2, r):
        h1, h3 = ops.matmul_nt_group(x, (w1, w3))
        return ops.matmul_nt(ops.swiglu(h1, h3), w2, residual=r)

    y0, f0 = vjp(unfused, x, w1, w3, w2, r)
    y1, f1 = vjp(ops.ffn, x, w1, w3, w2, r)
    h = L.swiglu_fwd(L.linear_fwd(xr, w1r), L.linear_fwd(xr, w3r))
    check(y1, L.linear_fwd(h, w2r) + rr, dt, "ffn value")
    for name, u, v in zip(("dx", "dw1", "dw3", "dw2", "dr"), f0(dy), f1(dy)):
        check(v, host(u), dt, "ffn " + name + " against the separate operators", factor=0.5)


@pytest.mark.parametrize("B,S,nh,d,D_in,dt", [(16, 256, 24, 128, 256, "bf16"),    # one launch: 16 x 12 tiles of 256 x 256, MFMA adjoint
                                              (16, 256, 48, 64, 128, "bf16"),     # head_dim 64: a wave strip holds one whole head
                                              (4, 192, 128, 128, 64, "bf16"),     # one launch; wave tiles that straddle two sequences
                                              (2, 200, 4, 64, 96, "bf16"),        # ragged: product + rope pass; MFMA adjoint with a partial block
                                              (2, 40, 3, 16, 48, "f32")])         # generic kernels, rope passes in place
def test_rope_in_epilogues(ops, B, S, nh, d, D_in, dt):
    """emi_gemm_rope (test/llama.py:149-168: a projection with the rotation in its epilogue) and emi_attn_bwd_rope (the
    attention adjoint of :178-206 that hands back the cotangents of q and k before their rotation), through the C ABI and
    their XLA-FFI handlers, against the oracle; and the `attention_block` operator built on them (value and every
    gradient) against the oracle's chain."""
    import ctypes as C
    import ffi_frames as F
    from enzyme_ad.jax import _native as N, vjp
    _say("rope in epilogues", B, S, nh, d, D_in, dt)
    lib = N.lib()
    st = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(B * S + d)
    D, T = nh * d, B * S
    code = N.EMI_BF16 if dt == "bf16" else N.EMI_F32
    x, xr = dev(rng.standard_normal((B, S, D_in)), dt)
    wq, wqr = dev(rng.standard_normal((D, D_in)) * 0.2, dt)
    wk, wkr = dev(rng.standard_normal((D, D_in)) * 0.2, dt)
    wv, wvr = dev(rng.standard_normal((D, D_in)) * 0.2, dt)
    do, dor = dev(rng.standard_normal((B, S, D)), dt)
    table = ops.rope_table(S, d, 10000.0, 0)
    cos, sin = L.rope_angles(S, d)
    # the projection
    q = torch.empty((B, S, D), dtype=x.dtype, device="cuda")
    N.check(lib.emi_gemm_rope(st, x.data_ptr(), wq.data_ptr(), q.data_ptr(), table.data_ptr(), T, D, D_in, S, d, code))
    qr = L.rope_fwd(L.linear_fwd(xr, wqr).reshape(B, S, nh, d), cos, sin).reshape(B, S, D)
    check(q, qr, dt, "rope(x wq^T)")
    k = torch.empty_like(q)
    N.check(lib.emi_gemm_rope(st, x.data_ptr(), wk.data_ptr(), k.data_ptr(), table.data_ptr(), T, D, D_in, S, d, code))
    v = ops.gemm(x.reshape(T, D_in), wv, False, True).reshape(B, S, D)
    # the adjoint: oracle operands are [B, h, S, d]
    o, lse = ops.attention(q, k, v, nh, return_lse=True)
    bhsd = lambda t: host(t).reshape(B, S, nh, d).transpose(0, 2, 1, 3)
    rdq, rdk, rdv = L.attention_bwd(bhsd(q), bhsd(k), bhsd(v), bhsd(do))
    back = lambda a: a.transpose(0, 2, 1, 3)
    rdq = L.rope_bwd(back(rdq), cos, sin).reshape(B, S, D)
    rdk = L.rope_bwd(back(rdk), cos, sin).reshape(B, S, D)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    nb = lib.emi_attn_bwd_workspace_bytes(B, nh, S, d)
    ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
    scale = 1.0 / np.sqrt(d)
    N.check(lib.emi_attn_bwd_rope(st, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), do.data_ptr(),
                                  dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), table.data_ptr(), ws.data_ptr(), nb, B, nh, S, d,
                                  S * D, d, D, scale, 1, code))
    check(dq, rdq, dt, "dq before the rotation")
    check(dk, rdk, dt, "dk before the rotation")
    check(dv, back(rdv).reshape(B, S, D), dt, "dv")
    # the handlers
    xla = F.FakeXla(stream=st)
    codes = {torch.float32: F.F32, torch.bfloat16: F.BF16, torch.uint8: F.U8}
    buf = lambda t, shape=None: xla.buffer(codes[t.dtype], list(t.shape if shape is None else shape), t.data_ptr())

    def call(name, args, rets, attrs):
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = C.c_void_p, [C.POINTER(F.CallFrame)]
        cf = xla.frame(args, rets, attrs)
        assert fn(C.byref(cf)) is None, (name, xla.errors)

    q2 = torch.empty_like(q)
    call("emi_gemm_rope_ffi", [buf(x, (T, D_in)), buf(wq), buf(table)], [buf(q2, (T, D))], {})
    dq2, dk2, dv2 = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    r4 = (B, S, nh, d)
    call("emi_attn_bwd_rope_ffi", [buf(q, r4), buf(k, r4), buf(v, r4), buf(o, r4), buf(lse), buf(do, r4), buf(table)],
         [buf(dq2, r4), buf(dk2, r4), buf(dv2, r4), buf(ws)], {"scale": (F.F32, scale), "causal": (F.PRED, 1), "bshd": (F.PRED, 1)})
    torch.cuda.synchronize()
    assert torch.equal(q2, q) and torch.equal(dq2, dq) and torch.equal(dk2, dk) and torch.equal(dv2, dv)
    # the operator
    y1, f1 = vjp(lambda *a: ops.attention_block(*a, nh), x, wq, wk, wv)
    ro, _ = L.attention_fwd(bhsd(q), bhsd(k), bhsd(v))
    check(y1, back(ro).reshape(B, S, D), dt, "attention_block value")
    rdv = back(rdv).reshape(B, S, D)
    x2r = xr.reshape(T, D_in)
    want = {"dx": (rdq @ wqr + rdk @ wkr + rdv @ wvr), "dwq": rdq.reshape(T, D).T @ x2r, "dwk": rdk.reshape(T, D).T @ x2r,
            "dwv": rdv.reshape(T, D).T @ x2r}
    for name, w in zip(("dx", "dwq", "dwk", "dwv"), f1(do)):
        check(w, want[name], dt, "attention_block " + name)
