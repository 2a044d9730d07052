#!/usr/bin/env python3
"""Benchmark of the llama forward + VJP path on one MI355X.

Default workload (the configuration the metric is quoted on):
one Llama-2-7B-shaped decoder layer, dim 4096, SwiGLU hidden 11008, 32 heads of
128, batch 4 x seq 4096, bf16 weights N(0,0.02), activations and output
cotangent N(0,1), RMSNorm eps 1e-5, RoPE theta 10000.  A step is one forward
plus one VJP (all input and weight gradients) through `enzyme_jax_ir` + `vjp`.

Prints ONE JSON line on stdout (everything else goes to stderr):
  value     tokens/s of the whole step, inputs resident in HBM
  roofline  the dominant kernel (the bf16 MFMA GEMM, 21 launches per step):
            algorithmic flops / HIP-event time of exactly those launches
  kernels   the same figure for every other kernel of the path at its
            configuration-C2/C3/C5 shape (HBM GB/s or MFMA TFLOP/s)
            (`vendor`: torch.matmul = hipBLASLt timed on the same launches in the same
            run, a yardstick only: the library is never on the product path; entries
            with a `yardstick` key - a device copy, a plain sum over one weight - say
            what a pass of that size and shape reaches here, next to the transposes and
            the single-token mat-vec kernels they are measured against)
  cpu_baseline  a PyTorch-CPU fp32 restatement of test/llama.py (oracle/llama_torch.py,
            autograd as the VJP) timed on the host cores on a bounded sample
            (reported next to the GPU number, not a target)
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "enzyme-jax_amd"))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E
# HBM-side bytes per GEMM launch (average over the 21 launches of one step) from the
# FETCH_SIZE and WRITE_SIZE counter runs summarised in
# profiles/gemm_bf16_llama7b_layer_hbm_traffic.txt (only valid for the default workload).
GEMM_TRAFFIC_BYTES_PER_LAUNCH = 1.674e9

C5 = dict(dim=4096, hidden_dim=11008, n_heads=32, batch=4, seq=4096)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def event_time(fn, iters, warmup=2):
    """Average seconds per call from HIP events on the current stream."""
    import torch
    st = torch.cuda.current_stream()
    for _ in range(warmup):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    st.synchronize()
    e0.record(st)
    for _ in range(iters):
        fn()
    e1.record(st)
    e1.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / iters


def make_layer_inputs(cfg, seed=5):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    D, H, B, S = cfg["dim"], cfg["hidden_dim"], cfg["batch"], cfg["seq"]

    def n(shape, std):
        return (torch.randn(shape, generator=g, device="cuda", dtype=torch.float32) * std).to(torch.bfloat16)

    lw = {"rms_att_weight": n((D,), 0.02), "wq": n((D, D), 0.02), "wk": n((D, D), 0.02), "wv": n((D, D), 0.02),
          "wo": n((D, D), 0.02), "rms_ffn_weight": n((D,), 0.02), "w1": n((H, D), 0.02), "w2": n((D, H), 0.02),
          "w3": n((H, D), 0.02)}
    x = n((B, S, D), 1.0)
    dy = n((B, S, D), 1.0)
    return x, lw, dy


def layer_flops(cfg):
    D, H, T, S, B, h = cfg["dim"], cfg["hidden_dim"], cfg["batch"] * cfg["seq"], cfg["seq"], cfg["batch"], cfg["n_heads"]
    gemm_fwd = T * (8 * D * D + 6 * D * H)
    attn_fwd = 2 * B * h * S * S * (D // h)
    return dict(gemm=3 * gemm_fwd, attn_fwd=attn_fwd, attn_bwd=2.5 * attn_fwd, total=3 * gemm_fwd + 3.5 * attn_fwd)


def gemm_launches(cfg):
    """(role, M, N, K) of the 21 GEMM launches of one fwd+VJP step.  Y and dX run in the
    NT layout C[M,N] = A[M,K] . B[N,K]^T (the weight is transposed for dX), dW in the TN
    layout C[M,N] = A[K,M]^T . B[K,N] on dY and X as stored (ops.matmul_nt)."""
    D, H, T = cfg["dim"], cfg["hidden_dim"], cfg["batch"] * cfg["seq"]
    out = []
    for (n_out, k_in) in [(D, D)] * 4 + [(H, D)] * 2 + [(D, H)]:
        out.append(("Y", T, n_out, k_in))         # Y  = X W^T
        out.append(("dX", T, k_in, n_out))        # dX = dY (W^T)^T
        out.append(("dW", n_out, k_in, T))        # dW = dY^T X
    return out


def bench_gemms(cfg, iters):
    import torch
    from enzyme_ad.jax import ops
    D, H, T = cfg["dim"], cfg["hidden_dim"], cfg["batch"] * cfg["seq"]
    big = max(D, H)
    flat_a = torch.randn((T * big,), device="cuda").to(torch.bfloat16)
    flat_b = (torch.randn((T * big,), device="cuda") * 0.02).to(torch.bfloat16)
    calls = []
    for (role, M, N, K) in gemm_launches(cfg):
        if role == "dW":
            calls.append((role, flat_a[:M * K].view(K, M), flat_b[:N * K].view(K, N), 2.0 * M * N * K))
        else:
            calls.append((role, flat_a[:M * K].view(M, K), flat_b[:N * K].view(N, K), 2.0 * M * N * K))
    per_role = {}
    for role in ("Y", "dX", "dW"):
        mine = [c for c in calls if c[0] == role]
        ta, tb = (True, False) if role == "dW" else (False, True)
        t = event_time(lambda: [ops.gemm(a, b, ta, tb) for (_, a, b, _) in mine], iters)
        fl = sum(c[3] for c in mine)
        per_role[role] = dict(launches=len(mine), seconds=t, tflops=fl / t / 1e12)
    t_all = event_time(lambda: [ops.gemm(a, b, r == "dW", r != "dW") for (r, a, b, _) in calls], iters)
    # per distinct shape of the forward (NT) products, this library and the vendor library side by side
    per_shape = {}
    for (role, a, b, fl) in calls:
        key = "%s_%dx%dx%d" % (role, a.shape[1] if role == "dW" else a.shape[0], b.shape[1] if role == "dW" else b.shape[0],
                               a.shape[0] if role == "dW" else a.shape[1])
        if key in per_shape:
            continue
        ta, tb = (True, False) if role == "dW" else (False, True)
        # The board sits at its power limit in these kernels and its clock takes milliseconds to settle after a change of
        # load: the two libraries take turns three times and each reports its median turn (one turn each, in a fixed
        # order, differed by 10 % between two identical shapes).
        ven_fn = (lambda: torch.matmul(a.t(), b)) if role == "dW" else (lambda: torch.matmul(a, b.t()))
        t_own, t_ven = [], []
        for _ in range(3):
            t_own.append(event_time(lambda: ops.gemm(a, b, ta, tb), iters))
            t_ven.append(event_time(ven_fn, iters))
        per_shape[key] = dict(tflops=round(fl / sorted(t_own)[1] / 1e12, 1), vendor_tflops=round(fl / sorted(t_ven)[1] / 1e12, 1))
    t_vendor = event_time(lambda: [torch.matmul(a.t(), b) if r == "dW" else torch.matmul(a, b.t()) for (r, a, b, _) in calls], iters)
    vendor = dict(library="torch.matmul (hipBLASLt), same operands, same run; yardstick only",
                  tflops=round(sum(c[3] for c in calls) / t_vendor / 1e12, 1), avg_launch_us=round(t_vendor / len(calls) * 1e6, 1),
                  per_shape=per_shape)
    return t_all, sum(c[3] for c in calls), len(calls), per_role, vendor


def bench_kernels(cfg, iters):
    """Roofline figures of the non-GEMM kernels at their configuration shapes.  The
    launchers are called straight through the C ABI on preallocated buffers so that
    the HIP-event time is kernel time, not host allocation time."""
    import torch
    from enzyme_ad.jax import ops, _native as N
    lib = N.lib()
    st = torch.cuda.current_stream().cuda_stream
    out = {}
    bf = torch.bfloat16

    def P(t):
        return t.data_ptr()

    def graph_time(fn, reps=20):
        """Seconds per call of `fn` inside a HIP graph of `reps` calls: for kernels of 10-20 us, which a Python
        loop of C-ABI calls cannot issue fast enough to keep the queue full (the stream-launch figure of such a
        kernel is the host's call rate, not the kernel)."""
        nonlocal st
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        outer = st
        with torch.cuda.graph(g):
            st = torch.cuda.current_stream().cuda_stream        # the lambdas read `st` when called
            for _ in range(reps):
                fn()
        st = outer
        return event_time(g.replay, iters) / reps

    # under rocprofv3 (which preloads its tool library) the kernels are launched on the stream as usual: the
    # profiler's own kernel durations are the figure of interest there
    profiled = bool(os.environ.get("ROCP_TOOL_LIBRARIES")) or "rocprofiler" in os.environ.get("LD_PRELOAD", "")

    def hbm(name, fn, nbytes, in_graph=False):
        in_graph = in_graph and not profiled
        t = graph_time(fn) if in_graph else event_time(fn, iters)
        out[name] = dict(bound="hbm", achieved=nbytes / t / 1e9, peak=PEAK_HBM_GBS, unit="GB/s",
                         frac=nbytes / t / 1e9 / PEAK_HBM_GBS, us=t * 1e6)
        if in_graph:
            out[name]["timing"] = "HIP events around replays of a HIP graph of 20 launches"

    def mfma(name, fn, flops):
        t = event_time(fn, iters)
        out[name] = dict(bound="mfma", achieved=flops / t / 1e12, peak=PEAK_BF16_TFLOPS, unit="TFLOP/s",
                         frac=flops / t / 1e12 / PEAK_BF16_TFLOPS, us=t * 1e6)

    # C2: x [16, 2048, 4096], bf16 and fp32; RoPE over 32 heads x 128
    for dt, s, code in ((bf, 2, N.EMI_BF16), (torch.float32, 4, N.EMI_F32)):
        tag = "bf16" if dt == bf else "f32"
        rows, D = 16 * 2048, 4096
        x = torch.randn((16, 2048, D), device="cuda").to(dt)
        gam = (torch.rand(D, device="cuda") + 0.5).to(dt)
        dy = torch.randn((16, 2048, D), device="cuda").to(dt)
        y, dgam = torch.empty_like(x), torch.empty_like(gam)
        wsb = lib.emi_rmsnorm_bwd_workspace_bytes(rows, D)
        ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
        table = ops.rope_table(2048, 128)
        n = x.numel()
        hbm("rmsnorm_fwd_" + tag, lambda: N.check(lib.emi_rmsnorm_fwd(st, P(x), P(gam), P(y), rows, D, 1e-5, code)), 2 * n * s)
        hbm("rmsnorm_bwd_" + tag, lambda: N.check(lib.emi_rmsnorm_bwd(st, P(x), P(gam), P(dy), None, P(y), P(dgam), P(ws), wsb,
                                                                      rows, D, 1e-5, code)), 3 * n * s)
        hbm("rmsnorm_jvp_" + tag, lambda: N.check(lib.emi_rmsnorm_jvp(st, P(x), P(gam), P(dy), P(gam), P(y), rows, D, 1e-5, code)), 3 * n * s)
        hbm("rope_fwd_" + tag, lambda: N.check(lib.emi_rope(st, P(x), P(table), P(y), 16, 2048, 32, 128, 0, code)), 2 * n * s)
        hbm("rope_bwd_" + tag, lambda: N.check(lib.emi_rope(st, P(dy), P(table), P(y), 16, 2048, 32, 128, 1, code)), 2 * n * s)
        del x, dy, y, ws
    # Generic operators of the StableHLO front end at the C2 size [32768, 4096]: elementwise maps
    # (multiply reads 2, writes 1; exponential reads 1, writes 1), convert, a row broadcast
    # (writes N), the transpose through the strided copy, and sums over rows and columns.
    from enzyme_ad.jax import hlo_ops as HO
    import ctypes
    rows, D = 16 * 2048, 4096
    n = rows * D
    i64 = lambda xs: (ctypes.c_int64 * len(xs))(*xs)
    for dt, s, code in ((bf, 2, N.EMI_BF16), (torch.float32, 4, N.EMI_F32)):
        tag = "bf16" if dt == bf else "f32"
        a, b = (torch.randn((rows, D), device="cuda").to(dt) for _ in range(2))
        y = torch.empty_like(a)
        row = torch.randn(D, device="cuda").to(dt)
        col = torch.empty(rows, device="cuda").to(dt)
        hbm("map_multiply_" + tag, lambda: N.check(lib.emi_map_binary(st, HO.BINARY["multiply"], P(a), P(b), P(y), n, 0, 0, code)), 3 * n * s)
        hbm("map_exp_" + tag, lambda: N.check(lib.emi_map_unary(st, HO.UNARY["exponential"], P(a), P(y), n, code)), 2 * n * s)
        hbm("broadcast_row_" + tag, lambda: N.check(lib.emi_strided_copy(st, P(row), P(y), 2, i64([rows, D]), i64([0, 1]), 0,
                                                                         i64([D, 1]), 0, s)), n * s)
        hbm("transpose_copy_" + tag, lambda: N.check(lib.emi_strided_copy(st, P(a), P(y), 2, i64([D, rows]), i64([1, D]), 0,
                                                                          i64([rows, 1]), 0, s)), 2 * n * s)
        # what a plain read-and-write pass over the same bytes reaches here: torch's device copy (a yardstick for the
        # transpose above; not a product kernel)
        hbm("device_copy_yardstick_" + tag, lambda: y.copy_(a), 2 * n * s)
        out["device_copy_yardstick_" + tag]["yardstick"] = "torch.Tensor.copy_ of the same [32768, 4096] operand"
        rwb = max(lib.emi_reduce_workspace_bytes(1, rows, D, code), lib.emi_reduce_workspace_bytes(1, n, 1, code), 16)
        rws = torch.empty(rwb, dtype=torch.uint8, device="cuda")
        hbm("reduce_rows_" + tag, lambda: N.check(lib.emi_reduce(st, HO.REDUCE["add"], P(a), P(col), None, 0, rows, D, 1, code)), n * s)
        hbm("reduce_cols_" + tag, lambda: N.check(lib.emi_reduce(st, HO.REDUCE["add"], P(a), P(row), P(rws), rwb, 1, rows, D, code)), n * s)
        hbm("reduce_all_" + tag, lambda: N.check(lib.emi_reduce(st, HO.REDUCE["add"], P(a), P(col), P(rws), rwb, 1, n, 1, code)), n * s)
        mask = torch.empty((rows, D), dtype=torch.bool, device="cuda")
        hbm("compare_" + tag, lambda: N.check(lib.emi_compare(st, HO.COMPARE["GT"], P(a), P(b), P(mask), n, 0, 0, code)), n * (2 * s + 1))
        hbm("select_" + tag, lambda: N.check(lib.emi_select(st, P(mask), P(a), P(b), P(y), n, 0, 0, 0, code)), n * (3 * s + 1))
        del mask
        if dt == torch.float32:
            yb = torch.empty((rows, D), dtype=bf, device="cuda")
            hbm("convert_f32_bf16", lambda: N.check(lib.emi_convert(st, P(a), P(yb), n, N.EMI_F32, N.EMI_BF16)), n * 6)
            del yb
        del a, b, y
    # C5 SwiGLU: [16384, 11008] bf16
    T, H = cfg["batch"] * cfg["seq"], cfg["hidden_dim"]
    a, b, dg = (torch.randn((T, H), device="cuda").to(bf) for _ in range(3))
    da, db = torch.empty_like(a), torch.empty_like(a)
    n = a.numel()
    hbm("swiglu_fwd_bf16", lambda: N.check(lib.emi_swiglu_fwd(st, P(a), P(b), P(da), n, N.EMI_BF16)), 3 * n * 2)
    hbm("swiglu_jvp_bf16", lambda: N.check(lib.emi_swiglu_jvp(st, P(a), P(b), P(dg), P(db), P(da), n, N.EMI_BF16)), 5 * n * 2)
    hbm("swiglu_bwd_bf16", lambda: N.check(lib.emi_swiglu_bwd(st, P(a), P(b), P(dg), P(da), P(db), n, N.EMI_BF16)), 5 * n * 2)
    del a, b, dg, da, db
    # C4 logits: cross-entropy over [8 x 1024 tokens, 32000], bf16 and fp32 (algorithmic bytes: the logits read
    # once forward, read and written once in the adjoint, logits and tangent read once in forward mode)
    Tk, V = 8 * 1024, 32000
    for dt, s, code in ((bf, 2, N.EMI_BF16), (torch.float32, 4, N.EMI_F32)):
        tag = "bf16" if dt == bf else "f32"
        z = (torch.randn((Tk, V), device="cuda") * 3).to(dt)
        tz, dz = torch.randn((Tk, V), device="cuda").to(dt), torch.empty((Tk, V), device="cuda", dtype=dt)
        tgt = torch.randint(0, V, (Tk,), device="cuda", dtype=torch.int32)
        loss, lse_t, dl = (torch.ones(Tk, device="cuda") for _ in range(3))
        hbm("cross_entropy_fwd_" + tag, lambda: N.check(lib.emi_cross_entropy_fwd(st, P(z), P(tgt), P(loss), P(lse_t), Tk, V, code)), Tk * V * s)
        hbm("cross_entropy_bwd_" + tag, lambda: N.check(lib.emi_cross_entropy_bwd(st, P(z), P(tgt), P(lse_t), P(dl), P(dz), Tk, V, code)), 2 * Tk * V * s)
        hbm("cross_entropy_jvp_" + tag, lambda: N.check(lib.emi_cross_entropy_jvp(st, P(z), P(tgt), P(lse_t), P(tz), P(loss), Tk, V, code)), 2 * Tk * V * s)
        del z, tz, dz
    # The four GEMM launches of the C5 step that carry an elementwise part of the layer in their epilogue, priced as the
    # plain product they replace (2 M N K flops): what the epilogue costs is the distance to the plain launch next to it.
    T5, D5, H5, S5, hd5 = cfg["batch"] * cfg["seq"], cfg["dim"], cfg["hidden_dim"], cfg["seq"], cfg["dim"] // cfg["n_heads"]
    x5 = torch.randn((T5, D5), device="cuda").to(bf)
    wq5 = (torch.randn((D5, D5), device="cuda") * 0.02).to(bf)
    w35 = (torch.randn((H5, D5), device="cuda") * 0.02).to(bf)
    w2t5 = (torch.randn((H5, D5), device="cuda") * 0.02).to(bf)
    y5 = torch.empty((T5, D5), device="cuda", dtype=bf)
    a5 = torch.randn((T5, H5), device="cuda").to(bf)
    b5, g5, d5 = (torch.empty((T5, H5), device="cuda", dtype=bf) for _ in range(3))
    tab5 = ops.rope_table(S5, hd5)
    mfma("gemm_plain_16384x4096x4096", lambda: N.check(lib.emi_gemm(st, P(x5), P(wq5), None, P(y5), T5, D5, D5, D5, D5, D5, D5, 0, 1,
                                                                    N.EMI_BF16)), 2.0 * T5 * D5 * D5)
    mfma("gemm_rope_16384x4096x4096", lambda: N.check(lib.emi_gemm_rope(st, P(x5), P(wq5), P(y5), P(tab5), T5, D5, D5, S5, hd5,
                                                                        N.EMI_BF16)), 2.0 * T5 * D5 * D5)
    mfma("gemm_plain_16384x11008x4096", lambda: N.check(lib.emi_gemm(st, P(x5), P(w35), None, P(b5), T5, H5, D5, D5, D5, H5, H5, 0, 1,
                                                                     N.EMI_BF16)), 2.0 * T5 * H5 * D5)
    mfma("gemm_swiglu_fwd_16384x11008x4096", lambda: N.check(lib.emi_gemm_swiglu_fwd(st, P(x5), P(w35), P(a5), P(b5), P(g5), T5, H5, D5,
                                                                                     N.EMI_BF16)), 2.0 * T5 * H5 * D5)
    mfma("gemm_swiglu_bwd_16384x11008x4096", lambda: N.check(lib.emi_gemm_swiglu_bwd(st, P(x5), P(w2t5), P(a5), P(b5), P(g5), P(d5), None,
                                                                                     0, T5, H5, D5, N.EMI_BF16)), 2.0 * T5 * H5 * D5)
    del x5, wq5, w35, w2t5, y5, a5, b5, g5, d5
    # C3: attention [8, 32, 2048, 128] bf16 causal
    B, h, S, d = 8, 32, 2048, 128
    q, k, v, do = (torch.randn((B, h, S, d), device="cuda").to(bf) for _ in range(4))
    o, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
    lse = torch.empty((B, h, S), dtype=torch.float32, device="cuda")
    wsb = lib.emi_attn_bwd_workspace_bytes(B, h, S, d)
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
    sc = d ** -0.5
    fl = 2.0 * B * h * S * S * d
    fwsb = lib.emi_attn_fwd_workspace_bytes(B, h, S, d)
    fws = torch.empty(fwsb, dtype=torch.uint8, device="cuda")
    mfma("attn_fwd_c3", lambda: N.check(lib.emi_attn_fwd_ws(st, P(q), P(k), P(v), P(o), P(lse), P(fws), fwsb, B, h, S, d,
                                                            h * S * d, S * d, d, sc, 1, N.EMI_BF16)), fl)
    mfma("attn_bwd_c3", lambda: N.check(lib.emi_attn_bwd(st, P(q), P(k), P(v), P(o), P(lse), P(do), P(dq), P(dk), P(dv), P(ws), wsb,
                                                         B, h, S, d, h * S * d, S * d, d, sc, 1, N.EMI_BF16)), 2.5 * fl)
    # forward mode: tangent of the same attention, counted like the adjoint at 2.5x the forward flops
    mfma("attn_jvp_c3", lambda: N.check(lib.emi_attn_jvp(st, P(q), P(k), P(v), P(lse), P(do), P(dq), P(dk), P(dv), B, h, S, d,
                                                         h * S * d, S * d, d, sc, 1, N.EMI_BF16)), 2.5 * fl)
    del q, k, v, do, o, dq, dk, dv, ws, fws
    # Single-token (decode) step at the 7B layer's widths: mat-vec over W [11008, 4096] and its
    # adjoints (weight read or written once), attention of one query per head over a
    # 4096-row cache for 8 sequences (cache rows read once; the adjoint also writes dK, dV).
    Bq, hq, Sk, dd = 8, 32, 4096, 128
    Dq = hq * dd
    qs, dos = (torch.randn((Bq, Dq), device="cuda").to(bf) for _ in range(2))
    kc, vc = (torch.randn((Bq, Sk, Dq), device="cuda").to(bf) for _ in range(2))
    os_, dqs = torch.empty_like(qs), torch.empty_like(qs)
    dkc, dvc = torch.empty_like(kc), torch.empty_like(vc)
    lses = torch.empty((Bq, hq), dtype=torch.float32, device="cuda")
    strides = (Dq, dd, Sk * Dq, dd, Dq)
    swb = lib.emi_attn_step_workspace_bytes(Bq, hq, Sk, dd)
    sws = torch.empty(swb, dtype=torch.uint8, device="cuda")
    hbm("step_attn_fwd_bf16", lambda: N.check(lib.emi_attn_step_fwd(st, P(qs), P(kc), P(vc), P(os_), P(lses), P(sws), swb, Bq, hq,
                                                                    Sk, dd, *strides, dd ** -0.5, N.EMI_BF16)), 2 * kc.numel() * 2)
    hbm("step_attn_bwd_bf16", lambda: N.check(lib.emi_attn_step_bwd(st, P(qs), P(kc), P(vc), P(os_), P(lses), P(dos), P(dqs),
                                                                    P(dkc), P(dvc), P(sws), swb, Bq, hq, Sk, dd, *strides,
                                                                    dd ** -0.5, N.EMI_BF16)), 4 * kc.numel() * 2)
    tqs = torch.randn((Bq, Dq), device="cuda").to(bf)
    tkc, tvc = (torch.randn((Bq, Sk, Dq), device="cuda").to(bf) for _ in range(2))
    del dkc, dvc
    hbm("step_attn_jvp_bf16", lambda: N.check(lib.emi_attn_step_jvp(st, P(qs), P(kc), P(vc), P(os_), P(lses), P(tqs), P(tkc), P(tvc),
                                                                    P(dqs), P(sws), swb, Bq, hq, Sk, dd, *strides, dd ** -0.5,
                                                                    N.EMI_BF16)), 4 * kc.numel() * 2)
    del qs, dos, kc, vc, os_, dqs, lses, sws, tqs, tkc, tvc
    # (the graph-timed entries last: stream-launch timings taken after a graph capture came out 10 % lower)
    # Four weights (and four dW results) in rotation: 4 x 90 MB is more than the 256 MB last-level cache keeps next to
    # the other operands, so every launch reads (writes) its matrix from HBM, as a decode step over a whole model does.
    D = cfg["dim"]
    wsr = [(torch.randn((H, D), device="cuda") * 0.02).to(bf) for _ in range(4)]
    dwr = [torch.empty_like(wsr[0]) for _ in range(4)]
    w = wsr[0]
    xv, yv, dyv, dxv = (torch.randn(n_, device="cuda").to(bf) for n_ in (D, H, H, D))
    turn = [0]

    def rot(bufs):
        turn[0] += 1
        return bufs[turn[0] & 3]

    gm = lambda A, Bm, C, M_, N_, K_, lda, ldb, ta, tb: N.check(lib.emi_gemm(st, P(A), P(Bm), None, P(C), M_, N_, K_, lda, ldb,
                                                                             N_, N_, ta, tb, N.EMI_BF16))
    hbm("step_matvec_bf16", lambda: gm(xv, rot(wsr), yv, 1, H, D, D, D, 0, 1), w.numel() * 2, in_graph=True)
    gwb = lib.emi_gemm_workspace_bytes(1, D, H, 0, 0, N.EMI_BF16)
    gws = torch.empty(max(gwb, 16), dtype=torch.uint8, device="cuda")
    hbm("step_matvec_dx_bf16", lambda: N.check(lib.emi_gemm_ws(st, P(dyv), P(rot(wsr)), None, P(dxv), P(gws), gwb, 1, D, H, H, D, D, D,
                                                               0, 0, N.EMI_BF16)), w.numel() * 2, in_graph=True)
    hbm("step_matvec_dw_bf16", lambda: gm(dyv, xv, rot(dwr), H, D, 1, H, D, 1, 0), w.numel() * 2, in_graph=True)
    # what reading such a matrix once costs with nothing else to do: a sum over all its elements, timed the same way
    # (a yardstick for the three mat-vec entries; not a kernel of the step)
    rwb1 = max(lib.emi_reduce_workspace_bytes(1, w.numel(), 1, N.EMI_BF16), 16)
    rws1 = torch.empty(rwb1, dtype=torch.uint8, device="cuda")
    one1 = torch.empty(1, device="cuda").to(bf)
    hbm("step_read_yardstick_bf16", lambda: N.check(lib.emi_reduce(st, HO.REDUCE["add"], P(rot(wsr)), P(one1), P(rws1), rwb1, 1, w.numel(), 1,
                                                                   N.EMI_BF16)), w.numel() * 2, in_graph=True)
    out["step_read_yardstick_bf16"]["yardstick"] = "emi_reduce(add) over one [11008, 4096] matrix, same rotation and timing"
    for k_ in ("step_matvec_bf16", "step_matvec_dx_bf16", "step_matvec_dw_bf16", "step_read_yardstick_bf16"):
        out[k_]["operands"] = "four [11008, 4096] matrices in rotation (360 MB), none of them cache-resident"
    del wsr, dwr, w, gws
    return out


def bench_frontend(iters):
    """The reference's own case (dim 288, hidden 768, 6 layers, 6 heads, fp32) handed over as
    StableHLO text: fwd + VJP of one token at position 255 through the parsed graph, with the
    clusters matched to the fused kernels and operator by operator.  Launch-bound at this size;
    the figure of interest is the ratio."""
    import torch
    from enzyme_ad.jax import stablehlo, vjp
    from enzyme_ad.jax.llama_text import WEIGHT_ORDER, llama_step_text
    cfg = dict(dim=288, hidden_dim=768, n_layers=6, n_heads=6, n_kv_heads=6)
    pos = 255
    text, order = llama_step_text(cfg, pos)
    g = torch.Generator(device="cuda").manual_seed(1)
    shapes = {"x": (288,), "rms_att_weight": (6, 288), "wq": (6, 288, 288), "wk": (6, 288, 288), "wv": (6, 288, 288),
              "wo": (6, 288, 288), "rms_ffn_weight": (6, 288), "w1": (6, 768, 288), "w2": (6, 288, 768), "w3": (6, 768, 288),
              "rms_final_weight": (288,), "key_cache": (6, pos, 288), "value_cache": (6, pos, 288)}
    args = [torch.randn(shapes[n], device="cuda", generator=g) * (0.05 if len(shapes[n]) == 3 and n[0] == "w" else 1.0)
            for n in order]
    dy = torch.randn(288, device="cuda", generator=g)
    out = {}
    for tag, fuse in (("fused", True), ("unfused", False)):
        exe = stablehlo.compile_text(text, fuse=fuse)

        def step():
            y, f_vjp = vjp(lambda *a: exe.run(list(a))[0], *args)
            return f_vjp(dy)

        t = event_time(step, iters)
        out["llama_step_text_" + tag] = dict(us_per_step=round(t * 1e6, 1), operators=len(exe.funcs["main"].ops) - 1,
                                             clusters=exe.fused)
    # the same step written by hand against the operator table (no text, no matcher)
    from enzyme_ad.jax import llama
    named = dict(zip(order, args))
    weights = {k: named[k] for k in WEIGHT_ORDER}
    hcfg = dict(cfg, vocab_size=32000, seq_len=256)

    def hand():
        y, f_vjp = vjp(lambda x, w, kc, vc: llama.forward_step(x, hcfg, w, kc, vc), named["x"], weights,
                       named["key_cache"], named["value_cache"])
        return f_vjp(dy)

    out["llama_step_hand_wired"] = dict(us_per_step=round(event_time(hand, iters) * 1e6, 1))
    # the same two programs captured once into a HIP graph and replayed (the counterpart of the
    # reference's compiled executable): launch and host overhead gone, kernel time left
    from enzyme_ad.jax.graph import capture

    def hand_fn(x, w, kc, vc, dy_):
        y, f_vjp = vjp(lambda a, b, c, d: llama.forward_step(a, hcfg, b, c, d), x, w, kc, vc)
        return y, f_vjp(dy_)

    g = capture(hand_fn, named["x"], weights, named["key_cache"], named["value_cache"], dy)
    out["llama_step_hand_wired_graph"] = dict(
        us_per_step=round(event_time(lambda: g(named["x"], weights, named["key_cache"], named["value_cache"], dy), 4 * iters) * 1e6, 1))
    exe = stablehlo.compile_text(text, fuse=True)

    def text_fn(dy_, *a):
        y, f_vjp = vjp(lambda *b: exe.run(list(b))[0], *a)
        return y, f_vjp(dy_)

    gt = capture(text_fn, dy, *args)
    out["llama_step_text_fused_graph"] = dict(us_per_step=round(event_time(lambda: gt(dy, *args), 4 * iters) * 1e6, 1))
    del g, gt
    # the headline workload handed over as text: one 7B-shaped layer over batch 4 x seq 4096, bf16,
    # matched onto the same GEMM / attention / norm kernels as the hand-wired layer
    from enzyme_ad.jax.llama_text import LAYER_ORDER, llama_layer_text
    c5 = dict(C5)
    ltext, lorder = llama_layer_text(dict(dim=c5["dim"], hidden_dim=c5["hidden_dim"], n_heads=c5["n_heads"]), c5["batch"], c5["seq"], "bf16")
    lexe = stablehlo.compile_text(ltext, fuse=True)
    x, lw, ldy = make_layer_inputs(c5)
    largs = [x] + [lw[k] for k in LAYER_ORDER]

    def layer_step():
        y, f_vjp = vjp(lambda *a: lexe.run(list(a))[0], *largs)
        return f_vjp(ldy)

    t = event_time(layer_step, iters, warmup=2)
    out["llama7b_layer_text_fused"] = dict(ms_per_step=round(t * 1e3, 3), tokens_per_s=round(c5["batch"] * c5["seq"] / t, 1),
                                           operators=len(lexe.funcs["main"].ops) - 1,
                                           clusters={k: v for k, v in lexe.fused.items() if v}, text_bytes=len(ltext))
    return out


def bench_models(iters, only=None):
    """The two whole-model configurations: tokens in, logits out, fwd + VJP with a cotangent on the
    logits (and, as `loss_*`, tokens in, mean cross-entropy out, fwd + VJP).  C4 stories110M (dim 768, hidden 2048, 12 layers, 12 heads x 64, vocab 32000, seq 1024,
    batch 8, bf16) and C1 stories15M (dim 288, hidden 768, 6 layers, 6 heads x 48, seq 256, batch 1,
    fp32)."""
    import torch
    from enzyme_ad.jax import enzyme_jax_ir, JaXPipeline, vjp, llama
    out = {}
    for name, cfg, B, S, dt in (("c4_stories110m_bf16", dict(dim=768, hidden_dim=2048, n_layers=12, n_heads=12, n_kv_heads=12,
                                                            vocab_size=32000, seq_len=1024), 8, 1024, torch.bfloat16),
                                ("c1_stories15m_f32", dict(dim=288, hidden_dim=768, n_layers=6, n_heads=6, n_kv_heads=6,
                                                          vocab_size=32000, seq_len=256), 1, 256, torch.float32)):
        if only is not None and not name.startswith(only):
            continue
        g = torch.Generator(device="cuda").manual_seed(4)
        L_, D, H, V = cfg["n_layers"], cfg["dim"], cfg["hidden_dim"], cfg["vocab_size"]
        n = lambda *shape: (torch.randn(shape, generator=g, device="cuda") * 0.02).to(dt)
        w = {"rms_att_weight": n(L_, D) + 1, "wq": n(L_, D, D), "wk": n(L_, D, D), "wv": n(L_, D, D), "wo": n(L_, D, D),
             "rms_ffn_weight": n(L_, D) + 1, "w1": n(L_, H, D), "w2": n(L_, D, H), "w3": n(L_, H, D), "rms_final_weight": n(D) + 1,
             "token_embedding_table": n(V, D), "wcls": n(V, D)}
        tok = torch.randint(0, V, (B, S), generator=g, device="cuda", dtype=torch.int32)
        dlogits = torch.randn((B, S, V), generator=g, device="cuda").to(dt)

        @enzyme_jax_ir(pipeline_options=JaXPipeline(), inner_jit=False)
        def fn(weights):
            return llama.forward(tok, cfg, weights, logits=True)

        def step():
            y, f_vjp = vjp(fn, w)
            return f_vjp(dlogits)

        t = event_time(step, iters, warmup=2)
        out[name] = dict(ms_per_step=round(t * 1e3, 3), tokens_per_s=round(B * S / t, 1), tokens_per_step=B * S)
        if only is not None:            # profiling run: the logits step alone
            continue
        # the same model as a training step: mean cross-entropy against random targets, all weight gradients
        tgt = torch.randint(0, V, (B, S), generator=g, device="cuda", dtype=torch.int32)
        one = torch.ones((), device="cuda")

        @enzyme_jax_ir(pipeline_options=JaXPipeline(), inner_jit=False)
        def loss_fn(weights):
            return llama.loss(tok, tgt, cfg, weights)

        def loss_step():
            y, f_vjp = vjp(loss_fn, w)
            return f_vjp(one)

        tl = event_time(loss_step, iters, warmup=2)
        out[name]["loss_ms_per_step"] = round(tl * 1e3, 3)
        out[name]["loss_tokens_per_s"] = round(B * S / tl, 1)
        # the same training step handed over as StableHLO text (tokens -> gather -> layers sliced out of the stacked
        # weights -> wcls -> mean softmax cross-entropy in the one-hot spelling), matched onto the same kernels
        from enzyme_ad.jax import stablehlo
        from enzyme_ad.jax.llama_text import MODEL_ORDER, llama_model_text
        mtext, _ = llama_model_text(cfg, B, S, "bf16" if dt == torch.bfloat16 else "f32", "onehot")
        mexe = stablehlo.compile_text(mtext, fuse=True)
        margs = [tok] + [w[k] for k in MODEL_ORDER] + [tgt]
        one_t = torch.ones((), device="cuda", dtype=dt)

        def text_step():
            y, f_vjp = vjp(lambda *a: mexe.run(list(a))[0], *margs)
            return f_vjp(one_t)

        tt = event_time(text_step, iters, warmup=2)
        out[name]["text_fused_loss_ms_per_step"] = round(tt * 1e3, 3)
        out[name]["text_fused_loss_tokens_per_s"] = round(B * S / tt, 1)
        out[name]["text_fused_clusters"] = {k: v for k, v in mexe.fused.items() if v}
        out[name]["text_bytes"] = len(mtext)
        del mexe, margs
        if B * S <= 1024:
            # small enough to be bound by launches and host code: the same step replayed from a HIP graph
            from enzyme_ad.jax.graph import capture

            def step_fn(weights, dl):
                y, f_vjp = vjp(lambda ww: llama.forward(tok, cfg, ww, logits=True), weights)
                return f_vjp(dl)

            gr = capture(step_fn, w, dlogits)
            tg = event_time(lambda: gr(w, dlogits), 4 * iters)
            out[name]["graph_replay_ms_per_step"] = round(tg * 1e3, 3)
            out[name]["graph_replay_tokens_per_s"] = round(B * S / tg, 1)
            del gr
        del w, dlogits
    return out


def _host_threads():
    """Threads for the CPU baseline: the host cores this process may use (the scheduler affinity and an
    OMP_NUM_THREADS limit both bound it)."""
    n = os.cpu_count() or 1
    try:
        n = min(n, len(os.sched_getaffinity(0)))
    except Exception:
        pass
    try:
        n = min(n, int(os.environ.get("OMP_NUM_THREADS", n)))
    except ValueError:
        pass
    return max(n, 1)


def _cpu_model_name():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(cfg, repeats=5, budget_s=25.0):
    """PyTorch-CPU restatement of test/llama.py (oracle/llama_torch.py), forward + autograd VJP in fp32 on all host
    cores this process may use; warm-up 1, then the minimum over up to `repeats` runs (the reference harness reports
    the minimum step time).  Always the 15M whole model (the configuration the reference's CPU path is quoted on); the
    headline `value` is the same 7B layer as the GPU figure on a bounded sample of one 512-token sequence."""
    import torch
    from oracle import llama_torch as LT
    threads = _host_threads()
    torch.set_num_threads(threads)

    def min_time(fn, budget):
        fn()                                            # warm-up
        best, taken, t_start = None, 0, time.perf_counter()
        for _ in range(repeats):
            t0 = time.perf_counter()
            fn()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
            taken += 1
            if time.perf_counter() - t_start > budget:
                break
        return best, taken

    g = torch.Generator().manual_seed(1)
    # C1: dim 288, hidden 768, 6 layers, 6 heads, vocab 32000, batch 1 x seq 256, fp32, cotangent on the logits
    c1 = dict(dim=288, hidden_dim=768, n_layers=6, n_heads=6, vocab_size=32000)
    L_, D1, H1, V1 = c1["n_layers"], c1["dim"], c1["hidden_dim"], c1["vocab_size"]
    shapes = dict(token_embedding_table=(V1, D1), rms_att_weight=(L_, D1), wq=(L_, D1, D1), wk=(L_, D1, D1), wv=(L_, D1, D1),
                  wo=(L_, D1, D1), rms_ffn_weight=(L_, D1), w1=(L_, H1, D1), w2=(L_, D1, H1), w3=(L_, H1, D1),
                  rms_final_weight=(D1,), wcls=(V1, D1))
    w1 = {k: (torch.randn(shp, generator=g) * 0.02).requires_grad_(True) for k, shp in shapes.items()}
    tok = torch.randint(0, V1, (1, 256), generator=g)
    dlogits = torch.randn((1, 256, V1), generator=g)

    def c1_step():
        for t in w1.values():
            t.grad = None
        LT.model(tok, w1, c1, True).backward(dlogits)

    t_c1, n_c1 = min_time(c1_step, 6.0)
    del w1, dlogits

    # the headline layer (dim 4096, hidden 11008, 32 heads) on one sequence of 512 tokens
    D, H, nh = cfg["dim"], cfg["hidden_dim"], cfg["n_heads"]
    B, S = 1, 512
    lw = {k: (torch.randn(shp, generator=g) * 0.02).requires_grad_(True) for k, shp in
          [("rms_att_weight", (D,)), ("wq", (D, D)), ("wk", (D, D)), ("wv", (D, D)), ("wo", (D, D)),
           ("rms_ffn_weight", (D,)), ("w1", (H, D)), ("w2", (D, H)), ("w3", (H, D))]}
    x = torch.randn((B, S, D), generator=g).requires_grad_(True)
    dy = torch.randn((B, S, D), generator=g)

    def layer_step():
        x.grad = None
        for t in lw.values():
            t.grad = None
        LT.layer(x, lw, nh).backward(dy)

    t_layer, n_layer = min_time(layer_step, budget_s - 8.0)
    return dict(value=round(B * S / t_layer, 1), unit="tokens/s", cores=threads, kind="port", cpu=_cpu_model_name(),
                sample="PyTorch-CPU fp32 restatement of test/llama.py (oracle/llama_torch.py), forward + autograd VJP, "
                       "torch.set_num_threads(%d), warm-up 1, min of %d timed runs (at most %d within the time budget): the 7B "
                       "layer of the GPU figure on batch 1 x seq 512 = 512 tokens (%.3f s per step)" % (threads, n_layer, repeats, t_layer),
                c1_stories15m=dict(tokens_per_s=round(256 / t_c1, 1), seconds_per_step=round(t_c1, 4), timed_runs=n_c1,
                                   sample="whole 15M model (dim 288, hidden 768, 6 layers, 6 heads, vocab 32000), "
                                          "batch 1 x seq 256 tokens -> logits, cotangent on the logits, fp32"))


def gemm_replay(cfg, reps):
    """Child mode of `measure_gemm_traffic`: the known-size calibration kernel, then the step's 21 GEMM launches."""
    import torch
    from enzyme_ad.jax import ops
    ca = torch.ones(1 << 28, dtype=torch.bfloat16, device="cuda")
    cb = torch.ones(1 << 28, dtype=torch.bfloat16, device="cuda")
    ops.add(ca, cb)                       # emi::add_kernel: reads 2 x 512 MiB, writes 512 MiB
    torch.cuda.synchronize()
    del ca, cb
    D, H, T = cfg["dim"], cfg["hidden_dim"], cfg["batch"] * cfg["seq"]
    big = max(D, H)
    flat_a = torch.randn((T * big,), device="cuda").to(torch.bfloat16)
    flat_b = (torch.randn((T * big,), device="cuda") * 0.02).to(torch.bfloat16)
    for _ in range(reps):
        for (role, M, N, K) in gemm_launches(cfg):
            if role == "dW":
                ops.gemm(flat_a[:M * K].view(K, M), flat_b[:N * K].view(K, N), True, False)
            else:
                ops.gemm(flat_a[:M * K].view(M, K), flat_b[:N * K].view(N, K), False, True)
    torch.cuda.synchronize()


def measure_gemm_traffic(cfg):
    """HBM-side bytes per GEMM launch, measured now: two child runs of this file under `rocprofv3 --pmc` (FETCH_SIZE,
    then WRITE_SIZE; one counter per run), each replaying the step's 21 GEMM launches after a copy-like kernel of known
    size (emi::add_kernel over 2^28 bf16: reads 1 GiB, writes 512 MiB) whose reading scales the counter.  Returns
    (bytes per launch, note); (None, reason) when the profiler is not available or a run fails."""
    import csv
    import glob
    import shutil
    import subprocess
    import tempfile
    if shutil.which("rocprofv3") is None:
        return None, "rocprofv3 not found"
    known = {"FETCH_SIZE": 2.0 * (1 << 29) / 1024.0, "WRITE_SIZE": 1.0 * (1 << 29) / 1024.0}       # KiB
    per_launch, scales = 0.0, {}
    env = dict(os.environ, TMPDIR="/tmp")
    for ctr in ("FETCH_SIZE", "WRITE_SIZE"):
        out = tempfile.mkdtemp(prefix="emi_pmc_", dir="/tmp")
        try:
            cmd = ["timeout", "-s", "KILL", "120", "rocprofv3", "--pmc", ctr, "--output-format", "csv", "-d", out, "-o", "t", "--",
                   "python3", os.path.abspath(__file__), "--gemm-replay", "1", "--seq", str(cfg["seq"]), "--batch", str(cfg["batch"])]
            r = subprocess.run(cmd, cwd="/tmp", env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
            files = glob.glob(os.path.join(out, "**", "*counter_collection.csv"), recursive=True)
            if r.returncode != 0 or not files:
                return None, "rocprofv3 --pmc %s failed (rc %d)" % (ctr, r.returncode)
            cal, gemm = [], []
            for row in csv.DictReader(open(files[0])):
                if row.get("Counter_Name") != ctr:
                    continue
                name, v = row["Kernel_Name"], float(row["Counter_Value"])
                if "add_kernel" in name:
                    cal.append(v)
                elif "gemm_bf16_pingpong_kernel" in name:
                    gemm.append(v)
            if not cal or not gemm or sum(cal) <= 0:
                return None, "no %s rows for the calibration or GEMM kernels" % ctr
            scales[ctr] = known[ctr] / (sum(cal) / len(cal))
            per_launch += scales[ctr] * (sum(gemm) / len(gemm)) * 1024.0
        finally:
            shutil.rmtree(out, ignore_errors=True)
    return per_launch, ("measured in this run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (one counter per child run of "
                        "`bench.py --gemm-replay 1`), scaled by the same counter's reading for emi::add_kernel over 2^28 bf16 "
                        "(factors %.3f / %.3f)" % (scales["FETCH_SIZE"], scales["WRITE_SIZE"]))


def power_probe(cfg, seconds=4.0):
    """Shader clock and socket power (amd-smi, sampled from a side thread) while one kernel family runs back to back,
    with the rate it achieves: the step's 21 GEMM launches on N(0,1) x N(0,0.02) operands, the same on all-zero
    operands (same binary, no switching in the data paths), causal attention forward and backward at the step's shape,
    and the whole step.  Prints a text table (the content of profiles/power_clock_summary.txt)."""
    import statistics
    import subprocess
    import threading
    import torch
    from enzyme_ad.jax import ops, enzyme_jax_ir, JaXPipeline, vjp, llama

    def sample():
        try:
            r = subprocess.run(["amd-smi", "metric", "-p", "-c", "--json"], stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True, timeout=5)
            g = json.loads(r.stdout)
            g = g["gpu_data"][0] if isinstance(g, dict) else g[0]
            clk = [v["clk"]["value"] for k, v in g["clock"].items() if k.startswith("gfx_") and isinstance(v["clk"], dict)]
            return float(g["power"]["socket_power"]["value"]), float(sum(clk)) / len(clk)
        except Exception:                                        # noqa: BLE001
            return None

    def run(name, fn, flops_per_call):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        samples, stop = [], threading.Event()

        def poll():
            time.sleep(0.8)                                      # past the clock ramp from idle
            while not stop.is_set():
                s_ = sample()
                if s_ is not None:
                    samples.append(s_)
                time.sleep(0.1)

        th = threading.Thread(target=poll)
        th.start()
        calls, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(4):
                fn()
                calls += 1
            torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        stop.set()
        th.join()
        pw = [s_[0] for s_ in samples]
        ck = [s_[1] for s_ in samples]
        row = dict(name=name, tflops=flops_per_call * calls / dt / 1e12, samples=len(samples),
                   power_w=(statistics.median(pw), min(pw), max(pw)) if pw else None,
                   clock_mhz=(statistics.median(ck), min(ck), max(ck)) if ck else None)
        print("%-58s %8.1f TFLOP/s  %s  %s  (%d samples)" % (
            name, row["tflops"],
            "power %4.0f W (%4.0f-%4.0f)" % row["power_w"] if pw else "power n/a",
            "shader clock %4.0f MHz (%4.0f-%4.0f)" % row["clock_mhz"] if ck else "clock n/a", len(samples)), flush=True)
        return row

    D, H, T = cfg["dim"], cfg["hidden_dim"], cfg["batch"] * cfg["seq"]
    big = max(D, H)
    launches = gemm_launches(cfg)
    gfl = sum(2.0 * M * N * K for (_, M, N, K) in launches)
    rows = []
    for tag, zero in (("N(0,1) x N(0,0.02) operands", False), ("all-zero operands (same binary)", True)):
        fa = torch.randn((T * big,), device="cuda").to(torch.bfloat16)
        fb = (torch.randn((T * big,), device="cuda") * 0.02).to(torch.bfloat16)
        if zero:
            fa.zero_()
            fb.zero_()

        def gemms():
            for (role, M, N, K) in launches:
                if role == "dW":
                    ops.gemm(fa[:M * K].view(K, M), fb[:N * K].view(K, N), True, False)
                else:
                    ops.gemm(fa[:M * K].view(M, K), fb[:N * K].view(N, K), False, True)

        rows.append(run("GEMM, the step's 21 launches, " + tag, gemms, gfl))
        del fa, fb
    B, S, nh = cfg["batch"], cfg["seq"], cfg["n_heads"]
    fl = layer_flops(cfg)
    for tag, zero in (("N(0,1) operands", False), ("all-zero operands", True)):
        q, k, v, do = (torch.randn((B, S, D), device="cuda").to(torch.bfloat16) for _ in range(4))
        if zero:
            for t_ in (q, k, v, do):
                t_.zero_()
        rows.append(run("attention forward [%d, %d, %d x %d], " % (B, S, nh, D // nh) + tag, lambda: ops.attention(q, k, v, nh), fl["attn_fwd"]))
        with ops.Tape() as tape:
            o = ops.attention(q, k, v, nh)
        rows.append(run("attention adjoint (dQ, dK, dV), " + tag, lambda: tape.backward([o], [do], [q, k, v]), fl["attn_bwd"]))
        del q, k, v, do, o, tape
    x, lw, dy = make_layer_inputs(cfg)

    @enzyme_jax_ir(pipeline_options=JaXPipeline(), inner_jit=False)
    def layer_fn(x, lw):
        return llama.layer(x, lw, nh)

    def step():
        out, f_vjp = vjp(layer_fn, x, lw)
        return f_vjp(dy)

    rows.append(run("whole step (forward + VJP of the layer)", step, fl["total"]))
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel roofline table")
    ap.add_argument("--no-frontend", action="store_true", help="skip the StableHLO front end timing (thousands of tiny launches)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run one emi_add over 3 x 512 MiB (reads 1 GiB, writes 512 MiB): the known-size kernel "
                         "that FETCH_SIZE / WRITE_SIZE counter runs are scaled by")
    ap.add_argument("--only-model", choices=["c1", "c4"], default=None,
                    help="run only the fwd + VJP steps of one whole-model configuration (c1 = stories15M fp32, c4 = "
                         "stories110M bf16) and print its timing: the command kernel traces of those models are taken from")
    ap.add_argument("--gemm-replay", type=int, default=0, metavar="REPS",
                    help="child mode of the traffic measurement: the calibration kernel and REPS replays of the step's 21 "
                         "GEMM launches, nothing else")
    ap.add_argument("--power-probe", action="store_true",
                    help="sample shader clock and socket power (amd-smi) while GEMM, attention and the whole step run back "
                         "to back, on random and on all-zero operands; prints a table")
    ap.add_argument("--no-traffic", action="store_true", help="skip the rocprofv3 child runs that measure roofline.traffic")
    ap.add_argument("--seq", type=int, default=C5["seq"])
    ap.add_argument("--batch", type=int, default=C5["batch"])
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the path shards by batch; no multi-GPU code here); use --gpus 1")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    if args.only_model:
        print(json.dumps({"whole_models": bench_models(max(args.steps, 5), only=args.only_model)}))
        return
    if args.gemm_replay:
        gemm_replay(dict(C5, seq=args.seq, batch=args.batch), args.gemm_replay)
        return
    if args.power_probe:
        power_probe(dict(C5, seq=args.seq, batch=args.batch))
        return
    from enzyme_ad.jax import enzyme_jax_ir, JaXPipeline, vjp, llama

    if args.calibrate:
        from enzyme_ad.jax import ops as _ops
        ca = torch.ones(1 << 28, dtype=torch.bfloat16, device="cuda")
        cb = torch.ones(1 << 28, dtype=torch.bfloat16, device="cuda")
        _ops.add(ca, cb)
        torch.cuda.synchronize()
        del ca, cb
    cfg = dict(C5, seq=args.seq, batch=args.batch)
    x, lw, dy = make_layer_inputs(cfg)
    nh = cfg["n_heads"]

    @enzyme_jax_ir(pipeline_options=JaXPipeline(), inner_jit=False)
    def layer_fn(x, lw):
        return llama.layer(x, lw, nh)

    def step():
        out, f_vjp = vjp(layer_fn, x, lw)
        return f_vjp(dy)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    tokens = cfg["batch"] * cfg["seq"]
    fl = layer_flops(cfg)
    name = "llama7b_layer_B%d_S%d" % (cfg["batch"], cfg["seq"])
    log("%s\tHIP\trocm\tPrimal+VJP\t%.6f s  (%.1f TFLOP/s over %.2f TFLOP algorithmic)" % (name, dt, fl["total"] / dt / 1e12, fl["total"] / 1e12))

    # the other two programs the reference's harness times next to reverse mode (test/test_utils.py:626-735):
    # the primal alone, and forward mode with a tangent on the input and on every weight
    from enzyme_ad.jax import jvp

    def optional(what, fn):
        """The sections after the headline measurement must not cost the JSON line: a failure is reported in it."""
        try:
            return fn()
        except Exception as e:                                   # noqa: BLE001
            log("bench.py: section '%s' failed: %s: %s" % (what, type(e).__name__, e))
            return {"error": "%s: %s" % (type(e).__name__, str(e)[:300])}

    def programs():
        tx = torch.randn_like(x)
        tlw = {k: torch.randn_like(v) * 0.02 for k, v in lw.items()}
        t_primal = event_time(lambda: layer_fn(x, lw), 5)
        t_forward = event_time(lambda: jvp(layer_fn, (x, lw), (tx, tlw)), 5)
        return {"Primal_ms": round(t_primal * 1e3, 3), "Forward_ms": round(t_forward * 1e3, 3), "BothRev_ms": round(dt * 1e3, 3)}

    modes = None
    if not args.no_kernels:
        modes = optional("programs", programs)
        log("layer programs:", modes)

    t_gemm, gemm_fl, n_gemm, per_layout, vendor = bench_gemms(cfg, max(5, min(args.steps, 20)))
    roofline = dict(bound="mfma", kernel="gemm_bf16_pingpong_kernel (256x256x64 tiles; %d launches per step: Y, dX in the NT form, dW in the TN form, 7 weights)" % n_gemm,
                    achieved=gemm_fl / t_gemm / 1e12, peak=PEAK_BF16_TFLOPS, unit="TFLOP/s",
                    frac=gemm_fl / t_gemm / 1e12 / PEAK_BF16_TFLOPS,
                    traffic=None, traffic_source=None,
                    avg_launch_us=t_gemm / n_gemm * 1e6, flops_per_launch=gemm_fl / n_gemm,
                    per_role={k: dict(tflops=round(v["tflops"], 1), avg_launch_us=round(v["seconds"] / v["launches"] * 1e6, 1))
                                for k, v in per_layout.items()},
                    vendor=vendor)
    log("GEMM: %.1f TFLOP/s (%.1f%% of bf16 MFMA peak); per role %s" % (roofline["achieved"], 100 * roofline["frac"], roofline["per_role"]))
    if not args.no_traffic:
        # the operand buffers of this process stay allocated meanwhile (a few GiB of 288); the child runs alone on the GPU
        torch.cuda.synchronize()
        try:
            traffic, note = measure_gemm_traffic(cfg)
        except Exception as e:                                   # noqa: BLE001
            traffic, note = None, "%s: %s" % (type(e).__name__, str(e)[:200])
        if traffic is None and (args.seq, args.batch) == (C5["seq"], C5["batch"]):
            traffic, note = GEMM_TRAFFIC_BYTES_PER_LAUNCH, ("not measured in this run (%s); figure of "
                                                            "profiles/gemm_bf16_llama7b_layer_hbm_traffic.txt" % note)
        roofline["traffic"], roofline["traffic_source"] = traffic, note
        log("GEMM traffic per launch: %s (%s)" % (traffic, note))
    log("vendor yardstick:", vendor)

    def kernel_table():
        table = bench_kernels(cfg, 5)
        for k, v in table.items():
            log("%-20s %8.1f %s  %5.1f%% of peak  (%.0f us)" % (k, v["achieved"], v["unit"], 100 * v["frac"], v["us"]))
        return {k: dict(bound=v["bound"], achieved=round(v["achieved"], 1), unit=v["unit"], frac=round(v["frac"], 4),
                        **({"timing": v["timing"]} if "timing" in v else {}))
                for k, v in table.items()}

    kernels = optional("kernels", kernel_table) if not args.no_kernels else None

    frontend = None
    if not args.no_kernels and not args.no_frontend:
        frontend = optional("stablehlo_frontend", lambda: bench_frontend(5))
        for k, v in frontend.items():
            log("%-28s %s" % (k, {a: b for a, b in v.items() if a != "clusters"} if isinstance(v, dict) else v))

    models = None
    if not args.no_kernels and not args.no_frontend:
        models = optional("whole_models", lambda: bench_models(5))
        for k, v in models.items():
            log("%-24s %s" % (k, v))

    cpu = None
    if not args.no_cpu_baseline:
        cpu = optional("cpu_baseline", lambda: cpu_baseline(cfg))
        log("cpu baseline:", cpu)

    print(json.dumps({
        "metric": "fwd+VJP tokens/sec per llama layer on 1 GPU",
        "value": tokens / dt, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "Llama-2-7B-shaped decoder layer fwd+VJP: dim 4096, hidden 11008, "
                               "32 heads x 128, batch %d x seq %d, bf16" % (cfg["batch"], cfg["seq"]),
                   "tokens_per_step": tokens, "algorithmic_tflop_per_step": fl["total"] / 1e12,
                   "step_tflops": fl["total"] / dt / 1e12},
        "roofline": roofline, "programs": modes, "kernels": kernels, "stablehlo_frontend": frontend, "whole_models": models, "cpu_baseline": cpu,
    }))


if __name__ == "__main__":
    main()
