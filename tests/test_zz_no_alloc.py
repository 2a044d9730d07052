"""The allocation-free RMSNorm adjoint entry point against the workspace one, through the C ABI: two calls in a row on
the same device, the second with a smaller input (the built-in scratch array keeps the first call's contents), plus
the size limit."""
import gc

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _run_pair(lib, N, rows, dim, dt, code, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn((rows, dim), device="cuda", generator=g).to(dt)
    dy = torch.randn((rows, dim), device="cuda", generator=g).to(dt)
    add = torch.randn((rows, dim), device="cuda", generator=g).to(dt)
    gamma = (torch.rand(dim, device="cuda", generator=g) + 0.5).to(dt)
    st = torch.cuda.current_stream().cuda_stream
    p = lambda t: t.data_ptr()
    nbytes = lib.emi_rmsnorm_bwd_workspace_bytes(rows, dim)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    dx_ref, dg_ref = torch.empty_like(x), torch.empty_like(gamma)
    N.check(lib.emi_rmsnorm_bwd(st, p(x), p(gamma), p(dy), p(add), p(dx_ref), p(dg_ref), p(ws), nbytes, rows, dim, 1e-5, code))
    dx, dg = torch.full_like(x, float("nan")), torch.full_like(gamma, float("nan"))
    torch.cuda.synchronize()
    gc.collect()                  # tensors that earlier tests left in reference cycles must not be freed inside the window
    gc.disable()
    try:
        before = torch.cuda.memory_allocated()
        N.check(lib.emi_rmsnorm_bwd_noalloc(st, p(x), p(gamma), p(dy), p(add), p(dx), p(dg), rows, dim, 1e-5, code))
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
    finally:
        gc.enable()
    assert torch.equal(dx, dx_ref), "dx differs (rows %d, dim %d)" % (rows, dim)
    assert torch.equal(dg, dg_ref), "dgamma differs (rows %d, dim %d)" % (rows, dim)


@pytest.mark.parametrize("dt,code", [(torch.bfloat16, 16), (torch.float32, 11)])
def test_noalloc_matches_workspace_entry_point_twice(dt, code):
    from enzyme_ad.jax import _native as N
    lib = N.lib()
    _run_pair(lib, N, 4096, 4096, dt, code, 1)       # large first: fills many partial rows of the scratch array
    _run_pair(lib, N, 37, 288, dt, code, 2)          # then a smaller, ragged one over the stale contents
    _run_pair(lib, N, 5, 1000, dt, code, 3)          # dim not a multiple of 8: the generic kernel


def test_noalloc_rejects_sizes_beyond_the_array():
    from enzyme_ad.jax import _native as N
    lib = N.lib()
    rows, dim = 2048, 16384                          # 1024 partial rows of 16384 floats > 16 MiB
    x = torch.zeros((rows, dim), device="cuda", dtype=torch.bfloat16)
    g = torch.ones(dim, device="cuda", dtype=torch.bfloat16)
    p = lambda t: t.data_ptr()
    rc = lib.emi_rmsnorm_bwd_noalloc(torch.cuda.current_stream().cuda_stream, p(x), p(g), p(x), None, p(x), p(g), rows, dim, 1e-5, 16)
    assert rc == 3 and b"scratch" in lib.emi_last_error()
