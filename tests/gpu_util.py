"""Helpers for the GPU parity tests: move seeded numpy inputs to the device in
the storage dtype under test, and hand the oracle the same (rounded) values."""
import numpy as np
import torch

TOL = {"f32": 1e-4, "bf16": 2e-2}      # max relative error allowed by the parity contract
TDTYPE = {"f32": torch.float32, "bf16": torch.bfloat16}


def dev(a, dt):
    """numpy -> device tensor in dtype `dt`; returns (tensor, float64 numpy of the stored values)."""
    t = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(TDTYPE[dt]).cuda()
    return t, t.float().cpu().numpy().astype(np.float64)


def host(t):
    return t.float().cpu().numpy().astype(np.float64)


def rel_err(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    den = float(np.max(np.abs(ref))) or 1.0
    return float(np.max(np.abs(got - ref))) / den


def check(got, ref, dt, what, factor=1.0):
    e = rel_err(host(got) if isinstance(got, torch.Tensor) else got, ref)
    assert np.all(np.isfinite(host(got) if isinstance(got, torch.Tensor) else got)), what + ": non-finite values"
    assert e <= TOL[dt] * factor, "%s: max rel err %.3e > %.1e" % (what, e, TOL[dt] * factor)
    return e


def check_rows(got, ref, dt, what, factor=1.0, floor=1e-3):
    """Row-wise companion of `check`: every row's error is bounded relative to that row's own largest reference
    entry (rows much smaller than the tensor's maximum are invisible to the max-norm metric).  `floor` (relative to
    the tensor's maximum) keeps rows that are zero up to cancellation from demanding more than the arithmetic has."""
    got = host(got) if isinstance(got, torch.Tensor) else np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    got, ref = got.reshape(-1, got.shape[-1]), ref.reshape(-1, ref.shape[-1])
    den = np.maximum(np.max(np.abs(ref), axis=1), floor * float(np.max(np.abs(ref))) or 1.0)
    e = np.max(np.abs(got - ref), axis=1) / den
    worst = int(np.argmax(e))
    assert e[worst] <= TOL[dt] * factor, "%s: row %d rel err %.3e > %.1e" % (what, worst, e[worst], TOL[dt] * factor)
    return float(e[worst])
