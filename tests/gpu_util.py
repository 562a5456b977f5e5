"""Helpers shared by the GPU parity tests."""
from __future__ import annotations

import numpy as np

from granite_amd import DeviceBuffer

ABS_TOL = 2e-3    # attention outputs: |d| <= 2e-3 or |d| <= 1e-2 |ref|
REL_TOL = 1e-2
LSE_TOL = 1e-4    # log-sum-exp, absolute


def dev(arr: np.ndarray) -> DeviceBuffer:
    return DeviceBuffer.from_numpy(arr)


def say(msg: str) -> None:
    print(msg, flush=True)


def assert_close(got, want, what, abs_tol=ABS_TOL, rel_tol=REL_TOL):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    d = np.abs(got - want)
    ok = (d <= abs_tol) | (d <= rel_tol * np.abs(want))
    if not ok.all():
        idx = np.unravel_index(np.argmax(np.where(ok, 0, d)), d.shape)
        raise AssertionError(f"{what}: {int((~ok).sum())} of {ok.size} elements off; worst at {idx}: "
                             f"got {got[idx]:.6f} want {want[idx]:.6f}")
    return float(d.max(initial=0.0))


def assert_lse(got, want, what, tol=LSE_TOL):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    d = np.abs(got - want)
    assert np.isfinite(got).all() and d.max(initial=0.0) <= tol, \
        f"{what}: lse max abs diff {d.max(initial=0.0):.3e} > {tol}"
    return float(d.max(initial=0.0))
