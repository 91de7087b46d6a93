"""Shared helpers of the GPU parity tests: context, uploads, tolerance rule."""
import numpy as np
import pytest

ATOL = 1e-4   # north-star parity bar: |a - e| <= 1e-4 + 1e-3 * |e|
RTOL = 1e-3


def gpu_available():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def make_ctx():
    from ferrotensor_amd import ComputeEngine, HipContext
    ctx = HipContext(0)
    return ctx, ComputeEngine(ctx)


def assert_close(name, got, want, atol=ATOL, rtol=RTOL):
    got = np.asarray(got, np.float64).reshape(-1)
    want = np.asarray(want, np.float64).reshape(-1)
    assert got.shape == want.shape, (name, got.shape, want.shape)
    err = np.abs(got - want)
    assert np.all(np.isfinite(got)), "%s: non-finite output" % name
    ratio = err / (atol + rtol * np.abs(want))
    worst = int(np.argmax(ratio)) if ratio.size else 0
    assert ratio.size == 0 or ratio[worst] <= 1.0, \
        "%s: element %d got %r want %r (|err| %.3e, allowed %.3e)" % (
            name, worst, got[worst], want[worst], err[worst], atol + rtol * abs(want[worst]))
