"""The entry point that allocates nothing, through the C ABI, against the allocating one.

`ft_rms_norm_backward_noalloc` keeps its per-workgroup partial rows in a fixed device array
instead of a pooled buffer. Both entry points launch the same kernels with the same grid, so gx and
gw must agree to the bit; both are also held to the oracle at the f32 bar. Two calls in a row,
the second smaller: the array still holds the first call's partial rows, which must not leak in.
"""
import numpy as np
import pytest

from oracle import cpu
from tests.gpu_util import assert_close, make_ctx

pytestmark = pytest.mark.gpu


def rnd(seed, *shape):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def _run(ctx, eng, rows, size, seed):
    from ferrotensor_amd import UnifiedTensor
    up = lambda a: UnifiedTensor.new(ctx, a, list(a.shape))
    x, w, gy = rnd(seed, rows, size), rnd(seed + 1, size), rnd(seed + 2, rows, size)
    eps = 1e-5
    tx, tw, tg = up(x), up(w), up(gy)
    gx_a, gw_a = UnifiedTensor.empty(ctx, [rows, size]), UnifiedTensor.empty(ctx, [size])
    eng.rms_norm_backward(ctx, tx, tw, tg, gx_a, gw_a, eps)
    live, idle = ctx.pool_stats()
    gx_n, gw_n = UnifiedTensor.empty(ctx, [rows, size]), UnifiedTensor.empty(ctx, [size])
    before = ctx.pool_stats()
    eng.rms_norm_backward_noalloc(ctx, tx, tw, tg, gx_n, gw_n, eps)
    assert ctx.pool_stats() == before          # nothing taken from, or returned to, the pool
    np.testing.assert_array_equal(gx_n.to_numpy(), gx_a.to_numpy())
    np.testing.assert_array_equal(gw_n.to_numpy(), gw_a.to_numpy())
    want_gx, want_gw = cpu.rms_norm_backward(x, w, gy, eps)
    assert_close("gx", gx_n.to_numpy(), want_gx)
    assert_close("gw", gw_n.to_numpy(), want_gw, atol=2e-4)


def test_no_alloc_rms_norm_backward_matches_the_allocating_entry_point():
    ctx, eng = make_ctx()
    try:
        _run(ctx, eng, 2048, 960, 1)       # 256 partial rows of 960
        _run(ctx, eng, 37, 96, 5)          # smaller: 10 partial rows of 96 over the first call's leftovers
        _run(ctx, eng, 4100, 2048, 9)      # the largest row the array holds
        _run(ctx, eng, 1, 4, 13)
    finally:
        ctx.close()


def test_no_alloc_rejects_what_does_not_fit():
    from ferrotensor_amd import FtError, UnifiedTensor
    ctx, eng = make_ctx()
    try:
        def call(rows, size, gw=True):
            x = UnifiedTensor.zeros(ctx, [rows, size])
            w = UnifiedTensor.zeros(ctx, [size])
            gx = UnifiedTensor.empty(ctx, [rows, size])
            gwt = UnifiedTensor.empty(ctx, [size])
            eng.rms_norm_backward_noalloc(ctx, x, w, x, gx, gwt, 1e-5)
        with pytest.raises(FtError, match="at most 2048"):
            call(3, 2052)
        with pytest.raises(FtError, match="multiple of 4"):
            call(3, 30)
        call(3, 2048)
    finally:
        ctx.close()
