"""skm_assign_full_noalloc (the entry point that allocates nothing) against skm_assign_full.

Both run the same kernels; the variant keeps its per-(granule, point) minima in the library's static device
array instead of the context's workspace.  Bar: indices and distances bit-identical.  Two calls in a row, the
second on a smaller input (the array keeps the first call's contents), then a shape whose points do not fit
the array at once (chunked), and the rejection of a k beyond the stated maximum.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _both(capi, ctx, X, C):
    n, d = X.shape
    k = C.shape[0]
    dX, dC = ctx.array(X), ctx.array(C)
    xn, cn = ctx.empty(n), ctx.empty(k)
    capi.check(ctx.lib.skm_norms(ctx.handle, dX.ptr, n, d, d, xn.ptr))
    capi.check(ctx.lib.skm_norms(ctx.handle, dC.ptr, k, d, d, cn.ptr))
    out = []
    for fn in (ctx.lib.skm_assign_full, ctx.lib.skm_assign_full_noalloc):
        idx, dist = ctx.empty(n, np.uint32), ctx.empty(n)
        capi.check(ctx.lib.skm_fill_u32(ctx.handle, idx.ptr, 0xFFFFFFFF, n))
        capi.check(ctx.lib.skm_fill_u32(ctx.handle, dist.ptr, 0xFFFFFFFF, n))
        capi.check(fn(ctx.handle, dX.ptr, n, dC.ptr, k, d, xn.ptr, cn.ptr, idx.ptr, dist.ptr))
        out.append((idx.download(), dist.download()))
        idx.free(), dist.free()
    for a in (dX, dC, xn, cn):
        a.free()
    return out


def test_two_calls_in_a_row_the_second_smaller(capi, ctx, oracle):
    g = np.random.default_rng(7)
    for n, k, d in [(5000, 1500, 128), (777, 300, 96)]:
        X = g.standard_normal((n, d)).astype(np.float32)
        C = g.standard_normal((k, d)).astype(np.float32)
        (ri, rd), (gi, gd) = _both(capi, ctx, X, C)
        assert np.array_equal(gi, ri), f"indices differ at n={n}, k={k}, d={d}"
        assert np.array_equal(gd.view(np.uint32), rd.view(np.uint32)), f"distances differ at n={n}, k={k}, d={d}"
        bi, best, second = oracle.brute_force(X, C)
        tie = (second - best) <= 1e-4 * np.maximum(best, 1e-12)
        assert np.all((gi == bi) | tie)


def test_points_beyond_one_chunk_of_the_static_array(capi, ctx):
    """k = 20,000 leaves room for 13,312 points per chunk; 30,000 points take three chunks."""
    g = np.random.default_rng(8)
    n, k, d = 30000, 20000, 32
    X = g.standard_normal((n, d)).astype(np.float32)
    C = g.standard_normal((k, d)).astype(np.float32)
    (ri, rd), (gi, gd) = _both(capi, ctx, X, C)
    assert np.array_equal(gi, ri)
    assert np.array_equal(gd.view(np.uint32), rd.view(np.uint32))


def test_sizes_beyond_the_maximum_are_rejected(capi, ctx):
    a = ctx.empty(64)
    rc = ctx.lib.skm_assign_full_noalloc(ctx.handle, a.ptr, 4, a.ptr, 2097153, 4, a.ptr, a.ptr, a.ptr, a.ptr)
    assert rc == capi.SKM_ERR_INVALID
    assert b"2097152" in ctx.lib.skm_last_error()
    a.free()
