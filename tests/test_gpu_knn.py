"""GPU parity of the k-nearest-neighbour search and the recall count behind training with queries.

Bars follow tests/test_distance_computers.cpp:201-262 of the reference: distances within 1e-4
relative, indices equal unless the two distances tie to 1e-4 relative, rows sorted.  The hand-built
cases are bit-exact (all arithmetic is exact in fp32).
"""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

FLT_MAX = np.finfo(np.float32).max


def _knn(capi, ctx, x, y, k, xnorm=None, ynorm=None, workspace_limit=None):
    nx, d = x.shape
    ny = y.shape[0]
    dx, dy = ctx.array(x), ctx.array(y)
    xn, yn = ctx.empty(max(nx, 1)), ctx.empty(max(ny, 1))
    if xnorm is None:
        capi.check(ctx.lib.skm_norms(ctx.handle, dx.ptr, nx, d, d, xn.ptr))
    else:
        xn.upload(np.ascontiguousarray(xnorm, dtype=np.float32))
    if ynorm is None:
        capi.check(ctx.lib.skm_norms(ctx.handle, dy.ptr, ny, d, d, yn.ptr))
    else:
        yn.upload(np.ascontiguousarray(ynorm, dtype=np.float32))
    idx, dist = ctx.empty((nx, k), np.uint32), ctx.empty((nx, k))
    if workspace_limit is not None:
        capi.check(ctx.lib.skm_ctx_set_workspace_limit(ctx.handle, workspace_limit))
    try:
        capi.check(ctx.lib.skm_knn(ctx.handle, dx.ptr, nx, dy.ptr, ny, d, xn.ptr, yn.ptr, k, idx.ptr, dist.ptr))
    finally:
        if workspace_limit is not None:
            capi.check(ctx.lib.skm_ctx_set_workspace_limit(ctx.handle, 24 << 30))
    out = idx.download(), dist.download()
    for a in (dx, dy, xn, yn, idx, dist):
        a.free()
    return out


@pytest.mark.parametrize("n_x,n_y,d,k,limit", [
    (1000, 500, 128, 10, None),      # the reference's own test shape
    (64, 3000, 96, 100, None),       # three batches of 1024, k = objective_k default
    (257, 5000, 130, 33, None),      # ragged, non-vectorisable row stride
    (1100, 20000, 32, 100, 64 << 20),  # smallest workspace: two chunks of whole batches
    (50, 4097, 32, 1024, None),      # largest k
    (7, 5, 16, 10, None),            # fewer rows than k: unfilled slots
])
def test_knn_matches_oracle_and_fp64_brute_force(capi, ctx, oracle, n_x, n_y, d, k, limit):
    rng = np.random.default_rng(n_x + n_y + d + k)
    x = rng.uniform(-10, 10, (n_x, d)).astype(np.float32)
    y = rng.uniform(-10, 10, (n_y, d)).astype(np.float32)
    gi, gd = _knn(capi, ctx, x, y, k, workspace_limit=limit)
    oi, od = oracle.find_knn(x, y, k)
    kk = min(k, n_y)
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    d64 = (x64 ** 2).sum(1)[:, None] + (y64 ** 2).sum(1)[None, :] - 2.0 * (x64 @ y64.T)
    order = np.argsort(d64, axis=1, kind="stable")[:, :kk]
    ref_d = np.take_along_axis(d64, order, axis=1)
    rel = np.abs(gd[:, :kk] - ref_d) / np.maximum(ref_d, 1e-6)
    assert rel.max() <= 1e-4
    assert np.all((gi[:, :kk] == order) | (rel <= 1e-4))
    assert np.all(np.diff(gd[:, :kk], axis=1) >= 0)
    # against the oracle: same sets, same order except where two fp32 distances differ in the last bits
    assert np.mean(gi == oi) > 0.999
    assert np.allclose(gd[:, :kk], od[:, :kk], rtol=1e-4, atol=1e-5)
    for q in range(n_x):
        assert len(set(gi[q, :kk].tolist())) == kk  # no duplicates
    if kk < k:
        assert np.all(gi[:, kk:] == 0xFFFFFFFF) and np.all(gd[:, kk:] == FLT_MAX)


def test_knn_batches_ties_and_progressive_clamp_bit_exact(capi, ctx, oracle):
    y = np.full((1030, 1), 100.0, dtype=np.float32)
    y[5, 0], y[900, 0], y[1025, 0], y[1027, 0] = 3.0, -3.0, 3.0, 1.0
    x = np.zeros((1, 1), dtype=np.float32)
    gi, gd = _knn(capi, ctx, x, y, 3)
    assert gi[0].tolist() == [1027, 5, 900] and gd[0].tolist() == [1.0, 9.0, 9.0]
    x = np.ones((1, 1), dtype=np.float32)
    y[1027, 0] = 2.0
    ynorm = (y[:, 0] ** 2).astype(np.float32)
    ynorm[5], ynorm[1025] = 3.0, 4.0  # raw distances -2 (batch 0) and -1 (batch 1)
    gi, gd = _knn(capi, ctx, x, y, 3, xnorm=np.ones(1, np.float32), ynorm=ynorm)
    oi, od = oracle.find_knn(x, y, 3, norms_x=np.ones(1, np.float32), norms_y=ynorm)
    assert gi[0].tolist() == [1025, 5, 1027] and gd[0].tolist() == [0.0, 0.0, 1.0]
    assert np.array_equal(gi, oi) and np.array_equal(gd, od)
    # a clamped pair left out of order by the last batch stays as the reference leaves it
    ynorm[1028] = 3.5   # with y = 3: -6 + 1 + 3.5 = -1.5, a second negative residue in the last batch
    y[1028, 0] = 3.0
    gi, gd = _knn(capi, ctx, x, y, 3, xnorm=np.ones(1, np.float32), ynorm=ynorm)
    oi, od = oracle.find_knn(x, y, 3, norms_x=np.ones(1, np.float32), norms_y=ynorm)
    assert np.array_equal(gi, oi) and np.array_equal(gd, od)
    assert gi[0].tolist() == [1028, 1025, 5] and gd[0].tolist() == [0.0, 0.0, 0.0]


def test_knn_integer_grid_is_bit_exact_with_oracle(capi, ctx, oracle):
    # Small integers: every product and sum is exact in fp32 whatever the summation order, so the device and
    # the oracle must agree bit for bit, including the many exact ties (broken by index).
    rng = np.random.default_rng(5)
    x = rng.integers(-3, 4, (200, 24)).astype(np.float32)
    y = rng.integers(-3, 4, (5000, 24)).astype(np.float32)
    gi, gd = _knn(capi, ctx, x, y, 50)
    oi, od = oracle.find_knn(x, y, 50)
    assert np.array_equal(gi, oi) and np.array_equal(gd, od)


def test_knn_argument_errors(capi, ctx):
    one = ctx.empty(16)
    rc = ctx.lib.skm_knn(ctx.handle, one.ptr, 1, one.ptr, 1, 1, one.ptr, one.ptr, 0, one.ptr, one.ptr)
    assert rc == capi.SKM_ERR_INVALID
    rc = ctx.lib.skm_knn(ctx.handle, one.ptr, 1, one.ptr, 1, 1, one.ptr, one.ptr, 1025, one.ptr, one.ptr)
    assert rc == capi.SKM_ERR_INVALID and b"1024" in ctx.lib.skm_last_error()
    one.free()


@pytest.mark.parametrize("nq,ok,explore,n_assign,k", [(2, 4, 2, 6, 8), (300, 100, 100, 50000, 10000), (17, 10, 1, 400, 7)])
def test_recall_hits_match_oracle(capi, ctx, oracle, nq, ok, explore, n_assign, k):
    rng = np.random.default_rng(nq + ok)
    if nq == 2:
        assign = np.array([0, 1, 2, 2, 3, 1], dtype=np.uint32)
        gt = np.array([[0, 1, 2, 3], [4, 5, 0, 1]], dtype=np.uint32)
        promising = np.array([[2, 7], [1, 3]], dtype=np.uint32)
    else:
        assign = rng.integers(0, k, n_assign).astype(np.uint32)
        gt = rng.integers(0, n_assign, (nq, ok)).astype(np.uint32)
        promising = np.stack([rng.permutation(k)[:explore] for _ in range(nq)]).astype(np.uint32)
    dgt, dpr, das = ctx.array(gt), ctx.array(promising), ctx.array(assign)
    hits = np.zeros(nq, dtype=np.uint32)
    capi.check(ctx.lib.skm_recall_hits(ctx.handle, dgt.ptr, dpr.ptr, das.ptr, assign.size, nq, ok, explore,
                                       hits.ctypes.data_as(ctypes.c_void_p)))
    expect = np.array([sum(assign[g] in set(promising[q].tolist()) for g in gt[q]) for q in range(nq)], dtype=np.uint32)
    assert np.array_equal(hits, expect)
    total = np.float32(0.0)
    for h in hits:
        total = np.float32(total + np.float32(h) / np.float32(ok))
    assert np.float32(total / np.float32(nq)) == np.float32(oracle.recall_from_lists(gt, promising, assign))
    if nq == 2:
        assert hits.tolist() == [2, 3]
    for a in (dgt, dpr, das):
        a.free()
