"""GPU parity of the dense stages against the CPU oracle: norms, rotation, exact search.

Tolerances follow the reference's own tests: distances within 1e-4 relative, indices equal unless
the two candidate distances are within 1e-4 relative (tests/test_distance_computers.cpp:83-152);
rotation round trip max error < 1e-4 (tests/test_rotation.cpp:56-149).
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _assign_full(capi, ctx, X, C):
    n, d = X.shape
    k = C.shape[0]
    dX, dC = ctx.array(X), ctx.array(C)
    xn, cn = ctx.empty(n), ctx.empty(k)
    idx, dist = ctx.empty(n, np.uint32), ctx.empty(n)
    capi.check(ctx.lib.skm_norms(ctx.handle, dX.ptr, n, d, d, xn.ptr))
    capi.check(ctx.lib.skm_norms(ctx.handle, dC.ptr, k, d, d, cn.ptr))
    capi.check(ctx.lib.skm_assign_full(ctx.handle, dX.ptr, n, dC.ptr, k, d, xn.ptr, cn.ptr, idx.ptr, dist.ptr))
    out = idx.download(), dist.download(), xn.download()
    for a in (dX, dC, xn, cn, idx, dist):
        a.free()
    return out


@pytest.mark.parametrize("rows,d,cols", [(1000, 768, 768), (1000, 768, 96), (333, 50, 50), (64, 1024, 85), (5, 3, 2)])
def test_norms_match_oracle(capi, ctx, oracle, rows, d, cols):
    x = np.random.default_rng(1).standard_normal((rows, d)).astype(np.float32)
    dx, out = ctx.array(x), ctx.empty(rows)
    capi.check(ctx.lib.skm_norms(ctx.handle, dx.ptr, rows, d, cols, out.ptr))
    got = out.download()
    ref = oracle.norms(x, cols)
    exact = (x[:, :cols].astype(np.float64) ** 2).sum(1)
    assert np.allclose(got, ref, rtol=1e-5, atol=0)
    assert np.allclose(got, exact, rtol=1e-5, atol=0)
    dx.free(), out.free()


# shapes of tests/test_distance_computers.cpp:89-95 plus ragged / non-vectorisable ones
@pytest.mark.parametrize("n,k,d", [(100, 50, 32), (1000, 100, 64), (5000, 1000, 128), (500, 2000, 256),
                                   (1000, 257, 50), (777, 3000, 600), (4097, 1025, 130), (1, 1, 1), (3, 1100, 7)])
def test_assign_full_matches_oracle_and_brute_force(capi, ctx, oracle, n, k, d):
    g = np.random.default_rng(n + k + d)
    X = g.standard_normal((n, d)).astype(np.float32)
    C = g.standard_normal((k, d)).astype(np.float32)
    gi, gd, _ = _assign_full(capi, ctx, X, C)
    oi, od = oracle.find_nn(X, C)
    bi, bbest, _ = oracle.brute_force(X, C)
    X64, C64 = X.astype(np.float64), C.astype(np.float64)
    for ref_idx in (oi, bi):
        for i in np.nonzero(gi != ref_idx)[0]:
            da = ((X64[i] - C64[gi[i]]) ** 2).sum()
            db = ((X64[i] - C64[ref_idx[i]]) ** 2).sum()
            assert abs(da - db) <= 1e-4 * max(db, 1e-12), f"point {i}: gpu {gi[i]} ({da}) vs ref {ref_idx[i]} ({db})"
    assert np.allclose(gd, bbest, rtol=1e-4, atol=1e-5)
    assert np.allclose(gd, od, rtol=1e-4, atol=1e-5)


def test_assign_full_clustered_data_exact_agreement(capi, ctx, oracle, blobs):
    """On well separated mixtures there are no near ties: indices must agree exactly (C1-like shape, reduced n)."""
    X = blobs(20000, 768, 1000, std=0.3, seed=5)
    C = X[np.random.default_rng(0).choice(len(X), 1000, replace=False)].copy()
    gi, gd, _ = _assign_full(capi, ctx, X, C)
    oi, od = oracle.find_nn(X, C)
    bi, bbest, bsecond = oracle.brute_force(X, C)
    tie = (bsecond - bbest) <= 1e-5 * np.maximum(bbest, 1e-12)
    assert np.all((gi == bi) | tie)
    assert np.mean(gi != oi) <= 1e-4
    # a point that coincides with a centroid has distance clamped at 0 (batch_computers.h:165)
    assert gd.min() >= 0.0


@pytest.mark.parametrize("n,k,d", [(70001, 1250, 96), (66000, 1500, 70), (70000, 1024, 33),
                                   (70000, 1040, 96), (66000, 1056, 70), (70001, 1029, 33), (140000, 517, 64),
                                   (70000, 1064, 96), (66000, 1120, 70), (70001, 1152, 33)])
def test_assign_full_workgroup_tile_shape_never_changes_a_bit(capi, ctx, oracle, n, k, d):
    """At least 1,024 tiles of 256 x 256 select the large workgroup shape, fewer the 128 x 128 one; a k that is up to
    128 more than a multiple of 256 (1040, 1056, 1029, 517, 1064, 1120, 1152) sends the leftover centroids through
    thin shapes of 32 to 128 rows in a launch of their own.  All accumulate every dot product in the same order, so one call over all points and
    calls over slices of 8,192 points must return identical bits (ragged n and k, rows that are not 16-byte aligned,
    a trailing partial slice of d), and a nearest centroid among the leftover ones must be found like any other."""
    g = np.random.default_rng(n + k + d)
    X = g.standard_normal((n, d)).astype(np.float32)
    C = g.standard_normal((k, d)).astype(np.float32)
    if k % 256 and k % 256 <= 128:
        X[::7] = C[-(np.arange(len(X[::7])) % (k % 256)) - 1] + 0.3 * X[::7]  # every 7th point sits near a leftover centroid
    gi, gd, _ = _assign_full(capi, ctx, X, C)
    if k % 256 and k % 256 <= 128:
        assert np.mean(gi[::7] >= k - k % 256) > 0.99
    for i0 in range(0, n, 8192):
        si, sd, _ = _assign_full(capi, ctx, X[i0:i0 + 8192], C)
        assert np.array_equal(gi[i0:i0 + 8192], si) and np.array_equal(gd[i0:i0 + 8192], sd)
    m = 4000  # and the oracle on the last points (the ragged last tile)
    bi, bbest, bsecond = oracle.brute_force(X[-m:], C)
    tie = (bsecond - bbest) <= 1e-4 * np.maximum(bbest, 1e-12)
    assert np.all((gi[-m:] == bi) | tie)
    assert np.allclose(gd[-m:], bbest, rtol=1e-4, atol=1e-5)


def test_assign_full_half_width_tiles_never_change_a_bit(capi, ctx, oracle):
    """39,000 points x 256 centroids are 610 tiles of 128 x 128 on 512 workgroup slots: the search then uses tiles of
    128 x 64; slices of 19,500 points (314 tiles) use whole tiles.  Same accumulation order, same bits."""
    g = np.random.default_rng(39)
    n, k, d = 39000, 256, 70
    X = g.standard_normal((n, d)).astype(np.float32)
    C = g.standard_normal((k, d)).astype(np.float32)
    gi, gd, _ = _assign_full(capi, ctx, X, C)
    for i0 in (0, 19500):
        si, sd, _ = _assign_full(capi, ctx, X[i0:i0 + 19500], C)
        assert np.array_equal(gi[i0:i0 + 19500], si) and np.array_equal(gd[i0:i0 + 19500], sd)
    bi, bbest, bsecond = oracle.brute_force(X[-3000:], C)
    tie = (bsecond - bbest) <= 1e-4 * np.maximum(bbest, 1e-12)
    assert np.all((gi[-3000:] == bi) | tie)


def test_rotate_large_tile_shape_equals_small_tile_shape(capi, ctx, oracle):
    n, d = 270000, 256  # 1,055 tiles of 256 x 256
    Q = oracle.rotation_matrix(d, seed=7)
    X = np.random.default_rng(4).standard_normal((n, d)).astype(np.float32)
    dX, dQ, dR = ctx.array(X), ctx.array(Q), ctx.empty((n, d))
    capi.check(ctx.lib.skm_rotate(ctx.handle, dX.ptr, n, d, dQ.ptr, dR.ptr))
    R = dR.download()
    m = 5000
    dS = ctx.empty((m, d))
    capi.check(ctx.lib.skm_rotate(ctx.handle, dX.ptr + (n - m) * d * 4, m, d, dQ.ptr, dS.ptr))
    assert np.array_equal(R[-m:], dS.download())
    assert np.abs(R[:m] - X[:m].astype(np.float64) @ Q.astype(np.float64).T).max() < 1e-5
    for a in (dX, dQ, dR, dS):
        a.free()


def test_assign_full_duplicate_centroids_take_lowest_index(capi, ctx):
    """Exact ties resolve to the lowest index inside a batch (minCoeff) and across batches (strict <)."""
    g = np.random.default_rng(3)
    base = g.standard_normal((8, 64)).astype(np.float32)
    C = np.tile(base, (300, 1))  # 2400 centroids: every centroid repeats every 8 rows, across 3 batches
    X = base + 0.01 * g.standard_normal((8, 64)).astype(np.float32)
    gi, _, _ = _assign_full(capi, ctx, X, C)
    assert np.array_equal(gi, np.arange(8, dtype=np.uint32))


def test_assign_full_chunked_by_workspace_limit(capi, ctx, oracle):
    """A tiny workspace forces several chunks of points; results must not change."""
    g = np.random.default_rng(9)
    X = g.standard_normal((3000, 96)).astype(np.float32)
    C = g.standard_normal((700, 96)).astype(np.float32)
    ref = _assign_full(capi, ctx, X, C)
    capi.check(ctx.lib.skm_ctx_set_workspace_limit(ctx.handle, 64 << 20))
    try:
        # 64 MiB / (11 granules * 8 B) is still > 3000 points, so shrink k-granule budget via a large k instead
        C2 = np.concatenate([C, g.standard_normal((40000, 96)).astype(np.float32) + 50.0])
        got = _assign_full(capi, ctx, np.tile(X, (5, 1)), C2)
    finally:
        capi.check(ctx.lib.skm_ctx_set_workspace_limit(ctx.handle, 24 << 30))
    assert np.array_equal(got[0][:3000], ref[0])
    assert np.array_equal(got[0][3000:6000], ref[0])


@pytest.mark.parametrize("d", [50, 128, 256, 512, 768, 1024])
def test_rotate_unrotate_match_oracle_and_round_trip(capi, ctx, oracle, d):
    n = 300
    Q = oracle.rotation_matrix(d, seed=42)
    X = np.random.default_rng(d).standard_normal((n, d)).astype(np.float32)
    dX, dQ, dQt, dR, dB = ctx.array(X), ctx.array(Q), ctx.empty((d, d)), ctx.empty((n, d)), ctx.empty((n, d))
    capi.check(ctx.lib.skm_transpose(ctx.handle, dQ.ptr, d, d, dQt.ptr))
    assert np.array_equal(dQt.download(), Q.T)
    capi.check(ctx.lib.skm_rotate(ctx.handle, dX.ptr, n, d, dQ.ptr, dR.ptr))
    capi.check(ctx.lib.skm_unrotate(ctx.handle, dR.ptr, n, d, dQt.ptr, dB.ptr))
    R, B = dR.download(), dB.download()
    exact = X.astype(np.float64) @ Q.astype(np.float64).T
    assert np.abs(R - exact).max() < 1e-5
    assert np.abs(R - oracle.rotate(Q, X)).max() < 1e-5
    assert np.abs(B - X).max() < 1e-4 and np.abs(B - X).mean() < 1e-5  # test_rotation.cpp:56-149
    # norm preservation, rel < 1e-5 (test_rotation.cpp:157-206)
    nx, nr = np.linalg.norm(X.astype(np.float64), axis=1), np.linalg.norm(R.astype(np.float64), axis=1)
    assert np.max(np.abs(nx - nr) / nx) < 1e-5
    for a in (dX, dQ, dQt, dR, dB):
        a.free()


def test_transpose_rectangular(capi, ctx):
    a = np.arange(37 * 101, dtype=np.float32).reshape(37, 101)
    da, dt = ctx.array(a), ctx.empty((101, 37))
    capi.check(ctx.lib.skm_transpose(ctx.handle, da.ptr, 37, 101, dt.ptr))
    assert np.array_equal(dt.download(), a.T)
    da.free(), dt.free()


def test_bad_arguments_are_rejected(capi, ctx):
    x = ctx.empty((4, 8))
    with pytest.raises(capi.SkmError):
        capi.check(ctx.lib.skm_norms(ctx.handle, x.ptr, 4, 8, 9, x.ptr))  # cols > d
    with pytest.raises(capi.SkmError):
        capi.check(ctx.lib.skm_assign_full(ctx.handle, x.ptr, 4, None, 2, 8, x.ptr, x.ptr, x.ptr, x.ptr))
    with pytest.raises(capi.SkmError):
        capi.check(ctx.lib.skm_rotate(ctx.handle, x.ptr, 4, 8, x.ptr, x.ptr))  # in place
    x.free()


def test_upload_on_the_transfer_stream_orders_before_later_work(capi, ctx):
    """skm_upload_overlapped copies on the context's second stream; what is queued afterwards must see the data, what
    was queued before keeps running.  Slabs are uploaded one after the other, each followed by the norms of its rows."""
    g = np.random.default_rng(5)
    n, d, slab = 60000, 512, 7000
    X = g.standard_normal((n, d)).astype(np.float32)
    dX, out = ctx.empty((n, d)), ctx.empty(n)
    for r0 in range(0, n, slab):
        m = min(slab, n - r0)
        rows = np.ascontiguousarray(X[r0:r0 + m])
        capi.check(ctx.lib.skm_upload_overlapped(ctx.handle, dX.ptr + r0 * d * 4, rows.ctypes.data, m * d * 4))
        capi.check(ctx.lib.skm_norms(ctx.handle, dX.ptr + r0 * d * 4, m, d, d, out.ptr + r0 * 4))
    ctx.sync()
    assert np.array_equal(dX.download(), X)
    assert np.allclose(out.download(), (X.astype(np.float64) ** 2).sum(1), rtol=1e-5)
    dX.free(), out.free()


def test_detached_upload_from_a_second_thread(capi, ctx):
    """skm_upload_detached returns when the bytes are in device memory and leaves the context's stream alone: a second
    thread feeds the slabs while this one queues the norms of every slab that has arrived."""
    import threading

    g = np.random.default_rng(8)
    n, d, slab = 50000, 512, 6000
    X = g.standard_normal((n, d)).astype(np.float32)
    dX, out = ctx.empty((n, d)), ctx.empty(n)
    starts = list(range(0, n, slab))
    arrived = [threading.Event() for _ in starts]
    failed = []

    def feed():
        try:
            for s, r0 in enumerate(starts):
                m = min(slab, n - r0)
                capi.check(ctx.lib.skm_upload_detached(ctx.handle, dX.ptr + r0 * d * 4, X[r0:r0 + m].ctypes.data, m * d * 4))
                arrived[s].set()
        except Exception as e:  # reported below, in the thread that runs the test
            failed.append(e)
            for a in arrived:
                a.set()

    t = threading.Thread(target=feed)
    t.start()
    for s, r0 in enumerate(starts):
        assert arrived[s].wait(60)
        assert not failed, failed
        m = min(slab, n - r0)
        capi.check(ctx.lib.skm_norms(ctx.handle, dX.ptr + r0 * d * 4, m, d, d, out.ptr + r0 * 4))
    t.join()
    ctx.sync()
    assert np.array_equal(dX.download(), X)
    assert np.allclose(out.download(), (X.astype(np.float64) ** 2).sum(1), rtol=1e-5)
    capi.check(ctx.lib.skm_upload_detached(ctx.handle, dX.ptr, X.ctypes.data, 0))
    with pytest.raises(capi.SkmError):
        capi.check(ctx.lib.skm_upload_detached(ctx.handle, None, X.ctypes.data, 16))
    dX.free(), out.free()


def test_large_download_through_the_lanes_is_byte_exact(capi, ctx):
    """From 64 MiB a download goes through four threads, each moving every fourth 4 MiB chunk through its own pinned
    block; the copy waits for the work queued before it.  Sizes with a ragged last chunk and with fewer chunks than
    lanes' turns; the small path beside it.  Twice, so the second call reuses the lanes."""
    g = np.random.default_rng(6)
    for count in (16 * 1024 * 1024 + 12345, 16 * 1024 * 1024, 20_000_003, 1_000_001):
        host = g.integers(0, 2 ** 32, count, dtype=np.uint32)
        dev = ctx.array(host)
        capi.check(ctx.lib.skm_fill_u32(ctx.handle, dev.ptr, 0xdeadbeef, 1000))  # queued work the copy must wait for
        got = dev.download()
        assert np.array_equal(got[:1000], np.full(1000, 0xdeadbeef, dtype=np.uint32))
        assert np.array_equal(got[1000:], host[1000:])
        dev.free()
