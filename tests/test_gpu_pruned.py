"""GPU parity of the pruned search (partial GEMM + ADSampling/PDX pruning) against the CPU oracle.

Bars (north_star): indices equal except where the top-2 gap is below 1e-5 relative, at most 0.01 %
of points; pruning never discards a candidate the oracle keeps (checked through: every GPU/oracle
disagreement must coincide with GPU == exact brute force, or be a tie)."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _pruned(capi, ctx, oracle, X, C, prev, partial_d, ratios, accounting=False, kernel=0, walk=0, launches=1):
    """kernel: skm_ctx_set_candidate_kernel (0 automatic, 1 tiled, 2 register-stationary where the shape allows);
    walk: skm_ctx_set_walk_kernel (0 automatic, 1 one point per wavefront, 2 / 3 four / eight points pooled per wavefront)."""
    n, d = X.shape
    k = C.shape[0]
    H, V = oracle.dimension_split(d)
    dX, dC = ctx.array(X), ctx.array(C)
    dP, dA = ctx.empty(k * d), ctx.empty((k, V))
    capi.check(ctx.lib.skm_pdxify(ctx.handle, dC.ptr, k, d, V, dP.ptr, dA.ptr))
    xn, cn = ctx.empty(n), ctx.empty(k)
    capi.check(ctx.lib.skm_norms(ctx.handle, dX.ptr, n, d, partial_d, xn.ptr))
    capi.check(ctx.lib.skm_norms(ctx.handle, dC.ptr, k, d, partial_d, cn.ptr))
    dR = ctx.array(np.ascontiguousarray(ratios, dtype=np.float32))
    idx, dist = ctx.array(np.ascontiguousarray(prev, dtype=np.uint32)), ctx.empty(n)
    total = ctypes.c_uint64()
    stages = (ctypes.c_uint64 * (H // 64 + 2))()
    capi.check(ctx.lib.skm_ctx_set_candidate_kernel(ctx.handle, kernel))
    capi.check(ctx.lib.skm_ctx_set_walk_kernel(ctx.handle, walk))
    capi.check(ctx.lib.skm_ctx_set_walk_launches(ctx.handle, launches))
    try:
        capi.check(ctx.lib.skm_assign_pruned(ctx.handle, dX.ptr, n, dC.ptr, dP.ptr, dA.ptr, k, d, V, partial_d, dR.ptr,
                                             xn.ptr, cn.ptr, idx.ptr, dist.ptr, ctypes.byref(total),
                                             stages if accounting else None))
    finally:
        capi.check(ctx.lib.skm_ctx_set_candidate_kernel(ctx.handle, 0))
        capi.check(ctx.lib.skm_ctx_set_walk_kernel(ctx.handle, 0))
        capi.check(ctx.lib.skm_ctx_set_walk_launches(ctx.handle, 1))
    out = idx.download(), dist.download(), total.value, np.array(list(stages), dtype=np.uint64)
    for a in (dX, dC, dP, dA, xn, cn, dR, idx, dist):
        a.free()
    return out


def _last_overflow(capi, ctx):
    over = ctypes.c_uint64()
    capi.check(ctx.lib.skm_ctx_get_last_overflow(ctx.handle, ctypes.byref(over)))
    return over.value


def _setup(oracle, blobs, n, d, k, seed, std=0.3):
    X = blobs(n, d, k, std=std, seed=seed)
    g = np.random.default_rng(seed + 1)
    C = X[g.choice(n, k, replace=False)].copy()
    # one Lloyd step so that "previous assignments" are a realistic seed for the threshold
    prev, _ = oracle.find_nn(X, C)
    C2, sizes = oracle.update_centroids(X, prev, k, scale=True)
    C2[sizes == 0] = C[sizes == 0]
    return X, C2, prev


@pytest.mark.parametrize("n,d,k,partial_d", [(4000, 128, 300, 32), (6000, 256, 1500, 32), (3000, 768, 1100, 96),
                                             (4000, 1024, 2500, 128), (1500, 600, 1030, 77), (1000, 132, 260, 23),
                                             # shapes of the slice pipeline of the candidate kernel: one centroid tile
                                             # of two slices; two tiles of one masked slice; a last slice of a single
                                             # masked group; round_up(d', 32) equal to the row length; unaligned rows
                                             (600, 128, 100, 64), (300, 256, 129, 17), (700, 192, 300, 33),
                                             (500, 128, 257, 63), (400, 130, 200, 40)])
def test_pruned_matches_oracle(capi, ctx, oracle, blobs, n, d, k, partial_d):
    X, C, prev = _setup(oracle, blobs, n, d, k, seed=n + d)
    ratios = oracle.ratios(d, 1.5)
    gi, gd, gtotal, gst = _pruned(capi, ctx, oracle, X, C, prev, partial_d, ratios, accounting=True)
    oi, od, ocounts, ost = oracle.find_nn_pruned(X, C, prev, partial_d, ratios, accounting=True)
    bi, bbest, bsecond = oracle.brute_force(X, C)
    mism = np.nonzero(gi != oi)[0]
    tie = (bsecond - bbest) <= 1e-5 * np.maximum(bbest, 1e-12)
    for i in mism:
        assert gi[i] == bi[i] or tie[i], f"point {i}: gpu {gi[i]} oracle {oi[i]} brute {bi[i]}"
    assert len(mism) <= max(1, int(1e-4 * n))
    same = gi == oi
    assert np.allclose(gd[same], od[same], rtol=1e-4, atol=1e-6)
    # returned distance is the full squared distance to the returned centroid
    full = ((X.astype(np.float64) - C[gi].astype(np.float64)) ** 2).sum(1)
    assert np.allclose(gd, full, rtol=1e-4, atol=1e-6)
    # Not-pruned statistics feed TunePartialD.  Pairs entering every pruning step agree to fp32
    # threshold noise.  The total of the first test is looser: a point that is the only member of
    # its cluster sits exactly on its centroid, so its threshold is 0 and whether the incumbent's
    # own partial distance (a rounding residue of |x|^2 + |c|^2 - 2 x.c) counts as "< 0" is a coin
    # flip on either side; such a pair never enters a pruning step (pdxearch.h:140-143).
    assert gtotal <= n * k
    singletons = int((np.bincount(prev, minlength=k)[prev] == 1).sum())
    assert abs(int(gtotal) - int(ocounts.sum())) <= singletons + max(3, int(2e-3 * ocounts.sum()))
    assert gst[0] == gtotal and ost[0] == ocounts.sum()
    assert np.all(np.abs(gst[1:].astype(np.int64) - ost[1:].astype(np.int64)) <= np.maximum(3, 2e-3 * ost[1:]))
    # survivors shrink monotonically through the horizontal steps
    hs = gst[1:-1]
    assert np.all(hs[:-1] >= hs[1:])


# The register-stationary candidate kernel: every number of 8-column groups with both wavefront shapes (up to 88
# columns a wavefront owns 64 points, up to 160 it owns 32), d' not a multiple of 8, fewer points than a workgroup
# owns, point and centroid counts that are not multiples of 64, a d' beyond its range (161: the tiled kernel runs).
@pytest.mark.parametrize("n,d,k,partial_d", [(700, 128, 300, 8), (1000, 128, 100, 16), (1000, 132, 260, 23),
                                             (1700, 256, 1500, 32), (900, 256, 321, 40), (1200, 256, 1100, 49),
                                             (777, 256, 640, 64), (1100, 600, 1030, 77), (1125, 768, 1100, 88),
                                             (1200, 768, 1100, 89), (1300, 768, 1280, 96), (2600, 1024, 2500, 128),
                                             (100, 1024, 60, 103), (1100, 1024, 1088, 160), (300, 1024, 300, 161),
                                             (131, 512, 63, 72),
                                             # long d' (the 256 x 256 kernel's range): whole slices, a trailing slice of
                                             # one to four groups, rows that are not 16-byte aligned, a last tile of
                                             # a few centroids and of a few points
                                             (1500, 1536, 1300, 192), (1100, 1536, 1030, 268), (2300, 1536, 2100, 300),
                                             (800, 1536, 700, 375), (600, 1026, 520, 230), (1100, 2048, 1025, 512)])
def test_both_candidate_kernels_give_the_same_bits(capi, ctx, oracle, blobs, n, d, k, partial_d):
    X, C, prev = _setup(oracle, blobs, n, d, k, seed=n + d + partial_d)
    ratios = oracle.ratios(d, 1.5)
    tiled = _pruned(capi, ctx, oracle, X, C, prev, partial_d, ratios, accounting=True, kernel=1)
    stationary = _pruned(capi, ctx, oracle, X, C, prev, partial_d, ratios, accounting=True, kernel=2)
    assert np.array_equal(tiled[0], stationary[0])
    assert np.array_equal(tiled[1].view(np.uint32), stationary[1].view(np.uint32))
    assert tiled[2] == stationary[2]
    assert np.array_equal(tiled[3], stationary[3])
    big = _pruned(capi, ctx, oracle, X, C, prev, partial_d, ratios, accounting=True, kernel=3)  # 256 x 256 tiles
    _same_bits(tiled, big)
    oi, od, ocounts = oracle.find_nn_pruned(X, C, prev, partial_d, ratios)
    bi, bbest, bsecond = oracle.brute_force(X, C)
    tie = (bsecond - bbest) <= 1e-5 * np.maximum(bbest, 1e-12)
    gi = stationary[0]
    for i in np.nonzero(gi != oi)[0]:
        assert gi[i] == bi[i] or tie[i], f"point {i}: gpu {gi[i]} oracle {oi[i]} brute {bi[i]}"
    assert np.sum(gi != oi) <= max(1, int(1e-4 * n))


def _same_bits(a, b):
    assert np.array_equal(a[0], b[0])
    assert np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32))
    assert a[2] == b[2]
    assert np.array_equal(a[3], b[3])


# The two list walks (one point per wavefront; eight points pooled per wavefront): same assignments, same distance
# bits, same not-pruned totals and, with accounting, the same pairs entering every step.  Shapes: one batch and many,
# a last batch of a few centroids, point counts that leave the last wavefront with one to seven points, tight seeds
# (few survivors: the few-entry path) and random seeds (hundreds of survivors per batch: pool rounds, overflowing lists).
@pytest.mark.parametrize("n,d,k,partial_d,random_seeds", [(4000, 128, 300, 32, False), (6001, 256, 1500, 32, False),
                                                          (3003, 768, 1100, 96, False), (4000, 1024, 2500, 128, False),
                                                          (1502, 600, 1030, 76, False), (1000, 132, 260, 23, False),
                                                          (2050, 256, 1500, 32, True), (1237, 768, 3100, 64, True),
                                                          (9, 128, 20, 16, False), (3, 256, 1100, 16, True),
                                                          (2500, 512, 5000, 48, True)])
@pytest.mark.parametrize("accounting", [False, True])
def test_both_list_walks_give_the_same_bits(capi, ctx, oracle, blobs, n, d, k, partial_d, random_seeds, accounting):
    X, C, prev = _setup(oracle, blobs, max(n, k + 10), d, k, seed=3 * n + d + partial_d)
    X, prev = X[:n], prev[:n]
    if random_seeds:
        prev = np.random.default_rng(n).integers(0, k, n).astype(np.uint32)
    ratios = oracle.ratios(d, 1.5)
    single = _pruned(capi, ctx, oracle, X, C, prev, partial_d, ratios, accounting=accounting, walk=1)
    for walk in (2, 3):
        pooled = _pruned(capi, ctx, oracle, X, C, prev, partial_d, ratios, accounting=accounting, walk=walk)
        _same_bits(single, pooled)
    # the pooled walk split into one launch per batch, or per range of batches, resumes from the state the launch before left
    for walk, launches in ((2, 2), (3, 1000)):
        split = _pruned(capi, ctx, oracle, X, C, prev, partial_d, ratios, accounting=accounting, walk=walk, launches=launches)
        _same_bits(single, split)


def test_both_list_walks_with_loose_ratios(capi, ctx, oracle, blobs):
    """Loose ratios: nearly every candidate survives many blocks, pools fill up (rounds over whole points, a point
    alone filling most of a pool) and most lists overflow into the pass over dense rows."""
    n, d, k = 3000, 256, 2600
    X, C, _ = _setup(oracle, blobs, n, d, k, seed=11)
    prev = np.random.default_rng(3).integers(0, k, n).astype(np.uint32)
    ratios = np.minimum(1.0, 3.0 * oracle.ratios(d, 1.5)).astype(np.float32)
    ratios[d] = 1.0
    for accounting in (False, True):
        single = _pruned(capi, ctx, oracle, X, C, prev, 40, ratios, accounting=accounting, walk=1)
        for walk in (2, 3):
            pooled = _pruned(capi, ctx, oracle, X, C, prev, 40, ratios, accounting=accounting, walk=walk)
            _same_bits(single, pooled)
    ones = np.ones(d + 1, dtype=np.float32)  # nothing is ever pruned: every pool is as full as it can get
    single = _pruned(capi, ctx, oracle, X[:600], C, prev[:600], 40, ones, accounting=True, walk=1)
    for walk in (2, 3):
        pooled = _pruned(capi, ctx, oracle, X[:600], C, prev[:600], 40, ones, accounting=True, walk=walk)
        _same_bits(single, pooled)
    bi, bbest, bsecond = oracle.brute_force(X[:600], C)
    tie = (bsecond - bbest) <= 1e-5 * np.maximum(bbest, 1e-12)
    assert np.all((pooled[0] == bi) | tie)


def test_both_candidate_kernels_with_overflowing_lists(capi, ctx, oracle, blobs):
    """Random seeds at k > 1024: thresholds are loose, many points collect more candidates than their list holds
    (cap = 1024 slots) and are searched again through dense rows; the two kernels must still agree bit for bit."""
    n, d, k = 3000, 256, 2600
    X, C, _ = _setup(oracle, blobs, n, d, k, seed=11)
    prev = np.random.default_rng(3).integers(0, k, n).astype(np.uint32)
    ratios = np.minimum(1.0, 3.0 * oracle.ratios(d, 1.5)).astype(np.float32)  # looser still: most lists overflow
    ratios[d] = 1.0
    tiled = _pruned(capi, ctx, oracle, X, C, prev, 40, ratios, kernel=1)
    over = _last_overflow(capi, ctx)
    assert n // 2 < over <= n  # most points went through the second pass
    stationary = _pruned(capi, ctx, oracle, X, C, prev, 40, ratios, kernel=2)
    assert _last_overflow(capi, ctx) == over
    big = _pruned(capi, ctx, oracle, X, C, prev, 40, ratios, kernel=3)
    assert np.array_equal(tiled[0], stationary[0]) and np.array_equal(tiled[0], big[0])
    assert np.array_equal(tiled[1].view(np.uint32), stationary[1].view(np.uint32))
    assert np.array_equal(tiled[1].view(np.uint32), big[1].view(np.uint32))
    assert tiled[2] == stationary[2] == big[2]
    oi, od, ocounts = oracle.find_nn_pruned(X, C, prev, 40, ratios)
    assert np.mean(stationary[0] == oi) >= 0.9999


def test_automatic_choice_of_the_candidate_kernel_at_many_points(capi, ctx, oracle, blobs):
    """49,152 points and more select the register-stationary kernel by themselves; checked against the oracle."""
    n, d, k, partial_d = 60000, 128, 1100, 32
    X, C, prev = _setup(oracle, blobs, n, d, k, seed=9)
    ratios = oracle.ratios(d, 1.5)
    auto = _pruned(capi, ctx, oracle, X, C, prev, partial_d, ratios)
    tiled = _pruned(capi, ctx, oracle, X, C, prev, partial_d, ratios, kernel=1)
    assert np.array_equal(auto[0], tiled[0]) and np.array_equal(auto[1].view(np.uint32), tiled[1].view(np.uint32))
    assert auto[2] == tiled[2]
    oi, od, ocounts = oracle.find_nn_pruned(X, C, prev, partial_d, ratios)
    bi, bbest, bsecond = oracle.brute_force(X, C)
    tie = (bsecond - bbest) <= 1e-5 * np.maximum(bbest, 1e-12)
    mism = np.nonzero(auto[0] != oi)[0]
    assert all(auto[0][i] == bi[i] or tie[i] for i in mism)
    assert len(mism) <= int(1e-4 * n)


@pytest.mark.parametrize("n,d,k,partial_d,random_seeds", [(3001, 768, 1100, 96, False), (2050, 256, 1500, 32, True),
                                                          (37, 128, 20, 16, False)])
def test_visiting_order_left_by_the_update_does_not_change_results(capi, ctx, oracle, blobs, n, d, k, partial_d, random_seeds):
    """After skm_update on a context, the pruned search of the same number of points takes them grouped by the
    assignments that update sorted (eight contiguous ranges of that order, one per compute die).  Results must be
    those of a context that never ran an update (plain point order), bit for bit, also when the order is stale
    (sorted by other assignments than the ones the search starts from) and when the last group of four points is
    incomplete or some dies get no group at all."""
    X, C, prev = _setup(oracle, blobs, n, d, k, seed=7 * n + d)
    g = np.random.default_rng(n)
    if random_seeds:
        prev = g.integers(0, k, n).astype(np.uint32)  # loose thresholds: overflowing lists take part as well
    ratios = oracle.ratios(d, 1.5)
    fresh = capi.Context(0)
    try:
        plain = _pruned(capi, fresh, oracle, X, C, prev, partial_d, ratios, accounting=True)
    finally:
        fresh.close()
    for sorted_by in (prev, g.integers(0, k, n).astype(np.uint32)):
        dX, dA = ctx.array(X), ctx.array(np.ascontiguousarray(sorted_by, dtype=np.uint32))
        sums, sizes = ctx.empty((k, d)), ctx.empty(k, np.uint32)
        capi.check(ctx.lib.skm_update(ctx.handle, dX.ptr, n, d, dA.ptr, k, sums.ptr, sizes.ptr))
        for a in (dX, dA, sums, sizes):
            a.free()
        ordered = _pruned(capi, ctx, oracle, X, C, prev, partial_d, ratios, accounting=True)
        assert np.array_equal(plain[0], ordered[0])
        assert np.array_equal(plain[1].view(np.uint32), ordered[1].view(np.uint32))
        assert plain[2] == ordered[2]
        assert np.array_equal(plain[3], ordered[3])


def test_pruned_with_unit_ratios_is_exact(capi, ctx, oracle, blobs):
    """With every ratio = 1 the bound partial <= full is safe, so the search must equal brute force."""
    n, d, k = 3000, 256, 1300
    X, C, prev = _setup(oracle, blobs, n, d, k, seed=77)
    ratios = np.ones(d + 1, dtype=np.float32)
    gi, gd, _, _ = _pruned(capi, ctx, oracle, X, C, prev, 32, ratios)
    bi, bbest, bsecond = oracle.brute_force(X, C)
    tie = (bsecond - bbest) <= 1e-5 * np.maximum(bbest, 1e-12)
    assert np.all((gi == bi) | tie)
    assert np.allclose(gd, bbest, rtol=1e-4, atol=1e-6)


def test_pruned_bad_seed_assignments_still_converge_to_nearest(capi, ctx, oracle, blobs):
    """Random previous assignments give a loose first threshold (many survivors) but the same answer."""
    n, d, k = 1500, 256, 1100
    X, C, _ = _setup(oracle, blobs, n, d, k, seed=5)
    prev = np.random.default_rng(1).integers(0, k, n).astype(np.uint32)
    ratios = oracle.ratios(d, 1.5)
    gi, gd, gtotal, _ = _pruned(capi, ctx, oracle, X, C, prev, 32, ratios)
    oi, od, ocounts = oracle.find_nn_pruned(X, C, prev, 32, ratios)
    bi, _, _ = oracle.brute_force(X, C)
    assert np.mean(gi == oi) >= 0.9999
    assert np.mean(gi == bi) >= 0.98  # tests/test_assign.cpp:152-155
    assert abs(int(gtotal) - int(ocounts.sum())) <= max(3, int(1e-2 * ocounts.sum()))


def test_pruned_incumbent_only_survivor_keeps_seed_distance(capi, ctx, oracle):
    """Two far apart centroids: the only survivor is the incumbent, so the seed distance (full
    Horizontal over d, batch_computers.h:372-377) is returned unchanged (pdxearch.h:140-143)."""
    d = 128
    g = np.random.default_rng(2)
    C = np.zeros((2, d), dtype=np.float32)
    C[1] += 100.0
    X = (C[np.array([0, 1, 0, 1])] + 0.01 * g.standard_normal((4, d))).astype(np.float32)
    prev = np.array([0, 1, 0, 1], dtype=np.uint32)
    ratios = oracle.ratios(d, 1.5)
    gi, gd, gtotal, _ = _pruned(capi, ctx, oracle, X, C, prev, 32, ratios)
    assert _last_overflow(capi, ctx) == 0
    assert np.array_equal(gi, prev)
    assert gtotal == 4
    full = ((X.astype(np.float64) - C[prev].astype(np.float64)) ** 2).sum(1)
    assert np.allclose(gd, full, rtol=1e-5)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_shapes_every_kernel_and_walk_same_bits(capi, ctx, oracle, blobs, seed):
    """Ten seeded random shapes per case (1 to 5,000 points, 65 to 3,300 centroids, d from 128 to 1539 with and without
    16-byte aligned rows, d' from 8 up to 400, tight and random seeds, the reference's ratios or looser ones): every
    choice of candidate kernel, walk and number of walk launches returns the bits of the tiled kernel with the
    one-point walk, and what differs from the oracle is a tie or the exact answer."""
    g = np.random.default_rng(seed)
    for case in range(10):
        d = int(g.choice([128, 132, 192, 256, 260, 384, 512, 600, 768, 1024, 1280, 1536]))
        if g.random() < 0.15:
            d += int(g.integers(1, 4))
        _, V = oracle.dimension_split(d)
        k = int(g.integers(65, 3300))
        n = int(g.integers(1, 5000))
        partial_d = int(g.integers(8, max(9, min(V - 1, 400))))
        random_seeds, accounting = bool(g.random() < 0.4), bool(g.random() < 0.5)
        X, C, prev = _setup(oracle, blobs, max(n, k + 10), d, k, seed=1000 * seed + case)
        X, prev = X[:n], prev[:n]
        if random_seeds:
            prev = g.integers(0, k, n).astype(np.uint32)
        ratios = oracle.ratios(d, 1.5)
        if g.random() < 0.2:
            ratios = np.minimum(1.0, 2.5 * ratios).astype(np.float32)
            ratios[d] = 1.0
        what = f"n={n} d={d} k={k} d'={partial_d} random_seeds={random_seeds} accounting={accounting}"
        base = _pruned(capi, ctx, oracle, X, C, prev, partial_d, ratios, accounting=accounting, kernel=1, walk=1)
        for kernel, walk, launches in ((0, 0, 1), (2, 2, 1), (3, 3, 1), (1, 3, 3), (3, 2, 1000), (2, 1, 1)):
            other = _pruned(capi, ctx, oracle, X, C, prev, partial_d, ratios, accounting=accounting, kernel=kernel,
                            walk=walk, launches=launches)
            try:
                _same_bits(base, other)
            except AssertionError as e:
                raise AssertionError(f"{what}: kernel {kernel}, walk {walk}, {launches} launches") from e
        oi, _, _ = oracle.find_nn_pruned(X, C, prev, partial_d, ratios)
        bi, bbest, bsecond = oracle.brute_force(X, C)
        mism = np.nonzero(base[0] != oi)[0]
        tie = (bsecond - bbest) <= 1e-5 * np.maximum(bbest, 1e-12)
        assert all(base[0][i] == bi[i] or tie[i] for i in mism), what
        assert len(mism) <= max(1, int(1e-4 * n)), what
