"""GPU parity of the HBM-bound stages against the CPU oracle: PDX relayout, gather/scatter,
centroid update, scaling, WCSS, shift, row edits.  Integer / copy work is compared bit-exactly;
the centroid sums are bit-exact too because the device visits each centroid's points in the same
ascending order as the reference (superkmeans.h:742-750)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("k,d", [(1024, 128), (2048, 256), (2500, 256), (500, 768), (10000, 1024), (1, 64), (1030, 600), (300, 100)])
def test_pdxify_bit_exact(capi, ctx, oracle, k, d):
    C = np.random.default_rng(k + d).standard_normal((k, d)).astype(np.float32)
    _, V = oracle.dimension_split(d)
    dC, dP, dA = ctx.array(C), ctx.empty(k * d), ctx.empty((k, V))
    capi.check(ctx.lib.skm_pdxify(ctx.handle, dC.ptr, k, d, V, dP.ptr, dA.ptr))
    assert np.array_equal(dP.download(), oracle.pdxify(C))
    assert np.array_equal(dA.download(), C[:, :V])
    for a in (dC, dP, dA):
        a.free()


def test_pdxify_rejects_bad_split(capi, ctx):
    x = ctx.empty((8, 128))
    with pytest.raises(capi.SkmError):
        capi.check(ctx.lib.skm_pdxify(ctx.handle, x.ptr, 8, 128, 60, x.ptr, None))
    x.free()


@pytest.mark.parametrize("n,d,k,nthreads", [(5000, 128, 100, 1), (20000, 256, 1000, 8), (3000, 50, 7, 3), (10000, 1024, 300, 8),
                                            (70000, 64, 70000, 8), (257, 1536, 1, 2),
                                            # few centroids, long segments: columns of a centroid spread over several
                                            # workgroups, 32 rows in flight per thread; the order of additions is the same
                                            (40000, 1024, 9, 4), (50000, 512, 20, 2),
                                            # ragged column groups of the row-sum kernel: 33 and 5 float4 lanes, 20 and 200
                                            # single-float lanes (the last wavefront of a centroid is partly idle)
                                            (30000, 132, 3000, 2), (20000, 20, 3000, 1), (5000, 20, 10, 1), (30000, 200, 600, 3),
                                            # one sort pass with every digit a centroid (k = 256) and all but one (255):
                                            # the segment offsets come from the scatter kernel there
                                            (6000, 96, 256, 2), (4001, 64, 255, 1), (39062, 128, 256, 4)])
def test_update_sums_and_sizes_bit_exact(capi, ctx, oracle, n, d, k, nthreads):
    g = np.random.default_rng(n + d)
    X = g.standard_normal((n, d)).astype(np.float32)
    a = g.integers(0, k, n).astype(np.uint32)
    if k > 3:
        a[a == 2] = 3  # force an empty cluster
    dX, dA, dS, dZ = ctx.array(X), ctx.array(a), ctx.empty((k, d)), ctx.empty(k, np.uint32)
    capi.check(ctx.lib.skm_update(ctx.handle, dX.ptr, n, d, dA.ptr, k, dS.ptr, dZ.ptr))
    sums, sizes = dS.download(), dZ.download()
    rs, rz = oracle.update_centroids(X, a, k, scale=False, n_threads=nthreads)
    assert np.array_equal(sizes, rz)
    assert np.array_equal(sizes, np.bincount(a, minlength=k).astype(np.uint32))
    assert np.array_equal(sums, rs)  # same summation order as the reference -> identical bits
    if (n + k) % 2 == 0:
        capi.check(ctx.lib.skm_scale_by_size(ctx.handle, dS.ptr, dZ.ptr, k, d))
    else:
        # the variant that hands the sizes to the host on its way (a pinned copy up to 16,384 clusters, a copy beyond)
        import ctypes
        fetched = np.full(k, 0xffffffff, dtype=np.uint32)
        capi.check(ctx.lib.skm_scale_by_size_fetch(ctx.handle, dS.ptr, dZ.ptr, k, d,
                                                   fetched.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))))
        assert np.array_equal(fetched, rz)
    means = dS.download()
    rm, _ = oracle.update_centroids(X, a, k, scale=True, n_threads=nthreads)
    assert np.array_equal(means, rm)
    # closed form: fp64 mean of the assigned rows
    for c in np.unique(a)[:20]:
        exact = X[a == c].astype(np.float64).mean(0)
        assert np.allclose(means[c], exact, rtol=1e-4, atol=1e-5)
    for arr in (dX, dA, dS, dZ):
        arr.free()


@pytest.mark.gpu
@pytest.mark.parametrize("n,k", [(5000, 16), (100_000, 256), (300_001, 300), (1, 1), (70_000, 70_000), (2_000_000, 1000)])
def test_group_by_assignment_is_the_counting_sort_of_the_reference(capi, ctx, n, k):
    """The partitioned index between mesoclustering and fine clustering (reference hierarchical_superkmeans.h:270-286:
    offsets from the sizes, then every point appended to its mesocluster's list in point order) equals a stable
    argsort of the assignments; the sizes are the counts.  Integer work: array_equal."""
    g = np.random.default_rng(n + k)
    a = g.integers(0, k, n).astype(np.uint32)
    if k > 3:
        a[a == 1] = 0  # an empty group
    dA, dI, dZ = ctx.array(a), ctx.empty(n, np.uint64), ctx.empty(k, np.uint32)
    capi.check(ctx.lib.skm_group_by_assignment(ctx.handle, dA.ptr, n, k, dI.ptr, dZ.ptr))
    ids, sizes = dI.download(), dZ.download()
    assert np.array_equal(sizes, np.bincount(a, minlength=k).astype(np.uint32))
    assert np.array_equal(ids, np.argsort(a, kind="stable").astype(np.uint64))
    for arr in (dA, dI, dZ):
        arr.free()


def test_update_is_run_to_run_deterministic(capi, ctx):
    g = np.random.default_rng(0)
    X = g.standard_normal((50000, 96)).astype(np.float32)
    a = g.integers(0, 64, 50000).astype(np.uint32)
    dX, dA, dS, dZ = ctx.array(X), ctx.array(a), ctx.empty((64, 96)), ctx.empty(64, np.uint32)
    outs = []
    for _ in range(3):
        capi.check(ctx.lib.skm_update(ctx.handle, dX.ptr, 50000, 96, dA.ptr, 64, dS.ptr, dZ.ptr))
        outs.append(dS.download())
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    for arr in (dX, dA, dS, dZ):
        arr.free()


def test_wcss_and_shift(capi, ctx):
    import ctypes

    g = np.random.default_rng(4)
    dist = g.random(1_000_003).astype(np.float32)
    dd = ctx.array(dist)
    out = ctypes.c_double()
    capi.check(ctx.lib.skm_wcss(ctx.handle, dd.ptr, dist.size, ctypes.byref(out)))
    assert abs(out.value - dist.astype(np.float64).sum()) <= 1e-9 * dist.size
    a = g.standard_normal((777, 130)).astype(np.float32)
    b = g.standard_normal((777, 130)).astype(np.float32)
    da, db = ctx.array(a), ctx.array(b)
    capi.check(ctx.lib.skm_shift(ctx.handle, da.ptr, db.ptr, 777, 130, ctypes.byref(out)))
    exact = ((a.astype(np.float64) - b.astype(np.float64)) ** 2).sum()
    assert abs(out.value - exact) <= 1e-6 * exact
    capi.check(ctx.lib.skm_wcss(ctx.handle, dd.ptr, 0, ctypes.byref(out)))
    assert out.value == 0.0
    # the two-step form: other reductions and an update run between the two calls and leave the pending sum alone
    capi.check(ctx.lib.skm_wcss(ctx.handle, dd.ptr, dist.size, ctypes.byref(out)))
    whole = out.value
    capi.check(ctx.lib.skm_wcss_begin(ctx.handle, dd.ptr, dist.size))
    capi.check(ctx.lib.skm_shift(ctx.handle, da.ptr, db.ptr, 777, 130, ctypes.byref(out)))
    assign = ctx.array((np.arange(777) % 10).astype(np.uint32))
    sums, sizes = ctx.empty((10, 130)), ctx.empty(10, np.uint32)
    capi.check(ctx.lib.skm_update(ctx.handle, da.ptr, 777, 130, assign.ptr, 10, sums.ptr, sizes.ptr))
    capi.check(ctx.lib.skm_wcss(ctx.handle, da.ptr, 777 * 130, ctypes.byref(out)))
    capi.check(ctx.lib.skm_wcss_end(ctx.handle, ctypes.byref(out)))
    assert out.value == whole
    for arr in (dd, da, db, assign, sums, sizes):
        arr.free()


def test_gather_rows_and_scatter_assignments(capi, ctx):
    g = np.random.default_rng(6)
    X = g.standard_normal((5000, 200)).astype(np.float32)
    norms = g.random(5000).astype(np.float32)
    index = g.permutation(5000)[:1234].astype(np.uint64)
    dX, dN, dI = ctx.array(X), ctx.array(norms), ctx.array(index)
    dO, dNo = ctx.empty((1234, 200)), ctx.empty(1234)
    capi.check(ctx.lib.skm_gather_rows(ctx.handle, dX.ptr, 200, dI.ptr, 1234, dO.ptr, dN.ptr, dNo.ptr))
    assert np.array_equal(dO.download(), X[index])
    assert np.array_equal(dNo.download(), norms[index])
    local = g.integers(0, 50, 1234).astype(np.uint32)
    dL = ctx.array(local)
    full = np.full(5000, 0xFFFFFFFF, dtype=np.uint32)
    dF = ctx.array(full)
    capi.check(ctx.lib.skm_scatter_assignments(ctx.handle, dI.ptr, dL.ptr, 1234, 700, dF.ptr))
    expect = full.copy()
    expect[index] = local + 700
    assert np.array_equal(dF.download(), expect)
    for arr in (dX, dN, dI, dO, dNo, dL, dF):
        arr.free()


def test_edit_rows_matches_split_clusters(capi, ctx, oracle):
    """The copy+perturb edit reproduces SplitClusters' row arithmetic (superkmeans.h:905-920).  Every cluster but one
    has a single member, so its acceptance probability (size - 1) / (n - k) is zero and the first empty cluster can
    only take from the large one; the second empty cluster takes from the large one or from the first recipient, and
    which one it was shows in the sizes the oracle returns."""
    g = np.random.default_rng(8)
    k, d = 12, 64
    C = g.standard_normal((k, d)).astype(np.float32)
    sizes = np.ones(k, dtype=np.uint32)
    big, first, second = 5, 3, 7
    sizes[[first, second]] = 0
    sizes[big] = 301
    n = int(sizes.sum())
    rc, rs, nsplit = oracle.split_clusters(C, sizes, n, seed=42, hierarchical=False)
    assert nsplit == 2
    # after the first split: first = 150, big = 151
    if rs[big] == 151:      # the second split halved the first recipient: 150 -> 75 + 75
        assert (rs[first], rs[second]) == (75, 75)
        donor2 = first
    else:                   # the second split halved the large cluster again: 151 -> 76 + 75
        assert (rs[big], rs[first], rs[second]) == (76, 150, 75)
        donor2 = big
    ops = np.array([0, first, big, 0, 0, second, donor2, 0], dtype=np.uint32)
    dC = ctx.array(C)
    capi.check(ctx.lib.skm_edit_rows(ctx.handle, dC.ptr, d, ops.ctypes.data, 2))
    got = dC.download()
    dC.free()
    assert np.array_equal(got, rc)
    untouched = [c for c in range(k) if c not in (big, first, second)]
    assert np.array_equal(got[untouched], C[untouched])


@pytest.mark.parametrize("k,n_ops,seed", [(6, 300, 0), (40, 500, 1), (3000, 2000, 2)])
def test_edit_rows_dependent_edits_apply_in_order(capi, ctx, k, n_ops, seed):
    """Edits run concurrently where they touch disjoint rows and in order where one reads or writes a row another
    wrote (or writes a row another read): any sequence must give what one-after-the-other application gives, bit for
    bit.  Few rows and many edits make long dependency chains; many rows make wide rounds."""
    g = np.random.default_rng(seed)
    d = 70
    C = g.standard_normal((k, d)).astype(np.float32)
    ops = np.zeros((n_ops, 4), dtype=np.uint32)
    exp = C.copy()
    eps = np.float32(1.0 / 1024.0)
    even = np.arange(d) % 2 == 0
    for o in range(n_ops):
        kind = int(g.integers(0, 2))
        dst, src = (int(v) for v in g.choice(k, 2, replace=False))
        w = np.float32(g.integers(1, 8))
        ops[o] = (kind, dst, src, w.view(np.uint32))
        if kind == 0:
            v = exp[src].copy()
            exp[dst] = np.where(even, v * (np.float32(1) + eps), v * (np.float32(1) - eps))
            exp[src] = np.where(even, v * (np.float32(1) - eps), v * (np.float32(1) + eps))
        else:
            exp[dst] = (np.float32(0) + w * exp[dst] + np.float32(1) * exp[src]) / (w + np.float32(1))
    dC = ctx.array(C)
    capi.check(ctx.lib.skm_edit_rows(ctx.handle, dC.ptr, d, ops.ctypes.data, n_ops))
    assert np.array_equal(dC.download(), exp)
    dC.free()


def test_edit_rows_balancing_and_normalize(capi, ctx):
    g = np.random.default_rng(10)
    C = g.standard_normal((5, 96)).astype(np.float32)
    w = np.float32(3.0)
    o = np.array([1, 2, 4, w.view(np.uint32)], dtype=np.uint32)
    dC = ctx.array(C)
    capi.check(ctx.lib.skm_edit_rows(ctx.handle, dC.ptr, 96, o.ctypes.data, 1))
    got = dC.download()
    exp = C.copy()
    exp[2] = (np.float32(0) + w * C[2] + np.float32(1) * C[4]) / (w + np.float32(1))
    assert np.array_equal(got, exp)
    capi.check(ctx.lib.skm_normalize_rows(ctx.handle, dC.ptr, 5, 96))
    nrm = np.linalg.norm(dC.download().astype(np.float64), axis=1)
    assert np.allclose(nrm, 1.0, atol=1e-5)  # test_superkmeans.cpp:376-407
    dC.free()


def test_device_block_cache_limit_and_trim(capi, ctx):
    """Released blocks are kept for reuse up to the cache's byte limit: with the limit at zero a freed block goes back
    to the driver, with room it is handed out again by the next allocation of its size; trimming empties the cache.
    Checked through the addresses the allocator returns (a block of an unusual size, so that nothing else takes it)."""
    lib = ctx.lib
    size = (37 << 20) + 512
    capi.check(lib.skm_device_cache_trim(0))
    try:
        capi.check(lib.skm_device_cache_set_limit(0, 1 << 30))
        a = ctx.empty(size // 4)
        first = a.ptr
        a.free()
        b = ctx.empty(size // 4)
        assert b.ptr == first  # came back from the cache
        b.free()
        capi.check(lib.skm_device_cache_set_limit(0, 0))  # the idle block leaves with the lowered limit
        c = ctx.empty(size // 4)
        c.free()  # nothing is kept now
        capi.check(lib.skm_device_cache_trim(0))
    finally:
        capi.check(lib.skm_device_cache_set_limit(0, 48 << 30))


def test_seeds_from_groups(capi, ctx):
    """skm_seeds_from_groups: open entries (0xffffffff) take the representative of the point's group, the others stay;
    a group out of range counts as the last one."""
    g = np.random.default_rng(3)
    n, groups = 100_003, 37
    seeds = g.integers(0, 5000, n, dtype=np.uint32)
    seeds[g.random(n) < 0.7] = 0xFFFFFFFF
    group = g.integers(0, groups, n, dtype=np.uint32)
    seeds[5] = seeds[77] = 0xFFFFFFFF
    group[5], group[77] = groups, 0xFFFFFFF0
    rep = g.integers(0, 5000, groups, dtype=np.uint32)
    dS, dG, dR = ctx.array(seeds), ctx.array(group), ctx.array(rep)
    capi.check(ctx.lib.skm_seeds_from_groups(ctx.handle, dS.ptr, dG.ptr, dR.ptr, groups, n))
    want = np.where(seeds == 0xFFFFFFFF, rep[np.minimum(group, groups - 1)], seeds)
    assert np.array_equal(dS.download(), want)
    capi.check(ctx.lib.skm_seeds_from_groups(ctx.handle, dS.ptr, dG.ptr, dR.ptr, groups, 0))
    with pytest.raises(capi.SkmError):
        capi.check(ctx.lib.skm_seeds_from_groups(ctx.handle, dS.ptr, dG.ptr, dR.ptr, 0, n))
    for a in (dS, dG, dR):
        a.free()
