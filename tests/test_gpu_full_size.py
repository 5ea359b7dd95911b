"""The benchmark configurations at their real sizes, checked through size-independent properties and
sampled exact comparisons (the CPU oracle cannot run these sizes in test time; it arbitrates samples).

C1  flat Train + Assign        n=100,000    d=768  k=1,000    (the one size the CPU oracle runs in full: whole runs compared)
C2  flat Train + Assign        n=1,000,000  d=1024 k=10,000
C3  Assign only                n=10,000,000 d=1024 k=10,000   (41 GB of points resident in HBM)
C4  hierarchical Train+Assign  n=10,000,000 d=1024 k=65,536
C5  flat Train + Assign        n=2,000,000  d=1536 k=4,096    (low intrinsic dimension, heavy tails)

Properties: every index < k; Assign equals fp64 brute force on random samples (ties excepted);
sum of cluster sizes = n and sum of all centroid sums = sum of all points (linearity of the update);
WCSS equals the sum of the per-point distances and never increases by more than 1 % across
iterations; assigning twice gives identical output (determinism); pruned search agrees with exact
search on >= 98 % of points and reports the true distance of what it returns.
"""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _sample_rows(dX, n, d, count, seed):
    """Downloads `count` random rows of a device matrix (row by row through the C ABI)."""
    g = np.random.default_rng(seed)
    ids = np.sort(g.choice(n, count, replace=False))
    out = np.empty((count, d), dtype=np.float32)
    lib, h = dX.ctx.lib, dX.ctx.handle
    from superkmeans_amd import _capi

    for j, i in enumerate(ids):
        _capi.check(lib.skm_download(h, out[j].ctypes.data, dX.offset(int(i) * d), d * 4))
    return ids, out


def _check_assign_sample(oracle, ids, rows, centroids, assign):
    bi, bbest, bsecond = oracle.brute_force(rows, centroids)
    tie = (bsecond - bbest) <= 1e-5 * np.maximum(bbest, 1e-12)
    got = assign[ids]
    assert np.all((got == bi) | tie), f"{np.sum((got != bi) & ~tie)} sampled points differ from exact brute force"


def test_c1_flat_train_and_assign_whole_run_against_the_oracle(capi, ctx, oracle):
    """n = 100,000, d = 768, k = 1,000, 25 iterations: 1,000 centres ~ N(0, I), point = centre + 0.3 N(0, I), rows
    L2-normalised.  The oracle runs the whole configuration in seconds, so the two runs are compared iteration by
    iteration: same control flow (iteration kinds, d' schedule, split counts), WCSS within 1e-3 (1e-4 before the first
    split-induced near tie), not-pruned fraction within 1 %, final centroids within 1e-2 relative L2, <= 0.1 % of the
    training assignments different, Assign equal to fp64 brute force except on near ties."""
    n, d, k, iters = 100_000, 768, 1_000, 25
    g = np.random.default_rng(1)
    centres = g.standard_normal((k, d)).astype(np.float32)
    X = centres[g.integers(0, k, n)] + 0.3 * g.standard_normal((n, d)).astype(np.float32)
    X = np.ascontiguousarray(X / np.linalg.norm(X, axis=1, keepdims=True), dtype=np.float32)
    cfg = dict(iters=iters, sampling_fraction=1.0, early_termination=0, seed=42, suppress_warnings=1)
    km, ok = capi.KMeans(k, d, **cfg), oracle.KMeans(k, d, **cfg)
    C, OC = km.train(X), ok.train(X)
    gs, os_ = km.stats(), ok.stats()
    assert len(gs) == len(os_) == iters
    for a, b in zip(gs, os_):
        assert (a.iteration, bool(a.is_gemm_only), a.partial_d, a.split) == \
               (b.iteration, bool(b.is_gemm_only), b.partial_d, b.split)
        assert abs(a.objective - b.objective_f64) <= 1e-3 * b.objective_f64
        if not a.is_gemm_only:
            assert abs(a.not_pruned_pct - b.not_pruned_pct) <= 1e-2 * b.not_pruned_pct + 1e-6
    for a, b in zip(gs[:2], os_[:2]):
        assert abs(a.objective - b.objective_f64) <= 1e-4 * b.objective_f64
    assert gs[0].is_gemm_only and not any(s.is_gemm_only for s in gs[1:])
    assert all(gs[i].objective <= gs[i - 1].objective * 1.01 for i in range(1, iters))
    num = np.linalg.norm(C.astype(np.float64) - OC.astype(np.float64))
    assert num / np.linalg.norm(OC.astype(np.float64)) <= 1e-2
    _, oa, _, _ = ok.state()
    assert np.mean(km.assignments(n) != oa) <= 1e-3
    a1 = km.assign(X, C)
    ids = np.sort(g.choice(n, 20000, replace=False))
    _check_assign_sample(oracle, ids, X[ids], C, a1)
    assert np.mean(a1 != ok.assign(X, C)) <= 1e-4
    assert np.mean(km.assign_training_points(X, C) == a1) >= 0.98  # test_assign.cpp:118-155
    km.close()


def test_c2_flat_train_and_assign_full_size(capi, ctx, oracle):
    n, d, k = 1_000_000, 1024, 10_000
    iters = 10  # every launch shape of the benchmark's Train: d' goes 128 -> 24
    km = capi.KMeans(k, d, iters=iters, sampling_fraction=1.0, early_termination=0, suppress_warnings=1)
    c = km.ctx
    dX = c.empty((n, d))
    capi.check(km.lib.skm_synth_gaussian_mixture(c.handle, dX.ptr, n, d, 0, k, 1234, 5678, 1.0, 0.3, 0.25, 1))
    C = km.train_device(dX, n)
    st = km.stats()
    assert [bool(s.is_gemm_only) for s in st] == [True] + [False] * (iters - 1)
    assert all(st[i].objective <= st[i - 1].objective * 1.01 for i in range(1, iters))
    assert all(0 < s.not_pruned_pct <= 1 for s in st[1:]) and st[1].partial_d == 128
    pds = [s.partial_d for s in st[1:]]
    assert all(pds[i] <= pds[i - 1] for i in range(1, len(pds))) and pds[-1] <= 32  # the tuner shortens d' on this data
    assert np.isfinite(C).all() and C.shape == (k, d)
    train_assign = km.assignments(n)
    assert train_assign.max() < k
    # Assign: exact search, twice (determinism), sampled against fp64 brute force
    dC, dA, dB = c.array(C), c.empty(n, np.uint32), c.empty(n, np.uint32)
    km.assign_device(dX, dC, n, k, dA)
    km.assign_device(dX, dC, n, k, dB)
    a = dA.download()
    assert np.array_equal(a, dB.download()) and a.max() < k
    ids, rows = _sample_rows(dX, n, d, 1500, seed=1)
    _check_assign_sample(oracle, ids, rows, C, a)
    # update invariants on the full matrix (linearity / checksum of checksums)
    sums, sizes = c.empty((k, d)), c.empty(k, np.uint32)
    capi.check(km.lib.skm_update(c.handle, dX.ptr, n, d, dA.ptr, k, sums.ptr, sizes.ptr))
    hs, hz = sums.download(), sizes.download()
    assert int(hz.sum()) == n and np.array_equal(hz, np.bincount(a, minlength=k))
    ones = c.array(np.zeros(n, dtype=np.uint32))
    tot, tz = c.empty((1, d)), c.empty(1, np.uint32)
    capi.check(km.lib.skm_update(c.handle, dX.ptr, n, d, ones.ptr, 1, tot.ptr, tz.ptr))  # sum of all points
    total = tot.download()[0].astype(np.float64)
    assert np.allclose(hs.astype(np.float64).sum(0), total, rtol=0, atol=2e-3 * np.abs(total).max() + 1e-3)
    # WCSS of the exact assignment equals the sum of sampled exact distances scaled (consistency of distances)
    xn, cn, dist = c.empty(n), c.empty(k), c.empty(n)
    capi.check(km.lib.skm_norms(c.handle, dX.ptr, n, d, d, xn.ptr))
    capi.check(km.lib.skm_norms(c.handle, dC.ptr, k, d, d, cn.ptr))
    capi.check(km.lib.skm_assign_full(c.handle, dX.ptr, n, dC.ptr, k, d, xn.ptr, cn.ptr, dB.ptr, dist.ptr))
    w = ctypes.c_double()
    capi.check(km.lib.skm_wcss(c.handle, dist.ptr, n, ctypes.byref(w)))
    hd = dist.download()
    assert abs(w.value - hd.astype(np.float64).sum()) <= 1e-9 * n
    exact = ((rows.astype(np.float64) - C[a[ids]].astype(np.float64)) ** 2).sum(1)
    assert np.allclose(hd[ids], exact, rtol=1e-4, atol=1e-6)
    km.close()


def test_c2_last_train_iteration_against_the_oracle_and_the_exact_search(capi, ctx, oracle):
    """The last of the ten iterations of the headline Train runs at the short end of the d' schedule (24 columns of
    1024), where ADSampling prunes hardest.  Train is deterministic, so a nine-iteration run of the same object gives
    the state that iteration started from (rotated centroids, assignments).  From that state: (i) the oracle's pruned
    search on 2,000 sampled points (same seeds, same d') must return what Train's tenth iteration assigned, near ties
    excepted; (ii) the exact search over all points says how often the pruning kept the true nearest centroid: the
    reference's own bar is 98 % (tests/test_assign.cpp:152-155), and the oracle must show the same rate on the sample."""
    n, d, k = 1_000_000, 1024, 10_000
    c = capi.Context(0)
    dRaw = c.empty((n, d))
    capi.check(c.lib.skm_synth_gaussian_mixture(c.handle, dRaw.ptr, n, d, 0, k, 1234, 5678, 1.0, 0.3, 0.25, 1))
    c.sync()
    runs = {}
    for iters in (9, 10):
        km = capi.KMeans(k, d, iters=iters, sampling_fraction=1.0, early_termination=0, suppress_warnings=1, unrotate_centroids=0)
        runs[iters] = (km.train_device(dRaw, n), km.assignments(n), km.stats())
        km.close()
    (C9, a9, st9), (C10, a10, st10) = runs[9], runs[10]
    assert [(s.partial_d, s.objective) for s in st9] == [(s.partial_d, s.objective) for s in st10[:9]]  # same trajectory
    pd = st10[9].partial_d
    assert not st10[9].is_gemm_only and pd <= 32
    Q, _ = capi.pruner_tables(d, 1.5, 42)
    dQ, dX = c.array(Q), c.empty((n, d))
    capi.check(c.lib.skm_rotate(c.handle, dRaw.ptr, n, d, dQ.ptr, dX.ptr))
    c.sync()
    dRaw.free()
    # (ii) exact search of all points among the centroids the tenth iteration searched
    dC9, xn, cn = c.array(C9), c.empty(n), c.empty(k)
    a_exact, d_exact = c.empty(n, np.uint32), c.empty(n)
    capi.check(c.lib.skm_norms(c.handle, dX.ptr, n, d, d, xn.ptr))
    capi.check(c.lib.skm_norms(c.handle, dC9.ptr, k, d, d, cn.ptr))
    capi.check(c.lib.skm_assign_full(c.handle, dX.ptr, n, dC9.ptr, k, d, xn.ptr, cn.ptr, a_exact.ptr, d_exact.ptr))
    ae = a_exact.download()
    kept = float(np.mean(ae == a10))
    print(f"C2 iteration 10 (d' = {pd}): pruned search kept the exact nearest centroid for {100 * kept:.3f} % of the points")
    assert kept >= 0.98
    # (i) the oracle on a sample, from the same state
    ids, rows = _sample_rows(dX, n, d, 2000, seed=5)
    oi, od, _ = oracle.find_nn_pruned(rows, C9, a9[ids], pd, oracle.ratios(d, 1.5))
    bi, bbest, bsecond = oracle.brute_force(rows, C9)
    tie = (bsecond - bbest) <= 1e-5 * np.maximum(bbest, 1e-12)
    mism = np.nonzero(a10[ids] != oi)[0]
    assert all(a10[ids][i] == bi[i] or tie[i] for i in mism), "a sampled point differs from the oracle beyond a near tie"
    assert len(mism) <= 1
    assert np.array_equal(bi == oi, bi == a10[ids]) or len(mism) <= 1  # the oracle loses the same points to pruning
    assert abs(float(np.mean(oi == bi)) - float(np.mean(ae[ids] == a10[ids]))) <= 2e-3
    c.close()


def test_c2_pruned_search_full_size_against_exact_search(capi, ctx, oracle):
    """One pruned iteration at n = 1M, k = 10k from a realistic state, against the exact search on the same
    centroids: >= 98 % identical (the reference's own bar for its approximate pruning, tests/test_assign.cpp:152-155),
    returned distances are true distances, the not-pruned fraction is a small positive number."""
    n, d, k = 1_000_000, 1024, 10_000
    c = capi.Context(0)
    dRaw = c.empty((n, d))
    capi.check(c.lib.skm_synth_gaussian_mixture(c.handle, dRaw.ptr, n, d, 0, k, 1234, 5678, 1.0, 0.3, 0.25, 1))
    # ADSampling pruning presupposes the random rotation (the raw data concentrate their energy in the
    # leading dimensions): rotate exactly as Train does.
    Q, _ = capi.pruner_tables(d, 1.5, 42)
    dQ, dX = c.array(Q), c.empty((n, d))
    capi.check(c.lib.skm_rotate(c.handle, dRaw.ptr, n, d, dQ.ptr, dX.ptr))
    c.sync()
    dRaw.free()
    seed_rows = np.random.default_rng(0).choice(n, k, replace=False).astype(np.uint64)
    dIdx = c.array(np.sort(seed_rows))
    dC0 = c.empty((k, d))
    capi.check(c.lib.skm_gather_rows(c.handle, dX.ptr, d, dIdx.ptr, k, dC0.ptr, None, None))
    xn, cn = c.empty(n), c.empty(k)
    a0, dist0 = c.empty(n, np.uint32), c.empty(n)
    capi.check(c.lib.skm_norms(c.handle, dX.ptr, n, d, d, xn.ptr))
    capi.check(c.lib.skm_norms(c.handle, dC0.ptr, k, d, d, cn.ptr))
    capi.check(c.lib.skm_assign_full(c.handle, dX.ptr, n, dC0.ptr, k, d, xn.ptr, cn.ptr, a0.ptr, dist0.ptr))
    C1, sizes = c.empty((k, d)), c.empty(k, np.uint32)
    capi.check(c.lib.skm_update(c.handle, dX.ptr, n, d, a0.ptr, k, C1.ptr, sizes.ptr))
    capi.check(c.lib.skm_scale_by_size(c.handle, C1.ptr, sizes.ptr, k, d))
    assert sizes.download().min() >= 1  # every centroid is a data point, so it keeps at least itself
    # exact search on the new centroids
    a_exact, d_exact = c.empty(n, np.uint32), c.empty(n)
    capi.check(c.lib.skm_norms(c.handle, C1.ptr, k, d, d, cn.ptr))
    capi.check(c.lib.skm_assign_full(c.handle, dX.ptr, n, C1.ptr, k, d, xn.ptr, cn.ptr, a_exact.ptr, d_exact.ptr))
    # pruned search seeded with the previous assignment
    H, V = capi.dimension_split(d)
    pd = 128
    pdx, aux = c.empty(k * d), c.empty((k, V))
    capi.check(c.lib.skm_pdxify(c.handle, C1.ptr, k, d, V, pdx.ptr, aux.ptr))
    xnp, cnp = c.empty(n), c.empty(k)
    capi.check(c.lib.skm_norms(c.handle, dX.ptr, n, d, pd, xnp.ptr))
    capi.check(c.lib.skm_norms(c.handle, C1.ptr, k, d, pd, cnp.ptr))
    ratios = c.array(oracle.ratios(d, 1.5))
    a_pr, d_pr = c.array(a0.download()), c.empty(n)
    total = ctypes.c_uint64()
    stages = (ctypes.c_uint64 * (H // 64 + 2))()
    capi.check(c.lib.skm_assign_pruned(c.handle, dX.ptr, n, C1.ptr, pdx.ptr, aux.ptr, k, d, V, pd, ratios.ptr, xnp.ptr,
                                       cnp.ptr, a_pr.ptr, d_pr.ptr, ctypes.byref(total), stages))
    ae, ap, de, dp = a_exact.download(), a_pr.download(), d_exact.download(), d_pr.download()
    assert np.mean(ae == ap) >= 0.98
    same = ae == ap
    assert np.allclose(dp[same], de[same], rtol=1e-3, atol=1e-5)  # two formulas for the same distance
    assert np.all(dp[~same] >= de[~same] * (1 - 1e-4) - 1e-6)     # a pruned-away winner can only cost distance
    st = np.array(list(stages), dtype=np.uint64)
    assert st[0] == total.value and 0 < total.value < n * k * 0.2
    assert np.all(np.diff(st[1:-1].astype(np.int64)) <= 0)
    ids, rows = _sample_rows(dX, n, d, 2000, seed=3)
    C1h = C1.download()
    true = ((rows.astype(np.float64) - C1h[ap[ids]].astype(np.float64)) ** 2).sum(1)
    assert np.allclose(dp[ids], true, rtol=1e-4, atol=1e-6)
    # The search of a point does not depend on the other points, so the oracle arbitrates a sample: the same
    # 2,000 rows, the same 10,000 centroids in ten batches, the same seeds.  Equal except near ties.
    oi, od, _ = oracle.find_nn_pruned(rows, C1h, a0.download()[ids], pd, oracle.ratios(d, 1.5))
    bi, bbest, bsecond = oracle.brute_force(rows, C1h)
    tie = (bsecond - bbest) <= 1e-5 * np.maximum(bbest, 1e-12)
    mism = np.nonzero(ap[ids] != oi)[0]
    assert all(ap[ids][i] == bi[i] or tie[i] for i in mism), "a sampled point differs from the oracle beyond a near tie"
    assert len(mism) <= 1
    assert np.allclose(dp[ids][ap[ids] == oi], od[ap[ids] == oi], rtol=1e-4, atol=1e-6)
    c.close()


def test_c3_assign_only_ten_million_points(capi, ctx, oracle):
    n, d, k = 10_000_000, 1024, 10_000
    km = capi.KMeans(k, d, sampling_fraction=1.0, suppress_warnings=1)
    c = km.ctx
    dX = c.empty((n, d))  # 41 GB
    capi.check(km.lib.skm_synth_gaussian_mixture(c.handle, dX.ptr, n, d, 0, k, 77, 78, 1.0, 0.5, 0.0, 1))
    dC = c.empty((k, d))  # the mixture's own centres: rows of the generator with zero noise
    capi.check(km.lib.skm_synth_gaussian_mixture(c.handle, dC.ptr, k, d, 0, 0, 0, 79, 0.0, 1.0, 0.0, 1))
    C = dC.download()
    dA = c.empty(n, np.uint32)
    km.assign_device(dX, dC, n, k, dA)
    a = dA.download()
    assert a.max() < k
    ids, rows = _sample_rows(dX, n, d, 1000, seed=5)
    _check_assign_sample(oracle, ids, rows, C, a)
    sizes = np.bincount(a, minlength=k)
    assert sizes.sum() == n
    km.close()


def test_c4_hierarchical_ten_million_points(capi, ctx, oracle):
    n, d, k = 10_000_000, 1024, 65_536
    km = capi.KMeans(k, d, hierarchical=True, suppress_warnings=1, early_termination=0)
    c = km.ctx
    dX = c.empty((n, d))
    capi.check(km.lib.skm_synth_two_level_mixture(c.handle, dX.ptr, n, d, 0, 256, 65_536, 9, 0.2, 0.1))
    C = km.train_device(dX, n)
    assert C.shape == (k, d) and np.isfinite(C).all()
    meso, fine, refine = km.stats(1), km.stats(2), km.stats(3)
    assert len(meso) == 3 and len(refine) == 0 and 0 < len(fine) <= 256 * 5
    assert all(s.is_gemm_only for s in meso)  # 256 mesoclusters <= pruning threshold
    assert all(meso[i].objective <= meso[i - 1].objective * 1.01 for i in range(1, 3))
    a = km.assignments(n)
    assert a.max() < k
    used = len(np.unique(a))
    assert used >= 0.95 * k  # tests/test_hierarchical_superkmeans.cpp:554-587
    # exact Assign of a slice of the points against the returned centroids, sampled against brute force
    m = 200_000
    dC, dA = c.array(C), c.empty(m, np.uint32)
    km.assign_device(dX, dC, m, k, dA)
    sa = dA.download()
    ids, rows = _sample_rows(dX, m, d, 300, seed=7)
    _check_assign_sample(oracle, ids, rows, C, sa)
    km.close()


def test_c5_low_intrinsic_dimension_heavy_tails(capi, ctx, oracle):
    n, d, k = 2_000_000, 1536, 4_096
    km = capi.KMeans(k, d, iters=3, sampling_fraction=1.0, early_termination=0, suppress_warnings=1)
    c = km.ctx
    dX = c.empty((n, d))
    capi.check(km.lib.skm_synth_low_rank(c.handle, dX.ptr, n, d, 0, 64, 21, 0.05))
    C = km.train_device(dX, n)
    st = km.stats()
    assert [bool(s.is_gemm_only) for s in st] == [True, False, False] and st[1].partial_d == 192
    assert all(st[i].objective <= st[i - 1].objective * 1.01 for i in range(1, 3))
    assert np.isfinite(C).all()
    dC, dA = c.array(C), c.empty(n, np.uint32)
    km.assign_device(dX, dC, n, k, dA)
    a = dA.download()
    assert a.max() < k and np.bincount(a, minlength=k).sum() == n
    ids, rows = _sample_rows(dX, n, d, 800, seed=11)
    _check_assign_sample(oracle, ids, rows, C, a)
    km.close()
