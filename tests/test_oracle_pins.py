"""Pins the CPU oracle itself (no GPU needed).

The oracle restates the reference's algorithm; nothing here retypes the oracle's formulas.  Each
check is either a golden table / property the reference's own tests hold, a closed form or hand-derived
value, an independent fp64 numpy computation, or an invariant the mathematics fixes.
"""
import numpy as np
import pytest


# ---- PDXLayout::GetDimensionSplit (pdx/layout.h:115-140) ----
def test_dimension_split_hand_derived_table(oracle):
    # d -> (horizontal, vertical), derived by hand from the rule
    table = {768: (576, 192), 1024: (768, 256), 1536: (1152, 384), 128: (64, 64), 64: (0, 64), 600: (448, 152),
             100: (0, 100), 1: (0, 1), 63: (0, 63), 65: (0, 65), 256: (64, 192), 257: (192, 65), 384: (320, 64),
             2048: (1536, 512), 900: (704, 196), 129: (64, 65), 192: (64, 128)}
    for d, hv in table.items():
        assert oracle.dimension_split(d) == hv, d


def test_dimension_split_properties(oracle):
    dims = [1, 2, 4, 8, 16, 32, 48, 63, 64, 65, 127, 128, 129, 191, 192, 193, 255, 256, 257, 384, 512, 600, 768, 900,
            1024, 1536, 2048, 3072, 4096]  # tests/test_pdx_layout.cpp:62-64
    for d in dims:
        h, v = oracle.dimension_split(d)
        assert h % 64 == 0 and h + v == d and v > 0  # :61-81, :100-108
        if d <= 64:
            assert h == 0  # :86-95


# ---- PDXify (pdx/layout.h:155-232), element map of tests/test_pdx_layout.cpp:30-52 ----
def _access_pdx(pdx, chunk, r, dim, d, V, m):
    off = chunk * 1024 * d
    if dim < V:
        return pdx[off + dim * m + r]
    h = dim - V
    return pdx[off + V * m + (h // 64) * m * 64 + r * 64 + (h % 64)]


@pytest.mark.parametrize("n,d", [(1024, 128), (2048, 256), (2500, 256), (500, 768), (3, 64), (1100, 600)])
def test_pdxify_element_map(oracle, n, d):
    x = np.random.default_rng(n + d).standard_normal((n, d)).astype(np.float32)
    pdx = oracle.pdxify(x)
    assert pdx.shape == (n * d,)
    _, V = oracle.dimension_split(d)
    g = np.random.default_rng(0)
    for _ in range(3000):
        i, j = int(g.integers(n)), int(g.integers(d))
        chunk, r = divmod(i, 1024)
        m = min(1024, n - chunk * 1024)
        assert _access_pdx(pdx, chunk, r, j, d, V, m) == x[i, j]
    assert np.array_equal(np.sort(pdx), np.sort(x.reshape(-1)))  # a permutation of the input


# ---- ADSampling ratios (pdx/adsampling.h:93-99,315-327) ----
def test_ratios_closed_form_and_spot_values(oracle):
    r = oracle.ratios(1024, 1.5)
    assert r.shape == (1025,) and r[0] == 1.0 and r[1024] == 1.0
    assert abs(r[128] - 0.125 * (1 + 1.5 / np.sqrt(128.0)) ** 2) < 1e-7  # ~0.16035
    assert abs(r[128] - 0.16035) < 1e-4
    assert abs(r[192] - 0.1875 * (1 + 1.5 / np.sqrt(192.0)) ** 2) < 1e-7
    v = np.arange(1, 1024, dtype=np.float64)
    exact = (v / 1024.0) * (1.0 + 1.5 / np.sqrt(v)) ** 2
    assert np.array_equal(r[1:1024], exact.astype(np.float32))
    assert np.all(np.diff(r[1:1024]) > 0)
    assert oracle.ratios(768, 1.1)[96] < oracle.ratios(768, 1.5)[96]  # hierarchical epsilon prunes harder


# ---- rotation (pdx/adsampling.h:48-86,156-299), invariants of tests/test_rotation.cpp ----
@pytest.mark.parametrize("d", [50, 128, 256, 512])
def test_rotation_invariants(oracle, d):
    Q = oracle.rotation_matrix(d, 42)
    Q64 = Q.astype(np.float64)
    assert np.abs(Q64 @ Q64.T - np.eye(d)).max() < 1e-5
    x = np.random.default_rng(d).standard_normal((200, d)).astype(np.float32)
    r = oracle.rotate(Q, x)
    assert np.abs(r - x.astype(np.float64) @ Q64.T).max() < 1e-5  # out = X Q^T
    back = oracle.unrotate(Q, r)
    assert np.abs(back - x).max() < 1e-4 and np.abs(back - x).mean() < 1e-5  # :56-149
    nx, nr = np.linalg.norm(x.astype(np.float64), axis=1), np.linalg.norm(r.astype(np.float64), axis=1)
    assert np.max(np.abs(nx - nr) / nx) < 1e-5  # :157-206
    ip_x, ip_r = x[:50].astype(np.float64) @ x[50:100].T, r[:50].astype(np.float64) @ r[50:100].T
    assert np.max(np.abs(ip_x - ip_r)) < 1e-4 * max(1.0, np.abs(ip_x).max())  # :217-259
    assert np.array_equal(Q, oracle.rotation_matrix(d, 42))  # same seed, :337-387
    assert not np.array_equal(Q, oracle.rotation_matrix(d, 43))


def test_rotation_spreads_energy(oracle):
    """After rotation the first d' coordinates carry about d'/d of every squared norm (the ADSampling premise)."""
    d = 256
    Q = oracle.rotation_matrix(d, 1)
    x = np.zeros((64, d), dtype=np.float32)
    x[np.arange(64), np.arange(64)] = 1.0  # axis-aligned: all energy in one coordinate
    r = oracle.rotate(Q, x)
    frac = (r[:, :64].astype(np.float64) ** 2).sum(1)
    assert abs(frac.mean() - 0.25) < 0.03


# ---- FindNearestNeighbor (batch_computers.h:104-171) ----
@pytest.mark.parametrize("n,k,d", [(100, 50, 32), (1000, 100, 64), (5000, 1000, 128), (500, 2000, 256), (1, 1, 1)])
def test_find_nn_against_fp64_brute_force(oracle, n, k, d):  # shapes of tests/test_distance_computers.cpp:89-95
    g = np.random.default_rng(n * 7 + k)
    X, C = g.standard_normal((n, d)).astype(np.float32), g.standard_normal((k, d)).astype(np.float32)
    idx, dist = oracle.find_nn(X, C)
    D = ((X.astype(np.float64)[:, None, :] - C.astype(np.float64)[None, :, :]) ** 2).sum(-1) if n * k * d < 5e7 else None
    if D is None:
        X64, C64 = X.astype(np.float64), C.astype(np.float64)
        D = (X64 ** 2).sum(1)[:, None] + (C64 ** 2).sum(1)[None, :] - 2 * X64 @ C64.T
    ref = D.argmin(1)
    for i in np.nonzero(idx != ref)[0]:
        assert abs(D[i, idx[i]] - D[i, ref[i]]) <= 1e-4 * D[i, ref[i]]
    assert np.allclose(dist, D.min(1), rtol=1e-4, atol=1e-5)
    bi, bbest, _ = oracle.brute_force(X, C)  # the oracle's own fp64 arbiter agrees with numpy
    assert np.array_equal(bi, ref) and np.allclose(bbest, D.min(1), rtol=1e-9)


def test_find_nn_ties_clamp_and_batch_rule(oracle):
    g = np.random.default_rng(3)
    base = g.standard_normal((8, 64)).astype(np.float32)
    C = np.tile(base, (300, 1))  # duplicates within and across the 1024-wide batches
    X = base + 0.01 * g.standard_normal((8, 64)).astype(np.float32)
    idx, dist = oracle.find_nn(X, C)
    assert np.array_equal(idx, np.arange(8, dtype=np.uint32))  # first minimum wins (minCoeff, strict <)
    idx0, dist0 = oracle.find_nn(base, C)  # points equal to centroids: distance clamped at 0 (:165)
    assert np.all(dist0 >= 0.0) and np.all(dist0 < 1e-4)
    assert np.all(idx0 % 8 == np.arange(8))


# ---- FindNearestNeighborWithPruning + PDXearch (batch_computers.h:297-409, pdxearch.h) ----
def _lloyd_state(oracle, blobs, n, d, k, seed):
    X = blobs(n, d, k, std=0.3, seed=seed)
    C = X[np.random.default_rng(seed).choice(n, k, replace=False)].copy()
    prev, _ = oracle.find_nn(X, C)
    C2, sizes = oracle.update_centroids(X, prev, k, scale=True)
    C2[sizes == 0] = C[sizes == 0]
    return X, C2, prev


def test_pruned_search_is_exact_when_ratios_are_one(oracle, blobs):
    X, C, prev = _lloyd_state(oracle, blobs, 3000, 256, 1300, 11)
    idx, dist, counts = oracle.find_nn_pruned(X, C, prev, 32, np.ones(257, dtype=np.float32))
    bi, bbest, bsecond = oracle.brute_force(X, C)
    tie = (bsecond - bbest) <= 1e-5 * np.maximum(bbest, 1e-12)
    assert np.all((idx == bi) | tie)
    assert np.allclose(dist, bbest, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("n,d,k,pd", [(4000, 128, 300, 32), (3000, 768, 1100, 96), (1500, 600, 1030, 77)])
def test_pruned_search_invariants(oracle, blobs, n, d, k, pd):
    X, C, prev = _lloyd_state(oracle, blobs, n, d, k, n + d)
    ratios = oracle.ratios(d, 1.5)
    idx, dist, counts, stages = oracle.find_nn_pruned(X, C, prev, pd, ratios, accounting=True)
    bi, bbest, _ = oracle.brute_force(X, C)
    assert np.mean(idx == bi) >= 0.98  # tests/test_assign.cpp:152-155
    X64, C64 = X.astype(np.float64), C.astype(np.float64)
    full = ((X64 - C64[idx]) ** 2).sum(1)
    assert np.allclose(dist, full, rtol=1e-4, atol=1e-6)  # returned distance is the full distance of the returned index
    seed_dist = ((X64 - C64[prev]) ** 2).sum(1)
    assert np.all(dist <= seed_dist * (1 + 1e-5) + 1e-7)  # never worse than the seed
    assert np.all(counts <= k) and stages[0] == counts.sum()
    assert np.all(np.diff(stages[1:-1].astype(np.int64)) <= 0)  # survivors only shrink
    assert stages[-1] <= stages[-2]


def test_pruned_search_two_clusters_by_hand(oracle):
    d = 128
    g = np.random.default_rng(2)
    C = np.zeros((2, d), dtype=np.float32)
    C[1] += 100.0
    X = (C[np.array([0, 1, 0, 1])] + 0.01 * g.standard_normal((4, d))).astype(np.float32)
    ratios = oracle.ratios(d, 1.5)
    idx, dist, counts = oracle.find_nn_pruned(X, C, np.array([0, 1, 0, 1], dtype=np.uint32), 32, ratios)
    assert np.array_equal(idx, [0, 1, 0, 1]) and np.array_equal(counts, [1, 1, 1, 1])
    idx2, _, counts2 = oracle.find_nn_pruned(X, C, np.array([1, 0, 1, 0], dtype=np.uint32), 32, ratios)
    assert np.array_equal(idx2, [0, 1, 0, 1])  # a wrong seed is corrected
    assert np.all(counts2 == 2)  # loose threshold: both centroids pass the first test


# ---- UpdateCentroids / ConsolidateCentroids (superkmeans.h:729-765,940-951) ----
def test_update_is_the_mean_of_assigned_rows_and_thread_independent(oracle):
    g = np.random.default_rng(5)
    X = g.standard_normal((20000, 96)).astype(np.float32)
    a = g.integers(0, 130, 20000).astype(np.uint32)
    a[a == 7] = 8
    s1, z1 = oracle.update_centroids(X, a, 130, scale=False, n_threads=1)
    s8, z8 = oracle.update_centroids(X, a, 130, scale=False, n_threads=8)
    assert np.array_equal(s1, s8) and np.array_equal(z1, z8)  # order of summation is ascending in i for any team size
    assert np.array_equal(z1, np.bincount(a, minlength=130)) and z1[7] == 0 and not s1[7].any()
    m, _ = oracle.update_centroids(X, a, 130, scale=True)
    for c in (0, 8, 50, 129):
        assert np.allclose(m[c], X[a == c].astype(np.float64).mean(0), rtol=1e-4, atol=1e-5)


# ---- SplitClusters (superkmeans.h:890-928; hierarchical_superkmeans.h:579-678) ----
def test_split_clusters_flat(oracle):
    g = np.random.default_rng(8)
    k, d = 12, 64
    C = g.standard_normal((k, d)).astype(np.float32)
    sizes = np.full(k, 100, dtype=np.uint32)
    sizes[[3, 7]] = 0
    sizes[0] = 5000
    n = int(sizes.sum())
    c2, s2, n_split = oracle.split_clusters(C, sizes, n, seed=42)
    assert n_split == 2 and s2.sum() == n and np.all(s2 > 0)  # sizes conserved, nothing left empty
    eps = np.float32(1 / 1024)
    sign = np.where(np.arange(d) % 2 == 0, 1, -1).astype(np.float32)
    for dst in (3, 7):
        # the new row is some donor row times (1 +/- eps) alternating; the donor was scaled the other way
        ratio = c2[dst] / C
        donors = [c for c in range(k) if c not in (3, 7) and np.allclose(ratio[c], (1 + sign * eps) ** 1, rtol=3e-3)]
        assert len(donors) >= 1
    untouched = [c for c in range(k) if s2[c] == sizes[c] and c not in (3, 7)]
    assert all(np.array_equal(c2[c], C[c]) for c in untouched)
    c3, s3, _ = oracle.split_clusters(C, sizes, n, seed=42)
    assert np.array_equal(c2, c3) and np.array_equal(s2, s3)  # engine reseeded on every call (:892)
    # exact arithmetic of one split with a forced donor: only cluster 0 can be accepted when all others have size 1
    sizes1 = np.ones(k, dtype=np.uint32)
    sizes1[3] = 0
    sizes1[0] = 1000
    c4, s4, ns = oracle.split_clusters(C, sizes1, int(sizes1.sum()), seed=1)
    assert ns == 1 and s4[3] == 500 and s4[0] == 500
    assert np.array_equal(c4[3], C[0] * (np.float32(1) + sign * eps))
    assert np.array_equal(c4[0], C[0] * (np.float32(1) - sign * eps))


def test_split_clusters_hierarchical_balancing(oracle):
    g = np.random.default_rng(9)
    k, d = 10, 64
    C = g.standard_normal((k, d)).astype(np.float32)
    sizes = np.full(k, 100, dtype=np.uint32)
    sizes[2] = 5     # below 25 % of the average (100): pulled towards a large cluster
    sizes[4] = 895   # the only cluster at or above the average besides the 100s
    n = int(sizes.sum())  # 1700 -> average 170, threshold 42
    c2, s2, n_split = oracle.split_clusters(C, sizes, n, seed=42, hierarchical=True)
    assert n_split == 1 and np.array_equal(s2, sizes)  # balancing does not change sizes
    w = np.float32(5.0)  # min(size, 7)
    expect = (np.float32(0) + w * C[2] + np.float32(1) * C[4]) / (w + np.float32(1))
    assert np.array_equal(c2[2], expect)
    assert all(np.array_equal(c2[c], C[c]) for c in range(k) if c != 2)


# ---- TunePartialD, ArrangeFineClusters, GetNMesoclusters ----
def test_tune_partial_d_table(oracle):
    n, k, V = 1000, 1000, 256
    def run(pct, pd):
        counts = np.full(n, int(pct * k), dtype=np.uint64)
        return oracle.tune_partial_d(counts, k, pd, V)
    assert run(0.04, 128) == (pytest.approx(0.04), 128)       # inside [3 %, 5 %]: unchanged
    assert run(0.10, 128)[1] == 128 + 51                        # + floor(128 * 0.2 * 2)
    assert run(0.10, 250)[1] == 256                             # clamped at vertical_d
    assert run(0.01, 128)[1] == 128 - 25                        # - floor(128 * 0.2)
    assert run(0.01, 18)[1] == 16                               # clamped at MIN_PARTIAL_D
    assert run(0.01, 16)[1] == 16
    assert run(0.10, 2)[1] == 3                                 # at least +1


def test_arrange_fine_clusters_and_mesoclusters(oracle):
    assert [oracle.n_mesoclusters(k) for k in (100, 1000, 10000, 65536, 2, 7)] == [10, 32, 100, 256, 1, 3]
    sizes = np.array([100, 300, 0, 600], dtype=np.uint32)
    out = oracle.arrange_fine_clusters(100, 1000, sizes)
    assert list(out) == [10, 30, 0, 60]
    sizes = np.array([1, 1, 998], dtype=np.uint32)
    out = oracle.arrange_fine_clusters(10, 1000, sizes)
    assert out.sum() == 10 and out[0] == 1 and out[1] == 1  # non-empty mesoclusters get at least one
    g = np.random.default_rng(0)
    for _ in range(20):
        sizes = g.integers(0, 500, 40).astype(np.uint32)
        sizes[-1] = max(sizes[-1], 1)
        ns = int(sizes.sum())
        out = oracle.arrange_fine_clusters(400, ns, sizes)
        assert out.sum() == 400 and np.all(out[sizes == 0][:-1] == 0) and np.all(out[:-1][sizes[:-1] > 0] >= 1)


# ---- ComputeShift, ShouldStopEarly, GetNVectorsToSample (superkmeans.h:988-998,1294-1333,1269-1277) ----
def test_shift_is_the_squared_movement_of_the_centroids(oracle, blobs):
    """stats[i].shift = sum_c |c_i - c_{i-1}|^2 over the rotated centroids: recomputed in fp64 from the centroids
    of two runs that differ by one iteration (runs are deterministic; a dropped square root, a missing square or a
    sum over the wrong pair of buffers would not pass)."""
    n, d, k = 4000, 64, 40
    X = blobs(n, d, k, std=0.4, seed=3)
    cfg = dict(sampling_fraction=1.0, early_termination=0, seed=42, unrotate_centroids=0)
    cents, shifts = [], None
    for iters in (1, 2, 3, 4):
        km = oracle.KMeans(k, d, iters=iters, **cfg)
        cents.append(km.train(X).astype(np.float64))
        shifts = [s.shift for s in km.stats()]
    for i in (1, 2, 3):
        exact = ((cents[i] - cents[i - 1]) ** 2).sum()
        assert shifts[i] == pytest.approx(exact, rel=1e-5), i
    assert shifts[1] > shifts[2] > shifts[3] > 0


def test_should_stop_early_follows_the_rule_of_the_statistics(oracle, blobs):
    """Early termination stops after the first iteration i (0-based) with shift_i < tol, or with i > 0 and
    cost_i / cost_{i-1} > 1 - tol.  The stopping iteration is predicted from the statistics of a run without early
    termination and compared with runs that have it, for tolerances that trigger either clause or neither."""
    n, d, k, iters = 5000, 64, 50, 12
    X = blobs(n, d, k, std=0.4, seed=5)
    base = dict(iters=iters, sampling_fraction=1.0, seed=42)
    full = oracle.KMeans(k, d, early_termination=0, **base)
    full.train(X)
    st = full.stats()
    assert len(st) == iters

    def predicted(tol):
        for i, s in enumerate(st):
            if s.shift < tol:
                return i + 1
            if i > 0 and np.float32(s.objective) / np.float32(st[i - 1].objective) > np.float32(1) - np.float32(tol):
                return i + 1
        return iters

    ratios = [st[i].objective / st[i - 1].objective for i in range(1, iters)]
    tols = [1e-12,                                  # neither clause: runs to the end unless the cost stalls exactly
            (1 - ratios[2]) * 1.5,                  # cost clause after a few iterations
            0.95,                                   # cost clause at once (second iteration)
            st[0].shift * 2.0]                      # shift clause in the first iteration
    seen = set()
    for tol in tols:
        km = oracle.KMeans(k, d, early_termination=1, tol=tol, **base)
        km.train(X)
        assert len(km.stats()) == predicted(tol), tol
        seen.add(len(km.stats()))
    assert 1 in seen and 2 in seen and len(seen) >= 3


def test_number_of_vectors_to_sample(oracle, blobs):
    """Flat: min(floor(float(n) * fraction), k * max_points_per_cluster), all n when the fraction is 1; hierarchical:
    floor(double(n) * fraction).  Observed through the number of training assignments a run keeps."""
    d = 16
    X = blobs(3001, d, 10, std=0.5, seed=1)
    def samples(n, k, hierarchical=False, **cfg):
        km = oracle.KMeans(k, d, hierarchical=hierarchical, iters=1, suppress_warnings=1, **cfg)
        km.train(X[:n])
        return len(km.state()[1])
    assert samples(3001, 10, sampling_fraction=1.0, max_points_per_cluster=1) == 3001
    assert samples(3001, 10, sampling_fraction=0.3, max_points_per_cluster=256) == 900        # floor(900.3)
    assert samples(3001, 10, sampling_fraction=0.5, max_points_per_cluster=100) == 1000       # 10 * 100 < 1500
    assert samples(2999, 7, sampling_fraction=0.9, max_points_per_cluster=99999) == int(np.floor(np.float32(2999) * np.float32(0.9)))
    assert samples(3001, 16, hierarchical=True, sampling_fraction=0.5, max_points_per_cluster=1,
                   iters_mesoclustering=1, iters_fineclustering=1) == 1500                   # no cap per cluster
    with pytest.raises(oracle.OracleError):
        samples(3001, 10, sampling_fraction=0.003, max_points_per_cluster=256)               # 9 samples < 10 clusters


# ---- whole Train(): reference golden WCSS tables and behavioural contract ----
def test_make_blobs_shape_statistics(golden_data):
    X = golden_data
    assert X.shape == (10000, 768) and np.isfinite(X).all()
    assert abs(X.std() - np.sqrt(25.0 + 0.0625)) < 0.2  # centres ~ N(0, 5^2), noise ~ N(0, 0.25^2)


@pytest.mark.parametrize("k", [10, 100, 250])
def test_flat_train_matches_reference_wcss_table(oracle, golden, golden_data, k):
    """tests/test_wcss.cpp:132-200 on the oracle: final WCSS within the reference's own bounds of its table."""
    for d_str, expected in golden["flat"][str(k)].items():
        d = int(d_str)
        km = oracle.KMeans(k, d, iters=10, seed=42, early_termination=0, sampling_fraction=1.0,
                           max_points_per_cluster=99999, n_threads=1)
        c = km.train(np.ascontiguousarray(golden_data[:, :d]))
        st = km.stats()
        assert len(st) == 10 and np.isfinite(c).all()
        for i in range(1, 10):
            assert st[i].objective <= st[i - 1].objective * 1.01  # :144-152
            assert st[i].iteration == i + 1
        assert expected * 0.5 <= st[-1].objective <= expected * 1.05, (k, d, st[-1].objective, expected)  # :154-170
        gemm_only = d < 128 or k <= 256  # :188-200
        assert st[0].is_gemm_only
        if gemm_only:
            assert all(s.is_gemm_only for s in st)
    oracle.set_threads(0)


@pytest.mark.parametrize("k", [100, 250])
def test_hierarchical_train_matches_reference_wcss_table(oracle, golden, golden_data, k):
    """tests/test_hierarchical_superkmeans.cpp:718-801 on the oracle (10 % tolerance)."""
    X = golden_data
    for d in (16, 128, 768):
        expected = golden["hierarchical"][str(k)][str(d)]
        km = oracle.KMeans(k, d, hierarchical=True, iters_mesoclustering=5, iters_fineclustering=5, iters_refinement=2,
                           seed=42, early_termination=0, suppress_warnings=1, n_threads=1)
        Xd = np.ascontiguousarray(X[:, :d])
        c = km.train(Xd)
        _, best, _ = oracle.brute_force(Xd, c)
        assert len(km.stats(1)) == 5 and len(km.stats(3)) == 2
        final = km.stats(3)[-1].objective
        assert expected * 0.5 <= final <= expected * 1.10, (k, d, final, expected)
    oracle.set_threads(0)


def test_train_contract(oracle, blobs):
    X = blobs(3000, 64, 50, seed=1)
    # exceptions (tests/test_superkmeans.cpp:91-211)
    for bad in (dict(iters=0), dict(sampling_fraction=0.0), dict(sampling_fraction=1.5)):
        with pytest.raises(oracle.OracleError) as e:
            oracle.KMeans(10, 64, **bad)
        assert e.value.kind == 1  # std::invalid_argument
    with pytest.raises(oracle.OracleError) as e:
        oracle.KMeans(0, 64)
    assert e.value.kind == 1
    km = oracle.KMeans(50, 64, iters=3)
    with pytest.raises(oracle.OracleError) as e:
        km.assign_training_points(X, X[:50])
    assert e.value.kind == 2  # std::runtime_error
    with pytest.raises(oracle.OracleError) as e:
        oracle.KMeans(50, 64).train(X[:49])
    assert e.value.kind == 2
    with pytest.raises(oracle.OracleError) as e:
        oracle.KMeans(50, 64, sampling_fraction=0.01).train(X)  # 30 samples < 50 clusters
    assert e.value.kind == 2
    c = km.train(X)
    with pytest.raises(oracle.OracleError) as e:
        km.train(X)
    assert e.value.kind == 2 and km.is_trained
    # all clusters used (:40-63), reproducible
    a = km.assign(X, c)
    assert len(np.unique(a)) == 50
    assert np.array_equal(c, oracle.KMeans(50, 64, iters=3).train(X))
    # angular -> unit-norm centroids (:376-407)
    ca = oracle.KMeans(50, 64, iters=3, angular=1).train(X)
    assert np.allclose(np.linalg.norm(ca.astype(np.float64), axis=1), 1.0, atol=1e-5)
    # early termination stops before the iteration budget on easy data (:217-310)
    ke = oracle.KMeans(50, 64, iters=25, early_termination=1, sampling_fraction=1.0)
    ke.train(X)
    assert len(ke.stats()) < 25


def test_assign_training_points_agreement(oracle, blobs):
    """>= 98 % agreement with brute-force Assign: full, sampled and hierarchical (tests/test_assign.cpp:118-246)."""
    X = blobs(20000, 128, 300, seed=4)
    for cfg in (dict(sampling_fraction=1.0), dict(sampling_fraction=0.5), dict(sampling_fraction=0.9)):
        km = oracle.KMeans(300, 128, iters=6, **cfg)
        c = km.train(X)
        assert np.mean(km.assign_training_points(X, c) == km.assign(X, c)) >= 0.98
    kh = oracle.KMeans(300, 128, hierarchical=True, suppress_warnings=1)
    ch = kh.train(X)
    assert np.mean(kh.assign_training_points(X, ch) == kh.assign(X, ch)) >= 0.98
    assert len(np.unique(kh.assign(X, ch))) >= 0.95 * 300


# ---- FindKNearestNeighbors (batch_computers.h:191-274), test shape of tests/test_distance_computers.cpp:201-262 ----
@pytest.mark.parametrize("n_x,n_y,d,k", [(1000, 500, 128, 10), (64, 3000, 96, 100), (7, 5, 16, 10)])
def test_find_knn_against_fp64_brute_force(oracle, n_x, n_y, d, k):
    rng = np.random.default_rng(42)
    x = rng.uniform(-10, 10, (n_x, d)).astype(np.float32)
    y = rng.uniform(-10, 10, (n_y, d)).astype(np.float32)
    knn, dist = oracle.find_knn(x, y, k)
    d64 = ((x.astype(np.float64)[:, None, :] - y.astype(np.float64)[None, :, :]) ** 2).sum(-1)
    order = np.argsort(d64, axis=1, kind="stable")[:, :k]
    kk = min(k, n_y)
    ref_d = np.take_along_axis(d64, order, axis=1)
    # indices equal unless the two distances tie to 1e-4 relative; distances within 1e-4 (the reference's bars)
    rel = np.abs(dist[:, :kk] - ref_d[:, :kk]) / np.maximum(ref_d[:, :kk], 1e-6)
    assert rel.max() <= 1e-4
    assert np.all((knn[:, :kk] == order[:, :kk]) | (rel <= 1e-4))
    assert np.mean(knn[:, :kk] == order[:, :kk]) > 0.999
    assert np.all(np.diff(dist[:, :kk], axis=1) >= 0)  # sorted
    if kk < k:  # slots beyond n_y stay unfilled (:204-205, :265-268)
        assert np.all(knn[:, kk:] == 0xFFFFFFFF) and np.all(dist[:, kk:] == np.finfo(np.float32).max)


def test_find_knn_batches_ties_and_progressive_clamp(oracle):
    # Hand-built: d = 1, queries and rows chosen so that every distance is exact in fp32.
    # Rows 0..1023 form batch 0, rows 1024.. batch 1.  Query 0 sits at 0.
    y = np.full((1030, 1), 100.0, dtype=np.float32)
    y[5, 0], y[900, 0], y[1025, 0], y[1027, 0] = 3.0, -3.0, 3.0, 1.0  # distances 9, 9, 9, 1
    x = np.zeros((1, 1), dtype=np.float32)
    knn, dist = oracle.find_knn(x, y, 3)
    # (distance, index) order: (1,1027), (9,5), (9,900); (9,1025) loses the tie on index
    assert knn[0].tolist() == [1027, 5, 900] and dist[0].tolist() == [1.0, 9.0, 9.0]
    # Progressive clamp: a negative raw distance is stored as 0 after its batch, so a smaller negative one
    # of a later batch sorts in front of it although its raw value is larger.
    x = np.ones((1, 1), dtype=np.float32)
    y[1027, 0] = 2.0                                   # -2*2 + 1 + 4 = 1
    ynorm = (y[:, 0] ** 2).astype(np.float32)          # rows at 100: -200 + 1 + 10000 = 9801
    xnorm = np.ones(1, dtype=np.float32)
    ynorm[5] = 3.0     # -2*3 + 1 + 3 = -2: a negative rounding residue, exaggerated
    ynorm[1025] = 4.0  # -2*3 + 1 + 4 = -1
    knn, dist = oracle.find_knn(x, y, 3, norms_x=xnorm, norms_y=ynorm)
    assert knn[0].tolist() == [1025, 5, 1027] and dist[0].tolist() == [0.0, 0.0, 1.0]


def test_recall_from_lists_by_hand(oracle):
    # 2 queries, objective_k = 4, explore = 2; assignments of 6 sample rows.
    assign = np.array([0, 1, 2, 2, 3, 1], dtype=np.uint32)
    gt = np.array([[0, 1, 2, 3], [4, 5, 0, 1]], dtype=np.uint32)          # clusters [0,1,2,2] and [3,1,0,1]
    promising = np.array([[2, 7], [1, 3]], dtype=np.uint32)                # hits: 2 of 4, 3 of 4
    assert oracle.recall_from_lists(gt, promising, assign) == np.float32((np.float32(0.5) + np.float32(0.75)) / 2)


# ---- DCT rotation variant (pdx/adsampling.h:52-74,162-189,229-271; reference builds with FFTW) ----
def test_dct_rotation_equals_sign_flip_plus_orthonormal_dct(oracle):
    from scipy.fft import dct
    d, seed = 512, 42
    rng = np.random.default_rng(0)
    x = rng.standard_normal((50, d)).astype(np.float32)
    out, used, m = oracle.rotate_kind(x, seed=seed, rotation_kind=1, want_matrix=True)
    assert used
    # signs: +1 where uniform_int_distribution<int>(0, 1) over mt19937(seed) draws 1, i.e. where the top bit
    # of the 32-bit draw is set; numpy's RandomState seeds MT19937 the same way as std::mt19937(seed)
    draws = np.random.RandomState(seed).randint(0, 2 ** 32, size=d, dtype=np.uint64)
    sign = np.where(draws >> 31 == 1, 1.0, -1.0)
    ref = dct(x.astype(np.float64) * sign, type=2, norm="ortho", axis=1)
    assert np.abs(out - ref).max() <= 2e-6 * np.abs(ref).max()
    m64 = m.astype(np.float64)
    assert np.abs(m64 @ m64.T - np.eye(d)).max() <= 1e-5          # orthonormal
    assert np.abs(x.astype(np.float64) @ m64.T - ref).max() <= 1e-5  # the explicit matrix is the same map
    back, _ = oracle.rotate_kind(out, seed=seed, rotation_kind=1, forward=False)
    assert np.abs(back - x).max() <= 1e-5                          # Unrotate inverts Rotate
    assert np.allclose((out.astype(np.float64) ** 2).sum(1), (x.astype(np.float64) ** 2).sum(1), rtol=1e-5)


def test_dct_rotation_applies_only_where_the_reference_would_use_it(oracle):
    x = np.ones((1, 256), dtype=np.float32)
    assert not oracle.rotate_kind(x, rotation_kind=1)[1] and not oracle.rotate_kind(x, rotation_kind=2)[1]  # d < 512
    x = np.ones((1, 768), dtype=np.float32)
    assert not oracle.rotate_kind(x, rotation_kind=1)[1]  # AVX2 builds: power of two only
    assert oracle.rotate_kind(x, rotation_kind=2)[1]
    assert not oracle.rotate_kind(np.ones((1, 1024), dtype=np.float32), rotation_kind=0)[1]
