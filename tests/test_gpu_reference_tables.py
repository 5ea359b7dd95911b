"""The reference's own end-to-end tests, run on the device path against the tables its tests hold.

Each test restates one TEST of the reference with the same configuration and the same acceptance
bars; the data are the regenerated MakeBlobs matrix the tables were produced on (a (k, d) cell uses
the first d columns).  The tables are fixtures (tests/golden/wcss_ground_truth.json), the oracle is
used only to regenerate the data and, where said, as a second opinion.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

FLAT = dict(iters=10, seed=42, early_termination=0, sampling_fraction=1.0, max_points_per_cluster=99999, n_threads=1)


def _check_flat(st, expected, k, d, tolerance):
    assert len(st) == 10
    for i in range(1, 10):
        assert st[i].objective <= st[i - 1].objective * 1.01, (k, d, i)  # test_wcss.cpp:144-152
        assert st[i].iteration == i + 1
    assert expected * 0.5 <= st[-1].objective <= expected * (1.0 + tolerance), (k, d, st[-1].objective, expected)


@pytest.mark.parametrize("k", [10, 100, 250])
def test_flat_wcss_table(capi, ctx, golden, golden_data, k):
    """tests/test_wcss.cpp:132-200: monotone WCSS, final value within 5 % above / 50 % below the table,
    pruning used exactly when d >= 128 and k > 256 (never on this grid) and the first iteration always GEMM only."""
    for d_str, expected in golden["flat"][str(k)].items():
        d = int(d_str)
        km = capi.KMeans(k, d, **FLAT)
        c = km.train(np.ascontiguousarray(golden_data[:, :d]))
        st = km.stats()
        assert c.shape == (k, d) and np.isfinite(c).all()
        _check_flat(st, expected, k, d, 0.05)
        assert st[0].is_gemm_only
        if d < 128 or k <= 256:  # test_wcss.cpp:188-200
            assert all(s.is_gemm_only for s in st)
        km.close()


@pytest.mark.parametrize("k", [10, 100, 250])
def test_flat_wcss_table_blas_only(capi, ctx, golden, golden_data, k):
    """tests/test_wcss.cpp:208-300: the same table with use_blas_only on the high-dimensional cells."""
    for d in (384, 512, 600, 768):
        expected = golden["flat"][str(k)][str(d)]
        km = capi.KMeans(k, d, use_blas_only=1, **FLAT)
        c = km.train(np.ascontiguousarray(golden_data[:, :d]))
        st = km.stats()
        assert np.isfinite(c).all()
        _check_flat(st, expected, k, d, 0.05)
        assert all(s.is_gemm_only for s in st)
        km.close()


def test_blas_only_disables_pruning_where_it_would_run(capi, ctx, oracle, golden_data):
    """A cell above both pruning thresholds (d >= 128, k > 256): with use_blas_only every iteration is GEMM only
    (superkmeans.h:164-170) and, before the first cluster split perturbs a centroid, the pruned run reaches the same
    objective because pruning is exact up to the ADSampling bound."""
    k, d = 300, 256
    X = np.ascontiguousarray(golden_data[:, :d])
    a = capi.KMeans(k, d, use_blas_only=1, **FLAT)
    b = capi.KMeans(k, d, **FLAT)
    o = oracle.KMeans(k, d, use_blas_only=1, **FLAT)
    a.train(X), b.train(X), o.train(X)
    sa, sb, so = a.stats(), b.stats(), o.stats()
    assert all(s.is_gemm_only for s in sa)
    assert sb[0].is_gemm_only and not any(s.is_gemm_only for s in sb[1:])
    for i in range(10):
        assert bool(so[i].is_gemm_only)
        if i and (so[i - 1].split or sa[i - 1].split or sb[i - 1].split):
            break
        assert abs(sa[i].objective - so[i].objective_f64) <= 1e-3 * so[i].objective_f64
        assert abs(sb[i].objective - sa[i].objective) <= 1e-3 * sa[i].objective
    a.close(), b.close()


@pytest.mark.parametrize("k", [10, 100, 250])
def test_hierarchical_wcss_table(capi, ctx, golden, golden_data, k):
    """tests/test_hierarchical_superkmeans.cpp:718-801: final refinement WCSS within 10 % above / 50 % below the
    table, refinement and every mesocluster's fine clustering monotone within 1 %, one block of
    iters_fineclustering entries per mesocluster."""
    n_meso = int(round(np.sqrt(k)))
    assert len(golden["hierarchical"][str(k)]) == 10  # all ten dimensionalities of test_hierarchical_superkmeans.cpp:805-809
    for d_str, expected in golden["hierarchical"][str(k)].items():
        d = int(d_str)
        km = capi.KMeans(k, d, hierarchical=True, iters_mesoclustering=5, iters_fineclustering=5, iters_refinement=2,
                         seed=42, early_termination=0, sampling_fraction=1.0, max_points_per_cluster=99999,
                         n_threads=1, suppress_warnings=1)
        c = km.train(np.ascontiguousarray(golden_data[:, :d]))
        assert c.shape == (k, d) and np.isfinite(c).all()
        ref, fine = km.stats(3), km.stats(2)
        assert len(ref) == 2
        assert expected * 0.5 <= ref[-1].objective <= expected * 1.10, (k, d, ref[-1].objective, expected)
        assert ref[1].objective <= ref[0].objective * 1.01
        assert len(fine) == n_meso * 5
        for m in range(n_meso):
            for i in range(1, 5):
                assert fine[m * 5 + i].objective <= fine[m * 5 + i - 1].objective * 1.01, (k, d, m, i)
        km.close()


def test_pre_rotated_data_gives_the_same_rotated_centroids(capi, ctx, golden_data):
    """tests/test_rotation.cpp:400-466: Train on raw data with unrotate_centroids off equals Train on data rotated
    beforehand with data_already_rotated on (same seed, so same rotation matrix and same initial centroids);
    every coordinate within 1e-4, as in the reference."""
    n, d, k = 10000, 256, 100
    g = np.random.default_rng(42)
    centers = g.uniform(-1, 1, (k, d)).astype(np.float32)
    X = (centers[g.integers(0, k, n)] + 0.1 * g.standard_normal((n, d))).astype(np.float32)
    cfg = dict(iters=10, seed=42, sampling_fraction=1.0, early_termination=0)
    a = capi.KMeans(k, d, unrotate_centroids=0, data_already_rotated=0, **cfg)
    Ca = a.train(X)
    Q, _ = capi.pruner_tables(d, 1.5, 42)
    dX, dQ, dR = ctx.array(X), ctx.array(Q), ctx.empty((n, d))
    capi.check(ctx.lib.skm_rotate(ctx.handle, dX.ptr, n, d, dQ.ptr, dR.ptr))
    Xrot = dR.download()
    b = capi.KMeans(k, d, unrotate_centroids=0, data_already_rotated=1, **cfg)
    Cb = b.train(Xrot)
    diff = np.abs(Ca - Cb)
    assert diff.max() < 1e-3 and diff.mean() < 1e-5  # test_rotation.cpp:451-465
    assert np.all(diff <= 1e-4)                      # test_rotation.cpp:441-449
    # the rotated centroids are the raw-space ones times Q^T (centroids are means, rotation is linear)
    c = capi.KMeans(k, d, unrotate_centroids=1, **cfg)
    Cc = c.train(X)
    assert np.abs(Cc.astype(np.float64) @ Q.astype(np.float64).T - Ca).max() < 1e-3
    for a_ in (dX, dQ, dR):
        a_.free()
    a.close(), b.close(), c.close()
