"""The Python package on the GPU backend: behaviour pinned by the reference's own API tests
(python/tests/test_superkmeans.py; cited per test)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pkg(ctx):  # ctx: skips when there is no device
    import superkmeans_amd

    return superkmeans_amd


def _data(n, d, seed=42):
    return np.random.default_rng(seed).standard_normal((n, d)).astype(np.float32)


def test_constructor_and_validation(pkg):
    km = pkg.SuperKMeans(n_clusters=10, dimensionality=50)  # :9-12
    assert km.n_clusters_ == 10 and not km.is_trained_
    assert km.iteration_stats == [] and km.hierarchical_iteration_stats is None
    for bad in (dict(n_clusters=0, dimensionality=50), dict(n_clusters=10, dimensionality=0),
                dict(n_clusters=10, dimensionality=50, sampling_fraction=1.5)):  # :26-32
        with pytest.raises(ValueError):
            pkg.SuperKMeans(**bad)
    r = repr(km)  # :171-180
    assert "SuperKMeans" in r and "n_clusters=10" in r and "dimensionality=50" in r and "trained=False" in r
    assert set(pkg.__all__) == {"__version__", "SuperKMeans", "SuperKMeansIterationStats",
                                "HierarchicalSuperKMeansIterationStats"}
    assert pkg.SuperKMeans.add is pkg.SuperKMeans.assign


def test_train_assign_shapes_dtypes_and_stats(pkg):
    n, d, k = 10000, 512, 100
    data = _data(n, d)
    km = pkg.SuperKMeans(n_clusters=k, dimensionality=d, iters=5)
    c = km.train(data)  # :34-48
    assert c.shape == (k, d) and c.dtype == np.float32 and km.is_trained_
    a = km.assign(data, c)  # :66-82
    assert a.shape == (n,) and a.dtype == np.uint32 and a.max() < k
    other = km.assign(_data(500, d, seed=1), c)  # :84-100
    assert other.shape == (500,) and other.max() < k
    stats = km.iteration_stats  # :100-117
    assert len(stats) == 5
    for i, s in enumerate(stats):
        assert isinstance(s, pkg.SuperKMeansIterationStats)
        assert s.iteration == i + 1 and s.objective > 0 and s.shift >= 0
    assert "trained=True" in repr(km) and "hierarchical=False" in repr(km)
    with pytest.raises(RuntimeError):
        km.train(data)  # already trained


def test_input_validation_messages(pkg):
    km = pkg.SuperKMeans(n_clusters=10, dimensionality=32)
    with pytest.raises(ValueError, match="dtype float32"):  # :119-123
        km.train(np.zeros((100, 32), dtype=np.float64))
    with pytest.raises(ValueError, match="2-dimensional"):  # :125-133
        km.train(np.zeros(100, dtype=np.float32))
    with pytest.raises(ValueError, match="2-dimensional"):
        km.train(np.zeros((100, 32, 2), dtype=np.float32))
    with pytest.raises(ValueError, match="dimensionality"):  # :135-139
        km.train(np.zeros((100, 64), dtype=np.float32))
    d, k = 256, 10
    km = pkg.SuperKMeans(n_clusters=k, dimensionality=d)
    wide = _data(100, d * 2)
    c = km.train(wide[:, ::2])  # non-contiguous input is accepted, :158-169
    assert c.shape == (k, d)
    with pytest.raises(ValueError, match="dtype float32"):  # :141-156
        km.assign(wide[:, ::2].astype(np.float64), c)
    with pytest.raises(ValueError, match="same dimensionality"):
        km.assign(_data(100, 16), c)


def test_same_seed_gives_identical_centroids(pkg):
    n, d, k = 10000, 512, 100  # :182-197
    data = _data(n, d)
    c1 = pkg.SuperKMeans(n_clusters=k, dimensionality=d, iters=5, seed=123).train(data)
    c2 = pkg.SuperKMeans(n_clusters=k, dimensionality=d, iters=5, seed=123).train(data)
    np.testing.assert_array_equal(c1, c2)
    c3 = pkg.SuperKMeans(n_clusters=k, dimensionality=d, iters=5, seed=7).train(data)
    assert not np.array_equal(c1, c3)


def test_hierarchical_selection_and_stats(pkg, blobs):
    d, k = 128, 400
    small = blobs(20000, d, 100, seed=1)
    km = pkg.SuperKMeans(n_clusters=k, dimensionality=d, hierarchical=True)  # explicit, :199-230
    c = km.train(small)
    assert km.hierarchical_ is True and c.shape == (k, d)
    hs = km.hierarchical_iteration_stats
    assert isinstance(hs, pkg.HierarchicalSuperKMeansIterationStats)
    assert len(hs.mesoclustering_iteration_stats) == 3 and len(hs.refinement_iteration_stats) == 0
    assert len(hs.fineclustering_iteration_stats) > 0
    assert "hierarchical=True" in repr(km)
    flat = pkg.SuperKMeans(n_clusters=k, dimensionality=d)  # automatic: n <= 100,000 -> flat, :232-283
    flat.train(small)
    assert flat.hierarchical_ is False and flat.hierarchical_iteration_stats is None
    big = blobs(100_001, 64, 50, seed=2)
    auto = pkg.SuperKMeans(n_clusters=300, dimensionality=64, iters_fineclustering=2)
    auto.train(big)
    assert auto.hierarchical_ is True


def test_assign_training_points_agrees_with_assign(pkg, blobs):
    n, d, k = 20000, 256, 300  # :392-412 (>= 95 %)
    data = blobs(n, d, k, seed=3)
    km = pkg.SuperKMeans(n_clusters=k, dimensionality=d, iters=5, sampling_fraction=1.0)
    c = km.train(data)
    fast, exact = km.assign_training_points(data, c), km.assign(data, c)
    assert fast.dtype == np.uint32 and fast.shape == (n,)
    assert np.mean(fast == exact) >= 0.95
    from superkmeans_amd import _superkmeans

    with pytest.raises(RuntimeError, match="trained first"):  # superkmeans.h:404-406
        _superkmeans.SuperKMeans(k, d).assign_training_points(data, c)


def test_train_with_queries(pkg):  # python/tests/test_superkmeans.py:49-64 of the reference
    np.random.seed(42)
    n, d, k, q = 10000, 512, 100, 50
    data = np.random.randn(n, d).astype(np.float32)
    queries = np.random.randn(q, d).astype(np.float32)
    km = pkg.SuperKMeans(n_clusters=k, dimensionality=d, iters=5, objective_k=10, verbose=False)
    centroids = km.train(data, queries=queries)
    assert centroids.shape == (k, d) and km.is_trained_ and len(km.iteration_stats) > 0
    assert all(0.0 <= s.recall <= 1.0 for s in km.iteration_stats)
    assert any(s.recall > 0.0 for s in km.iteration_stats)
    with pytest.raises(ValueError, match="dimensionality"):
        pkg.SuperKMeans(n_clusters=k, dimensionality=d).train(data, queries=queries[:, :100].copy())


def test_returned_centroids_prepared_ahead_equal_the_plain_path(pkg, capi):
    """From 16 MiB of host results Train touches the vector it returns (and the assignment and distance buffers) on a
    helper thread while the device works; the C ABI's train writes into the caller's buffer instead and starts no
    such thread for the centroids.  Same seed, same data: the two must return the same bits, the object must
    refuse a second Train, and its destructor must find the thread joined."""
    n, d, k = 9000, 1024, 4200  # 4200 x 1024 floats = 17.2 MB
    data = _data(n, d, seed=9)
    km = pkg.SuperKMeans(n_clusters=k, dimensionality=d, iters=2, sampling_fraction=1.0, seed=5)
    got = km.train(data)
    ck = capi.KMeans(k, d, iters=2, sampling_fraction=1.0, seed=5)
    want = ck.train(data)
    ck.close()
    assert got.shape == (k, d) and np.array_equal(got, want)
    with pytest.raises(RuntimeError, match="already been trained"):
        km.train(data)
    del km
