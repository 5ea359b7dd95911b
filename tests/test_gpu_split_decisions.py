"""SplitClusters decisions of the host classes against the oracle's restatement, state by state.

Both variants decide on the host from the cluster sizes and one mt19937(seed) stream: which empty cluster is re-seeded
from which donor (superkmeans.h:890-928), and in the hierarchical class which small cluster is pulled towards which
large one with which weight (hierarchical_superkmeans.h:579-678: threshold a quarter of the average size, weight
min(size, 7), acceptance by excess over the average).  skm_kmeans_split_clusters_on_state runs the object's own
SplitClusters on a given state; the edited rows and sizes must equal the oracle's bit for bit, which holds only if
every decision (donor, order, weight) and every draw was the same."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _state(k, d, seed, empty_fraction, small_fraction):
    g = np.random.default_rng(seed)
    C = g.standard_normal((k, d)).astype(np.float32)
    sizes = (g.pareto(1.5, k) * 40).astype(np.uint32) + 1
    order = g.permutation(k)
    n_empty, n_small = int(round(empty_fraction * k)), int(round(small_fraction * k))
    sizes[order[:n_empty]] = 0
    sizes[order[n_empty:n_empty + n_small]] = g.integers(1, 4, n_small)
    return C, sizes


@pytest.mark.parametrize("hierarchical", [False, True])
@pytest.mark.parametrize("k,d,empty,small", [(50, 64, 0.1, 0.1), (500, 96, 0.05, 0.2), (1200, 32, 0.02, 0.05),
                                             (300, 128, 0.0, 0.3), (64, 20, 0.5, 0.0)])
def test_split_decisions_and_rows_equal_the_oracle(capi, ctx, oracle, hierarchical, k, d, empty, small):
    C, sizes = _state(k, d, seed=k + d, empty_fraction=empty, small_fraction=small)
    n = int(sizes.sum())
    for seed in (42, 7):
        km = capi.KMeans(k, d, hierarchical=hierarchical, seed=seed, suppress_warnings=1)
        gc, gs, gn = km.split_clusters_on_state(C, sizes, n)
        oc, os_, on = oracle.split_clusters(C, sizes, n, seed=seed, hierarchical=hierarchical)
        km.close()
        assert gn == on
        assert np.array_equal(gs, os_)
        assert np.array_equal(gc, oc)
        if empty > 0 or (hierarchical and small > 0):
            assert gn > 0 and not np.array_equal(gc, C)  # the state did call for edits
        assert int(gs.sum()) == n


def test_split_on_state_needs_an_untrained_object(capi, ctx, blobs):
    X = blobs(3000, 64, 30, seed=1)
    km = capi.KMeans(30, 64, iters=2)
    km.train(X)
    with pytest.raises(capi.SkmError, match="untrained"):
        km.split_clusters_on_state(X[:30], np.full(30, 100, dtype=np.uint32), 3000)
    km.close()
