import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (gfx950) device; run with -m gpu")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (oracle/liboracle.so): the checker, never the thing under test on GPU runs."""
    from oracle import oracle as O

    O.load()
    O.set_threads(0)
    return O


@pytest.fixture(scope="session")
def capi():
    from superkmeans_amd import _capi

    return _capi


@pytest.fixture(scope="session")
def ctx(capi):
    """One device context for the whole GPU session.  Fails (not skips) when the HIP library is missing."""
    capi.load()
    if capi.device_count() == 0:
        pytest.skip("no HIP device visible")
    c = capi.Context(0)
    yield c
    c.close()


def make_blobs(n, d, k, std=0.3, seed=0, normalize=True, center_scale=1.0):
    """Seeded isotropic Gaussian mixture (the shape of the CPU-sized benchmark configuration)."""
    g = np.random.default_rng(seed)
    centers = (center_scale * g.standard_normal((k, d))).astype(np.float32)
    a = g.integers(0, k, n)
    x = centers[a] + std * g.standard_normal((n, d)).astype(np.float32)
    if normalize:
        x /= np.linalg.norm(x, axis=1, keepdims=True)
    return np.ascontiguousarray(x, dtype=np.float32)


@pytest.fixture(scope="session")
def blobs():
    return make_blobs


GOLDEN_WCSS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "wcss_ground_truth.json")


@pytest.fixture(scope="session")
def golden():
    """WCSS tables held by the reference's tests (tests/test_wcss.cpp:25-59, test_hierarchical_superkmeans.cpp:636-670)."""
    import json

    with open(GOLDEN_WCSS) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def golden_data(oracle):
    """The data the tables were made on, regenerated (tests/generate_wcss_ground_truth.cpp:15-31)."""
    return oracle.make_blobs(10000, 768, 500, False, 0.25, 5.0, 42)
