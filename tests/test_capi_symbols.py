"""The C-ABI libraries load and export every symbol the public headers declare (no GPU needed)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(skm_[a-z0-9_]+)\s*\(", text))


def test_every_declared_symbol_is_exported(capi):
    lib = ctypes.CDLL(capi.LIB_PATH)
    declared = _declared("skm_hip.h") | _declared("skm_kmeans.h")
    assert len(declared) >= 40
    missing = [s for s in sorted(declared) if not hasattr(lib, s)]
    assert not missing, f"declared in include/*.h but not exported: {missing}"


def test_python_prototypes_cover_the_headers(capi):
    declared = _declared("skm_hip.h") | _declared("skm_kmeans.h")
    assert declared == set(capi.exported_symbols())
    capi.load()  # attaches argtypes; raises if a symbol is missing


def test_missing_device_is_reported_not_hidden(capi):
    """Without a GPU the product path must fail loudly: there is no CPU fallback."""
    lib = capi.load()
    if capi.device_count() > 0:
        return
    h = ctypes.c_void_p()
    rc = lib.skm_ctx_create(0, ctypes.byref(h))
    assert rc != 0 and h.value is None
    assert b"device" in lib.skm_last_error().lower()
    try:
        capi.KMeans(10, 16)
    except capi.SkmError as e:
        assert "device" in str(e).lower()
    else:
        raise AssertionError("creating a model without a device must fail")


def test_error_codes_without_compute(capi):
    lib = capi.load()
    assert lib.skm_ctx_create(0, None) == -1  # SKM_ERR_INVALID
    assert lib.skm_sync(None) == -1
    assert lib.skm_norms(None, None, 1, 1, 1, None) == -1
    cfg = capi.KMeansConfig()
    lib.skm_kmeans_default_config(ctypes.byref(cfg), 0)
    assert (cfg.iters, cfg.max_points_per_cluster, cfg.seed, cfg.objective_k) == (10, 256, 42, 100)
    assert abs(cfg.sampling_fraction - 0.3) < 1e-7 and abs(cfg.tol - 1e-4) < 1e-10
    assert cfg.early_termination == 1 and cfg.unrotate_centroids == 1 and cfg.use_blas_only == 0
    assert (cfg.iters_mesoclustering, cfg.iters_fineclustering, cfg.iters_refinement) == (3, 5, 0)
    lib.skm_kmeans_default_config(ctypes.byref(cfg), 1)
    assert cfg.sampling_fraction == 1.0  # hierarchical_superkmeans.h:16


def test_host_dimension_split_equals_oracle(capi, oracle):
    for d in list(range(1, 300)) + [384, 512, 600, 768, 900, 1024, 1536, 2048, 3072, 4096]:
        assert capi.dimension_split(d) == oracle.dimension_split(d), d
