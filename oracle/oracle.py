"""ctypes wrapper of oracle/liboracle.so -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

The oracle is a CPU restatement of the reference's assign/update path (see skm_oracle.cpp).  Only
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module.
"""
import ctypes
import os
import subprocess
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_size_t, c_uint32, c_uint64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")


class Config(ctypes.Structure):
    """C layout of SuperKMeansConfig + HierarchicalSuperKMeansConfig (superkmeans.h:23-55,
    hierarchical_superkmeans.h:11-17)."""

    _fields_ = [
        ("iters", c_uint32),
        ("sampling_fraction", c_float),
        ("max_points_per_cluster", c_uint32),
        ("n_threads", c_uint32),
        ("seed", c_uint32),
        ("use_blas_only", c_int),
        ("tol", c_float),
        ("recall_tol", c_float),
        ("early_termination", c_int),
        ("sample_queries", c_int),
        ("objective_k", c_uint64),
        ("ann_explore_fraction", c_float),
        ("min_not_pruned_pct", c_float),
        ("max_not_pruned_pct", c_float),
        ("adjustment_factor_for_partial_d", c_float),
        ("unrotate_centroids", c_int),
        ("verbose", c_int),
        ("angular", c_int),
        ("suppress_warnings", c_int),
        ("data_already_rotated", c_int),
        ("iters_mesoclustering", c_uint32),
        ("iters_fineclustering", c_uint32),
        ("iters_refinement", c_uint32),
        ("dct_rotation", ctypes.c_int32),
    ]


class IterationStats(ctypes.Structure):
    _fields_ = [
        ("iteration", c_uint64),
        ("objective", c_float),
        ("shift", c_float),
        ("split", c_uint64),
        ("recall", c_float),
        ("not_pruned_pct", c_float),
        ("partial_d", c_uint32),
        ("is_gemm_only", c_int),
        ("objective_f64", c_double),
    ]


_lib = None


def build():
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def _fp(a):
    return a.ctypes.data_as(c_void_p)


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        build()
    lib = ctypes.CDLL(LIB_PATH)
    lib.oracle_last_error.restype = c_char_p
    lib.oracle_blas_name.restype = c_char_p
    lib.oracle_tune_partial_d.restype = c_float
    lib.oracle_horizontal.restype = c_float
    lib.oracle_kmeans_n_stats.restype = c_size_t
    lib.oracle_kmeans_n_samples.restype = c_size_t
    lib.oracle_kmeans_last_seeds.restype = c_size_t
    lib.oracle_kmeans_accounting.restype = c_size_t
    lib.oracle_split_clusters.restype = c_size_t
    lib.oracle_n_mesoclusters.restype = c_size_t
    lib.oracle_get_threads.restype = c_uint32
    _lib = lib
    bind_blas()
    return lib


def bind_blas():
    """Binds sgemm_ from the first BLAS found (the reference links one at build time, common.h:7-23)."""
    lib = _lib
    candidates = []
    env = os.environ.get("SKM_ORACLE_BLAS")
    if env:
        candidates.append(env)
    candidates += ["/opt/conda/lib/libmkl_rt.so", "libmkl_rt.so", "libopenblas.so", "libopenblas.so.0", "libblas.so.3"]
    try:
        import importlib.util

        spec = importlib.util.find_spec("torch")
        if spec and spec.origin:
            candidates.append(os.path.join(os.path.dirname(spec.origin), "lib", "libtorch_cpu.so"))
    except Exception:
        pass
    arr = (c_char_p * len(candidates))(*[c.encode() for c in candidates])
    lib.oracle_bind_blas(arr, len(candidates))
    return lib.oracle_blas_name().decode()


def blas_name():
    return load().oracle_blas_name().decode()


def set_threads(n):
    load().oracle_set_threads(c_uint32(n))


def get_threads():
    return load().oracle_get_threads()


def max_threads():
    return load().oracle_max_threads()


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def dimension_split(d):
    h, v = c_size_t(), c_size_t()
    load().oracle_dimension_split(c_size_t(d), ctypes.byref(h), ctypes.byref(v))
    return h.value, v.value


def pdxify(c):
    c = f32(c)
    out = np.empty_like(c)
    load().oracle_pdxify(_fp(c), _fp(out), c_size_t(c.shape[0]), c_size_t(c.shape[1]))
    return out.reshape(-1)


def ratios(d, epsilon0=1.5):
    out = np.empty(d + 1, dtype=np.float32)
    load().oracle_ratios(c_uint32(d), c_float(epsilon0), _fp(out))
    return out


def rotation_matrix(d, seed=42):
    out = np.empty((d, d), dtype=np.float32)
    load().oracle_rotation_matrix(c_uint32(d), c_uint32(seed), _fp(out))
    return out


def rotate(q, x):
    q, x = f32(q), f32(x)
    out = np.empty_like(x)
    load().oracle_rotate(_fp(q), c_uint32(q.shape[0]), _fp(x), c_uint32(x.shape[0]), _fp(out))
    return out


def unrotate(q, x):
    q, x = f32(q), f32(x)
    out = np.empty_like(x)
    load().oracle_unrotate(_fp(q), c_uint32(q.shape[0]), _fp(x), c_uint32(x.shape[0]), _fp(out))
    return out


def norms(x, cols=None):
    x = f32(x)
    n, d = x.shape
    out = np.empty(n, dtype=np.float32)
    load().oracle_norms(_fp(x), c_size_t(n), c_size_t(d), c_size_t(d if cols is None else cols), _fp(out))
    return out


def find_nn(x, y, norms_x=None, norms_y=None):
    x, y = f32(x), f32(y)
    nx = norms(x) if norms_x is None else f32(norms_x)
    ny = norms(y) if norms_y is None else f32(norms_y)
    knn = np.zeros(x.shape[0], dtype=np.uint32)
    dist = np.empty(x.shape[0], dtype=np.float32)
    load().oracle_find_nn(_fp(x), _fp(y), c_size_t(x.shape[0]), c_size_t(y.shape[0]), c_size_t(x.shape[1]), _fp(nx),
                          _fp(ny), _fp(knn), _fp(dist))
    return knn, dist


def rotate_kind(x, seed=42, rotation_kind=1, forward=True, want_matrix=False):
    """Rotate / Unrotate of the pruner built for `rotation_kind` (1, 2: DCT variants of pdx/adsampling.h:52-74).
    Returns (out, uses_dct[, matrix])."""
    x = f32(x)
    n, d = x.shape
    out = np.empty_like(x)
    m = np.empty((d, d), dtype=np.float32) if want_matrix else None
    used = load().oracle_rotate_kind(c_uint32(d), c_uint32(seed), c_int(rotation_kind), c_int(1 if forward else 0),
                                     _fp(x), c_uint32(n), _fp(out), _fp(m) if want_matrix else None)
    return (out, bool(used), m) if want_matrix else (out, bool(used))


def find_knn(x, y, k, norms_x=None, norms_y=None):
    """FindKNearestNeighbors (batch_computers.h:191-274): (indices, distances), each (n_x, k)."""
    x, y = f32(x), f32(y)
    nx = norms(x) if norms_x is None else f32(norms_x)
    ny = norms(y) if norms_y is None else f32(norms_y)
    knn = np.zeros((x.shape[0], k), dtype=np.uint32)
    dist = np.empty((x.shape[0], k), dtype=np.float32)
    lib = load()
    lib.oracle_find_knn(_fp(x), _fp(y), c_size_t(x.shape[0]), c_size_t(y.shape[0]), c_size_t(x.shape[1]), _fp(nx),
                        _fp(ny), c_size_t(k), _fp(knn), _fp(dist))
    return knn, dist


def recall_from_lists(gt, promising, assignments):
    """Recall loop of ComputeRecall (superkmeans.h:1059-1086) on (n_q, objective_k) / (n_q, explore) lists."""
    gt = np.ascontiguousarray(gt, dtype=np.uint32)
    promising = np.ascontiguousarray(promising, dtype=np.uint32)
    assignments = np.ascontiguousarray(assignments, dtype=np.uint32)
    lib = load()
    lib.oracle_recall_from_lists.restype = ctypes.c_float
    return float(lib.oracle_recall_from_lists(_fp(gt), _fp(promising), _fp(assignments), c_size_t(gt.shape[0]),
                                              c_size_t(gt.shape[1]), c_size_t(promising.shape[1])))


def find_nn_pruned(x, y, prev_assign, partial_d, ratio_table, accounting=False):
    """FindNearestNeighborWithPruning on rotated x and centroids y; returns (assign, dist, counts[, stage_pairs])."""
    x, y = f32(x), f32(y)
    n, d = x.shape
    k = y.shape[0]
    _, v = dimension_split(d)
    pdx = pdxify(y)
    aux = np.ascontiguousarray(y[:, :v])
    nxp, nyp = norms(x, partial_d), norms(y, partial_d)
    knn = np.ascontiguousarray(prev_assign, dtype=np.uint32).copy()
    dist = np.zeros(n, dtype=np.float32)
    counts = np.zeros(n, dtype=np.uint64)
    ratio_table = f32(ratio_table)
    h = d - v
    stages = np.zeros(h // 64 + 2, dtype=np.uint64)
    load().oracle_find_nn_pruned(_fp(x), _fp(y), c_size_t(n), c_size_t(k), c_size_t(d), _fp(nxp), _fp(nyp), _fp(knn),
                                 _fp(dist), _fp(pdx), _fp(aux), c_uint32(partial_d), _fp(ratio_table), _fp(counts),
                                 _fp(stages) if accounting else None)
    if accounting:
        return knn, dist, counts, stages
    return knn, dist, counts


def brute_force(x, y):
    """fp64 exact nearest neighbour: (index, best distance, second-best distance)."""
    x, y = f32(x), f32(y)
    knn = np.empty(x.shape[0], dtype=np.uint32)
    best = np.empty(x.shape[0], dtype=np.float64)
    second = np.empty(x.shape[0], dtype=np.float64)
    load().oracle_brute_force(_fp(x), _fp(y), c_size_t(x.shape[0]), c_size_t(y.shape[0]), c_size_t(x.shape[1]), _fp(knn),
                              _fp(best), _fp(second))
    return knn, best, second


def update_centroids(x, assign, k, scale=False, n_threads=0):
    x = f32(x)
    n, d = x.shape
    assign = np.ascontiguousarray(assign, dtype=np.uint32)
    sums = np.empty((k, d), dtype=np.float32)
    sizes = np.empty(k, dtype=np.uint32)
    load().oracle_update_centroids(_fp(x), c_size_t(n), c_size_t(d), _fp(assign), c_size_t(k), _fp(sums), _fp(sizes),
                                   c_int(1 if scale else 0), c_uint32(n_threads))
    return sums, sizes


def split_clusters(centroids, sizes, n_samples, seed=42, hierarchical=False):
    c = f32(centroids).copy()
    s = np.ascontiguousarray(sizes, dtype=np.uint32).copy()
    n_split = load().oracle_split_clusters(_fp(c), _fp(s), c_size_t(c.shape[0]), c_size_t(c.shape[1]),
                                           c_size_t(n_samples), c_uint32(seed), c_int(1 if hierarchical else 0))
    return c, s, n_split


def tune_partial_d(counts, k, partial_d, vertical_d, min_pct=0.03, max_pct=0.05, adj=0.20):
    counts = np.ascontiguousarray(counts, dtype=np.uint64)
    out = c_uint32()
    avg = load().oracle_tune_partial_d(_fp(counts), c_size_t(counts.shape[0]), c_size_t(k), c_uint32(partial_d),
                                       c_uint32(vertical_d), c_float(min_pct), c_float(max_pct), c_float(adj),
                                       ctypes.byref(out))
    return avg, out.value


def arrange_fine_clusters(n_clusters, n_samples, sizes):
    sizes = np.ascontiguousarray(sizes, dtype=np.uint32)
    out = np.empty(sizes.shape[0], dtype=np.uint64)
    load().oracle_arrange_fine_clusters(c_size_t(n_clusters), c_size_t(sizes.shape[0]), c_size_t(n_samples), _fp(sizes),
                                        _fp(out))
    return out


def make_blobs(n_samples, n_features, n_centers, normalize=False, cluster_std=1.0, center_spread=10.0, random_state=42):
    """MakeBlobs (pdx/utils.h:74-123) with one thread."""
    out = np.empty((n_samples, n_features), dtype=np.float32)
    load().oracle_make_blobs(c_size_t(n_samples), c_size_t(n_features), c_size_t(n_centers), c_int(1 if normalize else 0),
                             c_float(cluster_std), c_float(center_spread), c_uint32(random_state), _fp(out))
    return out


def n_mesoclusters(k):
    return load().oracle_n_mesoclusters(c_size_t(k))


def default_config(hierarchical=False, **overrides):
    cfg = Config()
    load().oracle_default_config(ctypes.byref(cfg), c_int(1 if hierarchical else 0))
    for key, val in overrides.items():
        if not hasattr(cfg, key):
            raise AttributeError(key)
        setattr(cfg, key, val)
    return cfg


class OracleError(Exception):
    def __init__(self, kind, msg):
        super().__init__(msg)
        self.kind = kind  # 1 invalid_argument, 2 runtime_error


class KMeans:
    """Oracle counterpart of skmeans::SuperKMeans / HierarchicalSuperKMeans."""

    def __init__(self, n_clusters, d, hierarchical=False, **cfg):
        self.lib = load()
        self.k, self.d, self.hierarchical = n_clusters, d, hierarchical
        self.config = default_config(hierarchical, **cfg)
        h = c_void_p()
        self._check(self.lib.oracle_kmeans_create(c_size_t(n_clusters), c_size_t(d), ctypes.byref(self.config),
                                                  c_int(1 if hierarchical else 0), ctypes.byref(h)))
        self.h = h

    def _check(self, rc):
        if rc != 0:
            raise OracleError(self.lib.oracle_error_kind(), self.lib.oracle_last_error().decode())

    def __del__(self):
        if getattr(self, "h", None):
            self.lib.oracle_kmeans_destroy(self.h)
            self.h = None

    def train(self, data, queries=None):
        data = f32(data)
        out = np.empty((self.k, self.d), dtype=np.float32)
        nq = 0 if queries is None else queries.shape[0]
        q = None if queries is None else _fp(f32(queries))
        self._check(self.lib.oracle_kmeans_train(self.h, _fp(data), c_size_t(data.shape[0]), q, c_size_t(nq), _fp(out)))
        return out

    def train_sampled_queries(self, data, n_queries):
        """Train with n_queries queries drawn from the data (config sample_queries=1, no query pointer)."""
        data = f32(data)
        out = np.empty((self.k, self.d), dtype=np.float32)
        self._check(self.lib.oracle_kmeans_train(self.h, _fp(data), c_size_t(data.shape[0]), None,
                                                 c_size_t(n_queries), _fp(out)))
        return out

    def assign(self, vectors, centroids):
        vectors, centroids = f32(vectors), f32(centroids)
        out = np.empty(vectors.shape[0], dtype=np.uint32)
        self._check(self.lib.oracle_kmeans_assign(self.h, _fp(vectors), _fp(centroids), c_size_t(vectors.shape[0]),
                                                  c_size_t(centroids.shape[0]), _fp(out)))
        return out

    def assign_training_points(self, vectors, centroids):
        vectors, centroids = f32(vectors), f32(centroids)
        out = np.empty(vectors.shape[0], dtype=np.uint32)
        self._check(self.lib.oracle_kmeans_assign_training_points(
            self.h, _fp(vectors), _fp(centroids), c_size_t(vectors.shape[0]), c_size_t(centroids.shape[0]), _fp(out)))
        return out

    def stats(self, which=0):
        n = self.lib.oracle_kmeans_n_stats(self.h, c_int(which))
        arr = (IterationStats * n)()
        if n:
            self.lib.oracle_kmeans_get_stats(self.h, c_int(which), arr)
        return list(arr)

    def state(self):
        ns = self.lib.oracle_kmeans_n_samples(self.h)
        c = np.empty((self.k, self.d), dtype=np.float32)
        a = np.empty(ns, dtype=np.uint32)
        dist = np.empty(ns, dtype=np.float32)
        sizes = np.empty(self.k, dtype=np.uint32)
        self.lib.oracle_kmeans_state(self.h, _fp(c), _fp(a), _fp(dist), _fp(sizes))
        return c, a, dist, sizes

    def training_seeds(self):
        """Seeds of the last assign_training_points (test hook of the restatement)."""
        n = self.lib.oracle_kmeans_last_seeds(self.h, None, c_size_t(0))
        out = np.empty(n, dtype=np.uint32)
        self.lib.oracle_kmeans_last_seeds(self.h, _fp(out), c_size_t(n))
        return out

    def collect_accounting(self, on=True):
        self.lib.oracle_kmeans_collect_accounting(self.h, c_int(1 if on else 0))

    def accounting(self):
        buf = np.zeros(128, dtype=np.uint64)
        n = self.lib.oracle_kmeans_accounting(self.h, _fp(buf), c_size_t(128))
        return buf[:n]

    @property
    def is_trained(self):
        return bool(self.lib.oracle_kmeans_is_trained(self.h))
