"""ctypes binding of libskm_hip.so (the C ABI declared in include/skm_hip.h).

This is plumbing for tests, the benchmark and the Python facade: every compute call goes to the
HIP library; there is no CPU fallback.  Loading fails loudly when the library has not been built.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_size_t, c_uint32, c_uint64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libskm_hip.so")

_F = c_void_p  # device pointers travel as opaque addresses


class SkmError(RuntimeError):
    pass


_PROTOTYPES = {
    "skm_last_error": (c_char_p, []),
    "skm_device_count": (c_int, [POINTER(c_int)]),
    "skm_ctx_create": (c_int, [c_int, POINTER(c_void_p)]),
    "skm_ctx_destroy": (c_int, [c_void_p]),
    "skm_sync": (c_int, [c_void_p]),
    "skm_ctx_set_workspace_limit": (c_int, [c_void_p, c_size_t]),
    "skm_ctx_set_candidate_kernel": (c_int, [c_void_p, c_int]),
    "skm_ctx_set_walk_kernel": (c_int, [c_void_p, c_int]),
    "skm_ctx_set_walk_launches": (c_int, [c_void_p, c_int]),
    "skm_ctx_get_last_overflow": (c_int, [c_void_p, POINTER(c_uint64)]),
    "skm_malloc": (c_int, [c_void_p, c_size_t, POINTER(c_void_p)]),
    "skm_free": (c_int, [c_void_p, c_void_p]),
    "skm_device_cache_trim": (c_int, [c_int]),
    "skm_device_cache_set_limit": (c_int, [c_int, c_size_t]),
    "skm_upload": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "skm_upload_overlapped": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "skm_upload_detached": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "skm_householder_q": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "skm_download": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "skm_copy": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "skm_fill_u32": (c_int, [c_void_p, c_void_p, c_uint32, c_size_t]),
    "skm_prof_enable": (c_int, [c_void_p, c_int]),
    "skm_prof_reset": (c_int, [c_void_p]),
    "skm_prof_get": (c_int, [c_void_p, c_char_p, POINTER(c_double), POINTER(c_uint64)]),
    "skm_prof_dump": (c_int, [c_void_p, c_char_p, c_size_t, POINTER(c_size_t)]),
    "skm_norms": (c_int, [c_void_p, _F, c_size_t, c_size_t, c_size_t, _F]),
    "skm_rotate": (c_int, [c_void_p, _F, c_size_t, c_size_t, _F, _F]),
    "skm_unrotate": (c_int, [c_void_p, _F, c_size_t, c_size_t, _F, _F]),
    "skm_transpose": (c_int, [c_void_p, _F, c_size_t, c_size_t, _F]),
    "skm_pdxify": (c_int, [c_void_p, _F, c_size_t, c_size_t, c_size_t, _F, _F]),
    "skm_assign_full": (c_int, [c_void_p, _F, c_size_t, _F, c_size_t, c_size_t, _F, _F, _F, _F]),
    "skm_assign_full_noalloc": (c_int, [c_void_p, _F, c_size_t, _F, c_size_t, c_size_t, _F, _F, _F, _F]),
    "skm_assign_pruned": (
        c_int,
        [c_void_p, _F, c_size_t, _F, _F, _F, c_size_t, c_size_t, c_size_t, c_uint32, _F, _F, _F, _F, _F,
         POINTER(c_uint64), POINTER(c_uint64)],
    ),
    "skm_update": (c_int, [c_void_p, _F, c_size_t, c_size_t, _F, c_size_t, _F, _F]),
    "skm_group_by_assignment": (c_int, [c_void_p, _F, c_size_t, c_size_t, _F, _F]),
    "skm_scale_by_size": (c_int, [c_void_p, _F, _F, c_size_t, c_size_t]),
    "skm_scale_by_size_fetch": (c_int, [c_void_p, _F, _F, c_size_t, c_size_t, POINTER(c_uint32)]),
    "skm_normalize_rows": (c_int, [c_void_p, _F, c_size_t, c_size_t]),
    "skm_edit_rows": (c_int, [c_void_p, _F, c_size_t, c_void_p, c_size_t]),
    "skm_wcss": (c_int, [c_void_p, _F, c_size_t, POINTER(c_double)]),
    "skm_wcss_begin": (c_int, [c_void_p, _F, c_size_t]),
    "skm_wcss_end": (c_int, [c_void_p, POINTER(c_double)]),
    "skm_shift": (c_int, [c_void_p, _F, _F, c_size_t, c_size_t, POINTER(c_double)]),
    "skm_gather_rows": (c_int, [c_void_p, _F, c_size_t, _F, c_size_t, _F, _F, _F]),
    "skm_scatter_assignments": (c_int, [c_void_p, _F, _F, c_size_t, c_uint32, _F]),
    "skm_seeds_from_groups": (c_int, [c_void_p, _F, _F, _F, c_size_t, c_size_t]),
    "skm_knn": (c_int, [c_void_p, _F, c_size_t, _F, c_size_t, c_size_t, _F, _F, c_size_t, _F, _F]),
    "skm_recall_hits": (c_int, [c_void_p, _F, _F, _F, c_size_t, c_size_t, c_size_t, c_size_t, c_void_p]),
    "skm_synth_gaussian_mixture": (
        c_int,
        [c_void_p, _F, c_size_t, c_size_t, c_size_t, c_uint32, c_uint32, c_uint32, c_float, c_float, c_float, c_int],
    ),
    "skm_synth_two_level_mixture": (
        c_int, [c_void_p, _F, c_size_t, c_size_t, c_size_t, c_uint32, c_uint32, c_uint32, c_float, c_float]),
    "skm_synth_low_rank": (c_int, [c_void_p, _F, c_size_t, c_size_t, c_size_t, c_uint32, c_uint32, c_float]),
    # include/skm_kmeans.h
    "skm_kmeans_default_config": (None, [c_void_p, c_int]),
    "skm_kmeans_create": (c_int, [c_size_t, c_size_t, c_void_p, c_int, POINTER(c_void_p)]),
    "skm_kmeans_destroy": (c_int, [c_void_p]),
    "skm_kmeans_train": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p]),
    "skm_kmeans_train_device": (c_int, [c_void_p, _F, c_size_t, _F, c_size_t, c_void_p]),
    "skm_kmeans_assign": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_void_p]),
    "skm_kmeans_assign_device": (c_int, [c_void_p, _F, _F, c_size_t, c_size_t, _F]),
    "skm_kmeans_assign_training_points": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_void_p]),
    "skm_kmeans_get_n_clusters": (c_int, [c_void_p, POINTER(c_size_t)]),
    "skm_kmeans_is_trained": (c_int, [c_void_p, POINTER(c_int)]),
    "skm_kmeans_n_stats": (c_int, [c_void_p, c_int, POINTER(c_size_t)]),
    "skm_kmeans_get_stats": (c_int, [c_void_p, c_int, c_void_p, c_size_t]),
    "skm_kmeans_get_assignments": (c_int, [c_void_p, c_void_p, c_size_t]),
    "skm_kmeans_get_training_seeds": (c_int, [c_void_p, c_void_p, c_size_t]),
    "skm_kmeans_get_training_overflow": (c_int, [c_void_p, POINTER(c_uint64)]),
    "skm_kmeans_split_clusters_on_state": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, POINTER(c_uint64)]),
    "skm_kmeans_context": (c_int, [c_void_p, POINTER(c_void_p)]),
    "skm_kmeans_set_prune_accounting": (c_int, [c_void_p, c_int]),
    "skm_kmeans_get_prune_accounting": (
        c_int, [c_void_p, c_size_t, c_void_p, c_size_t, POINTER(c_size_t), POINTER(c_size_t)]),
    "skm_dimension_split": (None, [c_size_t, POINTER(c_size_t), POINTER(c_size_t)]),
    "skm_pruner_tables": (c_int, [c_size_t, c_float, c_uint32, c_int, c_void_p, c_void_p]),
}


class KMeansConfig(ctypes.Structure):
    """skm_kmeans_config (include/skm_kmeans.h)."""

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
        ("dct_rotation", c_int),
    ]


class KMeansIterationStats(ctypes.Structure):
    """skm_kmeans_iteration_stats (include/skm_kmeans.h)."""

    _fields_ = [
        ("iteration", c_uint64),
        ("objective", c_float),
        ("shift", c_float),
        ("split", c_uint64),
        ("recall", c_float),
        ("not_pruned_pct", c_float),
        ("partial_d", c_uint32),
        ("is_gemm_only", c_int),
    ]

_lib = None


def exported_symbols():
    """Names every build of the library must export (mirrors include/skm_hip.h)."""
    return sorted(_PROTOTYPES)


def load():
    """Loads libskm_hip.so and attaches prototypes; raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise SkmError(
            f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C superkmeans_amd/csrc`"
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError here means header and library disagree
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


# Return codes of the C ABI (include/skm_hip.h, include/skm_kmeans.h).
SKM_OK, SKM_ERR_INVALID, SKM_ERR_HIP, SKM_ERR_NO_DEVICE, SKM_ERR_OOM, SKM_ERR_RUNTIME = 0, -1, -2, -3, -4, -5


def check(rc):
    if rc != 0:
        msg = load().skm_last_error()
        raise SkmError(f"libskm_hip error {rc}: {msg.decode() if msg else ''}")


class DeviceArray:
    """A typed device allocation owned by a Context."""

    def __init__(self, ctx, shape, dtype):
        self.ctx = ctx
        self.shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = c_void_p()
        check(ctx.lib.skm_malloc(ctx.handle, self.nbytes, ctypes.byref(p)))
        self.ptr = p.value
        ctx._live.append(self)

    @property
    def size(self):
        return int(np.prod(self.shape, dtype=np.int64))

    def upload(self, host):
        host = np.ascontiguousarray(host, dtype=self.dtype)
        if host.nbytes != self.nbytes:
            raise ValueError(f"upload size mismatch: {host.nbytes} != {self.nbytes}")
        check(self.ctx.lib.skm_upload(self.ctx.handle, self.ptr, host.ctypes.data, self.nbytes))
        return self

    def download(self, count=None):
        shape = self.shape if count is None else (int(count),) + self.shape[1:]
        out = np.empty(shape, dtype=self.dtype)
        check(self.ctx.lib.skm_download(self.ctx.handle, out.ctypes.data, self.ptr, out.nbytes))
        return out

    def offset(self, elements):
        """Device address `elements` items past the start."""
        return self.ptr + int(elements) * self.dtype.itemsize

    def free(self):
        if self.ptr:
            check(self.ctx.lib.skm_free(self.ctx.handle, self.ptr))
            self.ptr = None
            try:
                self.ctx._live.remove(self)
            except ValueError:
                pass


class Context:
    """One device + stream + workspace (skm_ctx)."""

    def __init__(self, device=0):
        self.lib = load()
        h = c_void_p()
        check(self.lib.skm_ctx_create(device, ctypes.byref(h)))
        self.handle = h.value
        self._live = []

    def close(self):
        if self.handle:
            for a in list(self._live):
                a.free()
            check(self.lib.skm_ctx_destroy(self.handle))
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def empty(self, shape, dtype=np.float32):
        return DeviceArray(self, shape, dtype)

    def array(self, host, dtype=None):
        host = np.ascontiguousarray(host, dtype=dtype if dtype is not None else host.dtype)
        return DeviceArray(self, host.shape, host.dtype).upload(host)

    def sync(self):
        check(self.lib.skm_sync(self.handle))

    def prof_enable(self, on=True):
        check(self.lib.skm_prof_enable(self.handle, 1 if on else 0))

    def prof_reset(self):
        check(self.lib.skm_prof_reset(self.handle))

    def prof(self):
        """Returns {scope: (milliseconds, calls)} of the device timers."""
        need = c_size_t()
        check(self.lib.skm_prof_dump(self.handle, None, 0, ctypes.byref(need)))
        buf = ctypes.create_string_buffer(need.value + 1)
        check(self.lib.skm_prof_dump(self.handle, buf, len(buf), ctypes.byref(need)))
        out = {}
        for item in buf.value.decode().split(";"):
            if not item:
                continue
            name, rest = item.split("=")
            ms, calls = rest.split("/")
            out[name] = (float(ms), int(calls))
        return out


class _BorrowedContext(Context):
    """A Context view over an skm_ctx owned by someone else (never destroyed here)."""

    def __init__(self, handle):
        self.lib = load()
        self.handle = handle
        self._live = []

    def close(self):
        for a in list(self._live):
            a.free()
        self.handle = None


class KMeans:
    """skm_kmeans: the C-ABI face of skmeans::SuperKMeans / HierarchicalSuperKMeans (HIP backend)."""

    def __init__(self, n_clusters, d, hierarchical=False, **cfg):
        self.lib = load()
        self.k, self.d, self.hierarchical = int(n_clusters), int(d), bool(hierarchical)
        self.config = KMeansConfig()
        self.lib.skm_kmeans_default_config(ctypes.byref(self.config), 1 if hierarchical else 0)
        for key, val in cfg.items():
            if not hasattr(self.config, key):
                raise AttributeError(key)
            setattr(self.config, key, val)
        h = c_void_p()
        self.handle = None
        check(self.lib.skm_kmeans_create(self.k, self.d, ctypes.byref(self.config), 1 if hierarchical else 0,
                                         ctypes.byref(h)))
        self.handle = h.value
        c = c_void_p()
        check(self.lib.skm_kmeans_context(self.handle, ctypes.byref(c)))
        self.ctx = _BorrowedContext(c.value)

    def close(self):
        if self.handle:
            self.ctx.close()
            check(self.lib.skm_kmeans_destroy(self.handle))
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def train(self, data, queries=None, n_queries=0):
        """`queries`: (n_queries, d) array, or None with n_queries > 0 when the config samples them."""
        data = np.ascontiguousarray(data, dtype=np.float32)
        out = np.empty((self.k, self.d), dtype=np.float32)
        qptr = None
        if queries is not None:
            queries = np.ascontiguousarray(queries, dtype=np.float32)
            qptr, n_queries = queries.ctypes.data, queries.shape[0]
        check(self.lib.skm_kmeans_train(self.handle, data.ctypes.data, data.shape[0], qptr, n_queries,
                                        out.ctypes.data))
        return out

    def train_device(self, d_data, n, d_queries=None, n_queries=0):
        out = np.empty((self.k, self.d), dtype=np.float32)
        ptr = d_data.ptr if isinstance(d_data, DeviceArray) else d_data
        qptr = d_queries.ptr if isinstance(d_queries, DeviceArray) else d_queries
        check(self.lib.skm_kmeans_train_device(self.handle, ptr, n, qptr, n_queries, out.ctypes.data))
        return out

    def assign(self, vectors, centroids):
        vectors = np.ascontiguousarray(vectors, dtype=np.float32)
        centroids = np.ascontiguousarray(centroids, dtype=np.float32)
        out = np.empty(vectors.shape[0], dtype=np.uint32)
        check(self.lib.skm_kmeans_assign(self.handle, vectors.ctypes.data, centroids.ctypes.data, vectors.shape[0],
                                         centroids.shape[0], out.ctypes.data))
        return out

    def assign_device(self, d_vectors, d_centroids, n, k, d_out):
        check(self.lib.skm_kmeans_assign_device(self.handle, d_vectors.ptr, d_centroids.ptr, n, k, d_out.ptr))

    def assign_training_points(self, vectors, centroids):
        vectors = np.ascontiguousarray(vectors, dtype=np.float32)
        centroids = np.ascontiguousarray(centroids, dtype=np.float32)
        out = np.empty(vectors.shape[0], dtype=np.uint32)
        check(self.lib.skm_kmeans_assign_training_points(self.handle, vectors.ctypes.data, centroids.ctypes.data,
                                                         vectors.shape[0], centroids.shape[0], out.ctypes.data))
        return out

    def stats(self, which=0):
        n = c_size_t()
        check(self.lib.skm_kmeans_n_stats(self.handle, which, ctypes.byref(n)))
        arr = (KMeansIterationStats * n.value)()
        if n.value:
            check(self.lib.skm_kmeans_get_stats(self.handle, which, arr, n.value))
        return list(arr)

    def set_prune_accounting(self, on=True):
        check(self.lib.skm_kmeans_set_prune_accounting(self.handle, 1 if on else 0))

    def prune_accounting(self):
        """List (one entry per pruned iteration) of arrays of pairs entering each pruning step."""
        rows, ln = c_size_t(), c_size_t()
        check(self.lib.skm_kmeans_get_prune_accounting(self.handle, 0, None, 0, ctypes.byref(ln), ctypes.byref(rows)))
        out = []
        for it in range(rows.value):
            buf = np.zeros(max(ln.value, 1), dtype=np.uint64)
            check(self.lib.skm_kmeans_get_prune_accounting(self.handle, it, buf.ctypes.data, buf.size,
                                                           ctypes.byref(ln), ctypes.byref(rows)))
            out.append(buf[: ln.value].copy())
        return out

    def assignments(self, count):
        out = np.empty(count, dtype=np.uint32)
        check(self.lib.skm_kmeans_get_assignments(self.handle, out.ctypes.data, count))
        return out

    def split_clusters_on_state(self, centroids, sizes, n_samples):
        """SplitClusters of the object's class on a given state: returns (edited centroids, edited sizes, splits)."""
        c = np.ascontiguousarray(centroids, dtype=np.float32).copy()
        s = np.ascontiguousarray(sizes, dtype=np.uint32).copy()
        n_split = c_uint64()
        check(self.lib.skm_kmeans_split_clusters_on_state(self.handle, c.ctypes.data, s.ctypes.data, c.shape[0], n_samples,
                                                          ctypes.byref(n_split)))
        return c, s, int(n_split.value)

    def training_seeds(self, count):
        out = np.empty(count, dtype=np.uint32)
        check(self.lib.skm_kmeans_get_training_seeds(self.handle, out.ctypes.data, count))
        return out

    def training_overflow(self):
        out = c_uint64()
        check(self.lib.skm_kmeans_get_training_overflow(self.handle, ctypes.byref(out)))
        return int(out.value)

    @property
    def is_trained(self):
        v = c_int()
        check(self.lib.skm_kmeans_is_trained(self.handle, ctypes.byref(v)))
        return bool(v.value)


def dimension_split(d):
    h, v = c_size_t(), c_size_t()
    load().skm_dimension_split(d, ctypes.byref(h), ctypes.byref(v))
    return h.value, v.value


def pruner_tables(d, epsilon0=1.5, seed=42, rotation_kind=0):
    m = np.empty((d, d), dtype=np.float32)
    r = np.empty(d + 1, dtype=np.float32)
    check(load().skm_pruner_tables(d, epsilon0, seed, rotation_kind, m.ctypes.data, r.ctypes.data))
    return m, r


def device_count():
    n = c_int()
    rc = load().skm_device_count(ctypes.byref(n))
    return n.value if rc == 0 else 0
