"""Super K-Means for AMD MI355X: Python package.

Drop-in counterpart of the reference's ``superkmeans`` package (python/superkmeans/__init__.py):
the same ``SuperKMeans`` facade (constructor keywords and defaults :80-104, validation messages
:139-158, automatic choice of the hierarchical variant above 100,000 samples :192-195, ``assign`` /
``add`` / ``assign_training_points`` :237-317, read-only properties :319-352, ``__repr__`` :354-361)
over a compiled ``_superkmeans`` module whose classes run on the GPU through libskm_hip.so.
There is no CPU fallback: importing the compiled module fails if it has not been built.
"""
from typing import Optional

import numpy as np

__version__ = "0.1.0"

from ._superkmeans import (  # noqa: E402  (compiled module; `make -C superkmeans_amd/csrc python`)
    HierarchicalSuperKMeans as _HierarchicalModel,
    HierarchicalSuperKMeansConfig as _HierarchicalConfig,
    HierarchicalSuperKMeansIterationStats,
    SuperKMeans as _FlatModel,
    SuperKMeansConfig as _FlatConfig,
    SuperKMeansIterationStats,
)

_AUTO_HIERARCHICAL_ABOVE = 100_000

# keyword -> default, in the order of the reference's constructor
_SHARED_OPTIONS = (
    "max_points_per_cluster",
    "n_threads",
    "seed",
    "use_blas_only",
    "tol",
    "recall_tol",
    "early_termination",
    "sample_queries",
    "objective_k",
    "verbose",
    "angular",
)


class SuperKMeans:
    """A super fast k-means for high-dimensional vectors (GPU backend).

    Parameters
    ----------
    n_clusters, dimensionality : int
        Number of clusters and of dimensions; both must be positive.
    hierarchical : bool or None
        ``None`` (default) picks the hierarchical variant when ``train`` sees more than 100,000 samples.
    iters : int
        Iterations of the flat variant (default 10).
    iters_mesoclustering, iters_fineclustering, iters_refinement : int
        Iterations of the three phases of the hierarchical variant (defaults 3, 5, 0).
    sampling_fraction : float in (0, 1] or None
        ``None`` keeps the variant's default (0.3 flat, 1.0 hierarchical).
    max_points_per_cluster, n_threads, seed, use_blas_only, tol, recall_tol, early_termination,
    sample_queries, objective_k, verbose, angular
        Forwarded to the configuration object; same meaning and defaults as in the reference.
    """

    def __init__(
        self,
        n_clusters: int,
        dimensionality: int,
        hierarchical: Optional[bool] = None,
        iters: int = 10,
        iters_mesoclustering: int = 3,
        iters_fineclustering: int = 5,
        iters_refinement: int = 0,
        sampling_fraction: Optional[float] = None,
        max_points_per_cluster: int = 256,
        n_threads: int = 0,
        seed: int = 42,
        use_blas_only: bool = False,
        tol: float = 1e-4,
        recall_tol: float = 0.005,
        early_termination: bool = True,
        sample_queries: bool = False,
        objective_k: int = 100,
        verbose: bool = False,
        angular: bool = False,
    ):
        if n_clusters <= 0:
            raise ValueError("n_clusters must be positive")
        if dimensionality <= 0:
            raise ValueError("dimensionality must be positive")
        if sampling_fraction is not None and not 0.0 < sampling_fraction <= 1.0:
            raise ValueError("sampling_fraction must be in (0.0, 1.0]")
        self._n_clusters = n_clusters
        self._dimensionality = dimensionality
        self._hierarchical_param = hierarchical
        self._hierarchical = None  # resolved by train()
        self._cpp_skmeans_obj = None
        local = locals()
        self._config_params = {name: local[name] for name in _SHARED_OPTIONS}
        self._config_params.update(
            iters=iters,
            iters_mesoclustering=iters_mesoclustering,
            iters_fineclustering=iters_fineclustering,
            iters_refinement=iters_refinement,
            sampling_fraction=sampling_fraction,
        )

    @staticmethod
    def validate_numpy_array(data, name: str, expected_dimensionality: Optional[int] = None) -> np.ndarray:
        """Checks dtype float32 and rank 2 (and optionally the width); returns a C-contiguous array."""
        if not isinstance(data, np.ndarray):
            data = np.asarray(data, dtype=np.float32)
        if data.dtype != np.float32:
            raise ValueError(f"{name} must have dtype float32, got {data.dtype}")
        if data.ndim != 2:
            raise ValueError(f"{name} must be 2-dimensional, got {data.ndim}")
        if expected_dimensionality is not None and data.shape[1] != expected_dimensionality:
            raise ValueError(f"{name} must have dimensionality {expected_dimensionality}, got {data.shape[1]}")
        return data if data.flags["C_CONTIGUOUS"] else np.ascontiguousarray(data)

    def _build_model(self):
        p = self._config_params
        if self._hierarchical:
            config = _HierarchicalConfig()
            config.iters_mesoclustering = p["iters_mesoclustering"]
            config.iters_fineclustering = p["iters_fineclustering"]
            config.iters_refinement = p["iters_refinement"]
            model_cls = _HierarchicalModel
        else:
            config = _FlatConfig()
            config.iters = p["iters"]
            model_cls = _FlatModel
        if p["sampling_fraction"] is not None:
            config.sampling_fraction = p["sampling_fraction"]
        for name in _SHARED_OPTIONS:
            setattr(config, name, p[name])
        return model_cls(self._n_clusters, self._dimensionality, config)

    def train(self, data, queries=None) -> np.ndarray:
        """Runs k-means on ``data`` (n_samples, dimensionality) float32 and returns the centroids
        (n_clusters, dimensionality).  ``queries`` enables recall tracking where the backend supports it.
        Raises ValueError for wrong dtype / rank / width and RuntimeError when already trained."""
        data = self.validate_numpy_array(data, "data", self._dimensionality)
        if self._hierarchical_param is None:
            self._hierarchical = data.shape[0] > _AUTO_HIERARCHICAL_ABOVE
        else:
            self._hierarchical = self._hierarchical_param
        if self._cpp_skmeans_obj is None:
            self._cpp_skmeans_obj = self._build_model()
        n_queries = 0
        if queries is not None:
            queries = self.validate_numpy_array(queries, "queries", self._dimensionality)
            n_queries = queries.shape[0]
        return self._cpp_skmeans_obj.train(data, queries, n_queries)

    def _checked_pair(self, vectors, centroids):
        vectors = self.validate_numpy_array(vectors, "vectors")
        centroids = self.validate_numpy_array(centroids, "centroids")
        if vectors.shape[1] != centroids.shape[1]:
            raise ValueError(
                f"vectors and centroids must have same dimensionality, got {vectors.shape[1]} and {centroids.shape[1]}"
            )
        return vectors, centroids

    def assign(self, vectors, centroids) -> np.ndarray:
        """Index (uint32) of the nearest centroid of every vector, by exact search; works for any vectors."""
        vectors, centroids = self._checked_pair(vectors, centroids)
        return self._cpp_skmeans_obj.assign(vectors, centroids)

    add = assign  # FAISS-style alias

    def assign_training_points(self, vectors, centroids) -> np.ndarray:
        """Faster assignment of the very points passed to train(), seeded with the training assignments.
        Raises RuntimeError when the model has not been trained."""
        vectors, centroids = self._checked_pair(vectors, centroids)
        return self._cpp_skmeans_obj.assign_training_points(vectors, centroids)

    @property
    def n_clusters_(self) -> int:
        return self._n_clusters if self._cpp_skmeans_obj is None else self._cpp_skmeans_obj.get_n_clusters()

    @property
    def is_trained_(self) -> bool:
        return False if self._cpp_skmeans_obj is None else self._cpp_skmeans_obj.is_trained()

    @property
    def hierarchical_(self) -> Optional[bool]:
        return self._hierarchical

    @property
    def iteration_stats(self):
        return [] if self._cpp_skmeans_obj is None else self._cpp_skmeans_obj.iteration_stats

    @property
    def hierarchical_iteration_stats(self):
        if self._cpp_skmeans_obj is None or not self._hierarchical:
            return None
        return getattr(self._cpp_skmeans_obj, "hierarchical_iteration_stats", None)

    def __repr__(self) -> str:
        hier = f", hierarchical={self._hierarchical}" if self._hierarchical is not None else ""
        return (
            f"SuperKMeans(n_clusters={self._n_clusters}, dimensionality={self._dimensionality}, "
            f"trained={self.is_trained_}{hier})"
        )


__all__ = [
    "__version__",
    "SuperKMeans",
    "SuperKMeansIterationStats",
    "HierarchicalSuperKMeansIterationStats",
]
