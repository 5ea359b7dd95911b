"""Benchmark-harness compatibility with the reference's `benchmarks/` tree.

Readers for its dataset files, its recall evaluation and its results CSV, so that a run of this
backend drops a row next to the reference's rows and its plotting scripts pick it up unchanged:

* `read_bin`: `data_<dataset>.bin` / `data_<dataset>_test.bin` are raw little-endian float32,
  row-major, no header (reference `benchmarks/end_to_end/end_to_end_superkmeans.cpp:62-75`);
* `load_ground_truth`: `ground_truth/<dataset>.json`, `{"<query index>": [vector ids ...]}`
  (`benchmarks/bench_utils.h:140-190`);
* `compute_recall`: for each exploration fraction, the share of a query's first `knn` ground-truth
  vectors whose cluster is among the query's nearest centroids, plus the vectors such a probe visits
  (`benchmarks/bench_utils.h:209-347`);
* `write_results_to_csv`: the column set and number formats of `benchmarks/bench_utils.h:408-524`;
* `run_end_to_end`: the flow of `benchmarks/end_to_end/end_to_end_superkmeans.cpp`; the clock runs
  around `Train()` on host-resident data, as there (:92-96), so it includes the upload.

Run as `python -m superkmeans_amd.bench_compat <dataset> [experiment] --data-dir DIR --gt-dir DIR
--results-dir DIR`, or with `--synthetic N D` when the dataset files are not at hand.
"""
import argparse
import csv
import json
import math
import os
import time
from datetime import datetime

import numpy as np

# (vectors, dimensions) of the reference's datasets (benchmarks/bench_utils.h:77-94)
DATASET_PARAMS = {
    "fmnist": (60000, 784), "yi": (187843, 128), "llama": (256921, 128), "sift": (1000000, 128),
    "yahoo": (677305, 384), "yandex": (1000000, 200), "glove200": (1183514, 200), "clip": (1281167, 512),
    "mxbai": (769382, 1024), "wiki": (260372, 3072), "contriever": (990000, 768), "gist": (1000000, 960),
    "openai": (999000, 1536), "arxiv": (2253000, 768), "cohere": (10000000, 1024), "cohere50m": (50000000, 1024),
}
ANGULAR_DATASETS = ("yandex", "glove200", "glove100", "glove50", "llama")
EXPLORE_FRACTIONS = (0.001, 0.002, 0.003, 0.004, 0.005, 0.006, 0.007, 0.008, 0.009, 0.0100, 0.0125, 0.0150, 0.0175,
                     0.0200, 0.0225, 0.0250, 0.0275, 0.0300, 0.0325, 0.0350, 0.0375, 0.0400, 0.0425, 0.0450, 0.0475,
                     0.0500, 0.1)
KNN_VALUES = (10, 100)
MAX_ITERS = 10
N_QUERIES = 1000


def get_default_n_clusters(n):
    """4 * sqrt(n), at least 1 (benchmarks/bench_utils.h:21-23)."""
    return max(1, int(math.sqrt(float(n)) * 4.0))


def read_bin(path, n, d):
    """First n rows of a raw float32 file, memory-mapped; raises if the file is shorter."""
    need = int(n) * int(d) * 4
    have = os.path.getsize(path)
    if have < need:
        raise ValueError(f"{path}: {have} bytes, expected at least {need} for {n} x {d} float32")
    return np.memmap(path, dtype="<f4", mode="r", shape=(int(n), int(d)))


def load_ground_truth(path):
    """{query index (int): [vector ids]}; empty when the file does not exist, like the reference's parser."""
    if not os.path.exists(path):
        return {}
    with open(path, "r") as f:
        raw = json.load(f)
    return {int(key): [int(v) for v in ids] for key, ids in raw.items()}


def compute_recall(gt_map, assignments, queries, centroids, knn):
    """List of (centroids_to_explore, explore_fraction, recall_mean, recall_std, avg_vectors_to_visit).

    Mean over all n_queries (queries without ground truth contribute zero, as in the reference), sample
    standard deviation over the queries that have ground truth.  fp32 distances ||q||^2 + ||c||^2 - 2 q.c,
    ties broken by the lower centroid index.
    """
    assignments = np.asarray(assignments)
    queries = np.ascontiguousarray(queries, dtype=np.float32)
    centroids = np.ascontiguousarray(centroids, dtype=np.float32)
    n_queries, n_clusters = queries.shape[0], centroids.shape[0]
    cluster_sizes = np.bincount(assignments.astype(np.int64), minlength=n_clusters)
    qn = np.einsum("ij,ij->i", queries, queries, dtype=np.float32)
    cn = np.einsum("ij,ij->i", centroids, centroids, dtype=np.float32)
    dist = (qn[:, None] + cn[None, :]) - np.float32(2.0) * (queries @ centroids.T)
    order = np.argsort(dist, axis=1, kind="stable")
    results = []
    for frac in EXPLORE_FRACTIONS:
        explore = max(1, int(n_clusters * np.float32(frac)))
        recalls, visited = [], 0
        for q in range(n_queries):
            ids = gt_map.get(q)
            if ids is None:
                continue
            top = order[q, :explore]
            visited += int(cluster_sizes[top].sum())
            gt_ids = ids[:knn]
            probe = set(top.tolist())
            found = sum(1 for v in gt_ids if int(assignments[v]) in probe)
            recalls.append(np.float32(found) / np.float32(len(gt_ids)))
        mean = float(np.sum(np.asarray(recalls, dtype=np.float32)) / np.float32(n_queries)) if n_queries else 0.0
        if len(recalls) > 1:
            dev = np.asarray(recalls, dtype=np.float32) - np.float32(mean)
            std = float(np.sqrt(np.sum(dev * dev) / np.float32(len(recalls) - 1)))
        else:
            std = 0.0
        results.append((explore, float(frac), mean, std, float(visited) / float(n_queries) if n_queries else 0.0))
    return results


def print_recall_results(results, knn):
    print(f"\n--- Recall@{knn} ---")
    for explore, frac, recall, std, vectors in results:
        print(f"Recall@{explore:4d} ({frac * 100:5.2f}% centroids, {vectors:8.0f} avg vectors): {recall:.4f} ± {std:.4f}")


def cluster_balance_stats(assignments, n_clusters):
    """mean, geometric mean (over non-empty clusters), stdev, coefficient of variation, min, max of the sizes."""
    sizes = np.bincount(np.asarray(assignments).astype(np.int64), minlength=n_clusters).astype(np.float64)
    mean = float(sizes.mean())
    stdev = float(sizes.std())
    positive = sizes[sizes > 0]
    gmean = float(np.exp(np.log(positive).mean())) if positive.size else 0.0
    return {"mean": mean, "geometric_mean": gmean, "stdev": stdev, "cv": stdev / mean if mean > 0 else 0.0,
            "min": int(sizes.min()), "max": int(sizes.max())}


def csv_header(has_recall_data):
    cols = ["timestamp", "algorithm", "dataset", "n_iters", "actual_iterations", "dimensionality", "data_size",
            "n_clusters", "construction_time_ms", "threads", "final_objective"]
    if has_recall_data:
        for knn in KNN_VALUES:
            for frac in EXPLORE_FRACTIONS:
                pct = f"{np.float32(frac) * np.float32(100.0):.2f}"
                cols += [f"recall@{knn}@{pct}", f"recall_std@{knn}@{pct}", f"centroids_explored@{knn}@{pct}",
                         f"vectors_explored@{knn}@{pct}"]
    return cols + ["balance_stats", "config"]


def write_results_to_csv(results_dir, experiment_name, algorithm, dataset, n_iters, actual_iterations, dimensionality,
                         data_size, n_clusters, construction_time_ms, threads, final_objective, config,
                         results_knn_10, results_knn_100, balance_stats=None):
    """Appends one row to <results_dir>/<SKM_ARCH or 'default'>/<experiment_name>.csv; returns the path."""
    arch = os.environ.get("SKM_ARCH", "default")
    out_dir = os.path.join(results_dir, arch)
    os.makedirs(out_dir, exist_ok=True)
    path = os.path.join(out_dir, f"{experiment_name}.csv")
    has_recall = bool(results_knn_10) or bool(results_knn_100)
    row = [datetime.now().strftime("%Y-%m-%d %H:%M:%S"), algorithm, dataset, n_iters, actual_iterations, dimensionality,
           data_size, n_clusters, f"{construction_time_ms:.2f}", threads, f"{final_objective:.6f}"]
    if has_recall:
        for results in (results_knn_10, results_knn_100):
            for explore, _, recall, std, vectors in results:
                row += [f"{recall:.6f}", f"{std:.6f}", str(explore), f"{vectors:.2f}"]
    row.append(json.dumps(balance_stats, separators=(",", ":")) if balance_stats else "")
    row.append(json.dumps(config, separators=(",", ":")))
    new_file = not os.path.exists(path)
    with open(path, "a", newline="") as f:
        writer = csv.writer(f)
        if new_file:
            writer.writerow(csv_header(has_recall))
        writer.writerow(row)
    print(f"Results written to: {path}")
    return path


def _synthetic(n, d, n_queries, seed=7):
    """Clustered stand-in data for machines without the dataset files; ground truth by exact search."""
    rng = np.random.default_rng(seed)
    centers = rng.standard_normal((max(16, int(math.sqrt(n))), d)).astype(np.float32)
    data = centers[rng.integers(0, centers.shape[0], n)] + 0.3 * rng.standard_normal((n, d)).astype(np.float32)
    queries = centers[rng.integers(0, centers.shape[0], n_queries)] + 0.3 * rng.standard_normal((n_queries, d)).astype(np.float32)
    dn = np.einsum("ij,ij->i", data, data)
    gt = {}
    for q0 in range(0, n_queries, 256):
        blk = queries[q0:q0 + 256]
        dist = dn[None, :] - 2.0 * (blk @ data.T)
        top = np.argsort(dist, axis=1, kind="stable")[:, :100]
        for i in range(blk.shape[0]):
            gt[q0 + i] = top[i].tolist()
    return data.astype(np.float32), queries.astype(np.float32), gt


def run_end_to_end(dataset, experiment_name="end_to_end", data_dir=None, gt_dir=None, results_dir="results",
                   synthetic=None, n_iters=MAX_ITERS, sampling_fraction=1.0, n_clusters=None):
    """The reference's end-to-end experiment on this backend; returns the dict of what was written."""
    from . import _capi

    if synthetic is not None:
        n, d = synthetic
        data, queries, gt_map = _synthetic(n, d, min(N_QUERIES, max(1, n // 10)))
    else:
        if dataset not in DATASET_PARAMS:
            raise ValueError(f"Unknown dataset '{dataset}'; known: {', '.join(sorted(DATASET_PARAMS))}")
        n, d = DATASET_PARAMS[dataset]
        data = np.ascontiguousarray(read_bin(os.path.join(data_dir, f"data_{dataset}.bin"), n, d))
        qpath = os.path.join(data_dir, f"data_{dataset}_test.bin")
        queries = np.ascontiguousarray(read_bin(qpath, N_QUERIES, d)) if os.path.exists(qpath) else None
        gt_map = load_ground_truth(os.path.join(gt_dir, f"{dataset}.json")) if gt_dir else {}
    k = int(n_clusters) if n_clusters else get_default_n_clusters(n)
    cfg = dict(iters=int(n_iters), verbose=0, n_threads=0, objective_k=100, ann_explore_fraction=0.01,
               unrotate_centroids=1, early_termination=0, sampling_fraction=float(sampling_fraction), use_blas_only=0,
               angular=1 if dataset in ANGULAR_DATASETS else 0)
    print(f"=== Running algorithm: superkmeans_amd ===\nDataset: {dataset} (n={n}, d={d})")
    print(f"n_clusters={k} n_iters={n_iters} sampling_fraction={sampling_fraction}")
    km = _capi.KMeans(k, d, **cfg)
    t0 = time.perf_counter()
    centroids = km.train(data)
    construction_ms = (time.perf_counter() - t0) * 1e3
    stats = km.stats()
    print(f"\nTraining completed in {construction_ms:.2f} ms\nActual iterations: {len(stats)} (requested: {n_iters})")
    print(f"Final objective: {stats[-1].objective}")
    results10, results100, balance = [], [], None
    if queries is not None and gt_map:
        assignments = km.assign_training_points(data, centroids)
        balance = cluster_balance_stats(assignments, k)
        results10 = compute_recall(gt_map, assignments, queries, centroids, 10)
        print_recall_results(results10, 10)
        results100 = compute_recall(gt_map, assignments, queries, centroids, 100)
        print_recall_results(results100, 100)
    c = km.config
    config = {"iters": c.iters, "sampling_fraction": round(float(c.sampling_fraction), 6), "n_threads": c.n_threads,
              "seed": c.seed, "use_blas_only": bool(c.use_blas_only), "tol": round(float(c.tol), 6),
              "recall_tol": round(float(c.recall_tol), 6), "early_termination": bool(c.early_termination),
              "sample_queries": bool(c.sample_queries), "objective_k": int(c.objective_k),
              "ann_explore_fraction": round(float(c.ann_explore_fraction), 6),
              "unrotate_centroids": bool(c.unrotate_centroids), "verbose": bool(c.verbose)}
    path = write_results_to_csv(results_dir, experiment_name, "superkmeans_amd", dataset, n_iters, len(stats), d, n, k,
                                construction_ms, 0, float(stats[-1].objective), config, results10, results100, balance)
    km.close()
    return {"csv": path, "construction_time_ms": construction_ms, "final_objective": float(stats[-1].objective),
            "n_clusters": k, "recall@10": results10, "recall@100": results100}


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("dataset", nargs="?", default="fmnist")
    ap.add_argument("experiment", nargs="?", default="end_to_end")
    ap.add_argument("--data-dir", default="benchmarks/data")
    ap.add_argument("--gt-dir", default="benchmarks/ground_truth")
    ap.add_argument("--results-dir", default="benchmarks/results")
    ap.add_argument("--synthetic", nargs=2, type=int, metavar=("N", "D"), help="generate clustered data instead of reading files")
    ap.add_argument("--iters", type=int, default=MAX_ITERS)
    ap.add_argument("--sampling-fraction", type=float, default=1.0)
    ap.add_argument("--n-clusters", type=int, default=None)
    args = ap.parse_args(argv)
    run_end_to_end(args.dataset, args.experiment, args.data_dir, args.gt_dir, args.results_dir,
                   tuple(args.synthetic) if args.synthetic else None, args.iters, args.sampling_fraction, args.n_clusters)


if __name__ == "__main__":
    main()
