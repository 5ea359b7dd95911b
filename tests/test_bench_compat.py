"""Harness compatibility with the reference's benchmarks/ tree: file formats, recall evaluation, CSV layout."""
import csv
import json

import numpy as np
import pytest

from superkmeans_amd import bench_compat as bc


def test_default_n_clusters_and_dataset_table():
    # benchmarks/bench_utils.h:21-23 and :77-94
    assert bc.get_default_n_clusters(1_000_000) == 4000 and bc.get_default_n_clusters(60000) == 979
    assert bc.get_default_n_clusters(0) == 1
    assert bc.DATASET_PARAMS["cohere"] == (10_000_000, 1024) and bc.DATASET_PARAMS["mxbai"] == (769382, 1024)


def test_read_bin_and_ground_truth_round_trip(tmp_path):
    x = np.arange(5 * 7, dtype=np.float32).reshape(5, 7)
    p = tmp_path / "data_toy.bin"
    x.tofile(p)
    assert np.array_equal(bc.read_bin(p, 5, 7), x) and np.array_equal(bc.read_bin(p, 3, 7), x[:3])
    with pytest.raises(ValueError, match="expected at least"):
        bc.read_bin(p, 6, 7)
    g = tmp_path / "toy.json"
    g.write_text(json.dumps({"0": [4, 2, 1], "3": [0]}))
    assert bc.load_ground_truth(g) == {0: [4, 2, 1], 3: [0]}
    assert bc.load_ground_truth(tmp_path / "missing.json") == {}


def test_compute_recall_by_hand():
    # 1000 one-dimensional centroids at 0, 1, 2, ...; 0.1 % explores 1 centroid, 0.2 % explores 2, 10 % explores 100
    k = 1000
    centroids = np.arange(k, dtype=np.float32)[:, None]
    queries = np.array([[10.2], [500.4]], dtype=np.float32)
    # data vector i is assigned to cluster i // 2 (2000 vectors, two per cluster)
    assignments = (np.arange(2 * k) // 2).astype(np.uint32)
    gt = {0: [20, 21, 22, 24], 1: [1000, 1002, 0, 1]}  # clusters {10, 10, 11, 12} and {500, 501, 0, 0}
    res = bc.compute_recall(gt, assignments, queries, centroids, knn=4)
    assert len(res) == len(bc.EXPLORE_FRACTIONS)
    e1 = res[0]   # nearest centroid only: query 0 -> {10}: 2 of 4; query 1 -> {500}: 1 of 4
    assert e1[0] == 1 and e1[2] == pytest.approx((0.5 + 0.25) / 2) and e1[4] == 2.0
    e2 = res[1]   # two nearest: {10, 11}: 3 of 4; {500, 501}: 2 of 4
    assert e2[0] == 2 and e2[2] == pytest.approx((0.75 + 0.5) / 2) and e2[4] == 4.0
    assert e2[3] == pytest.approx(np.std([0.75, 0.5], ddof=1))
    e100 = res[-1]  # 100 nearest cover cluster 12 but never cluster 0 for query 1
    assert e100[0] == 100 and e100[2] == pytest.approx((1.0 + 0.5) / 2) and e100[4] == 200.0
    # knn truncates the ground-truth list; a query without ground truth still counts in the mean's denominator
    res2 = bc.compute_recall({0: gt[0]}, assignments, queries, centroids, knn=2)
    assert res2[0][2] == pytest.approx(1.0 / 2) and res2[0][3] == 0.0


def test_csv_layout_matches_the_reference_columns(tmp_path, monkeypatch):
    monkeypatch.setenv("SKM_ARCH", "mi355x")
    r10 = [(max(1, int(4000 * f)), f, 0.5, 0.1, 1234.5) for f in bc.EXPLORE_FRACTIONS]
    r100 = [(max(1, int(4000 * f)), f, 0.25, 0.05, 1234.5) for f in bc.EXPLORE_FRACTIONS]
    cfg = {"iters": 10, "use_blas_only": False}
    for _ in range(2):
        path = bc.write_results_to_csv(tmp_path, "end_to_end", "superkmeans_amd", "toy", 10, 10, 1024, 1000000, 4000,
                                       512.345, 0, 195845.078125, cfg, r10, r100, {"mean": 250.0, "min": 1, "max": 900})
    assert path.endswith("mi355x/end_to_end.csv")
    rows = list(csv.reader(open(path)))
    assert len(rows) == 3  # header once, two rows
    header = rows[0]
    assert header[:11] == ["timestamp", "algorithm", "dataset", "n_iters", "actual_iterations", "dimensionality",
                           "data_size", "n_clusters", "construction_time_ms", "threads", "final_objective"]
    assert header[11:15] == ["recall@10@0.10", "recall_std@10@0.10", "centroids_explored@10@0.10", "vectors_explored@10@0.10"]
    assert header[-2:] == ["balance_stats", "config"] and "recall@100@10.00" in header and "recall@10@1.25" in header
    assert len(header) == 11 + 2 * len(bc.EXPLORE_FRACTIONS) * 4 + 2 == len(rows[1])
    row = rows[1]
    assert row[1:11] == ["superkmeans_amd", "toy", "10", "10", "1024", "1000000", "4000", "512.35", "0", "195845.078125"]
    assert row[11:15] == ["0.500000", "0.100000", "4", "1234.50"]
    assert json.loads(row[-1]) == cfg and json.loads(row[-2])["max"] == 900
    # a run without recall data writes the short header
    p2 = bc.write_results_to_csv(tmp_path, "no_recall", "superkmeans_amd", "toy", 10, 10, 8, 100, 40, 1.0, 0, 2.0, cfg, [], [])
    assert list(csv.reader(open(p2)))[0][-3:] == ["final_objective", "balance_stats", "config"]


def test_cluster_balance_stats():
    s = bc.cluster_balance_stats(np.array([0, 0, 0, 1, 3, 3], dtype=np.uint32), 4)  # sizes 3, 1, 0, 2
    assert s["mean"] == 1.5 and s["min"] == 0 and s["max"] == 3
    assert s["geometric_mean"] == pytest.approx((3 * 1 * 2) ** (1 / 3)) and s["cv"] == pytest.approx(np.std([3, 1, 0, 2]) / 1.5)


@pytest.mark.gpu
def test_end_to_end_driver_on_synthetic_data(tmp_path):
    out = bc.run_end_to_end("synthetic", "end_to_end", results_dir=str(tmp_path), synthetic=(20000, 64), n_iters=4)
    rows = list(csv.reader(open(out["csv"])))
    assert len(rows) == 2 and len(rows[0]) == len(rows[1]) == 11 + 2 * len(bc.EXPLORE_FRACTIONS) * 4 + 2
    assert rows[1][1] == "superkmeans_amd" and int(rows[1][7]) == out["n_clusters"] == 565
    rec = dict(zip(rows[0], rows[1]))
    assert 0.0 < float(rec["recall@10@0.10"]) <= float(rec["recall@10@10.00"]) <= 1.0
    assert float(rec["recall@100@10.00"]) > 0.9  # probing 10 % of the clusters of well-separated blobs finds the neighbours
    assert float(rec["construction_time_ms"]) > 0 and float(rec["final_objective"]) > 0
