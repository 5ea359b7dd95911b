#!/usr/bin/env python3
"""Benchmark of the Super K-Means assign/update hot path on one MI355X.

Workload (the headline configuration): n = 1,000,000 points, d = 1024, k = 10,000 centroids, fp32, seeded
Gaussian mixture of 10,000 centres with per-dimension variance decaying as 1/sqrt(j+1), rows
L2-normalised, generated directly in HBM.

One "step" is one Assign() pass (exact nearest centroid of every point) with points and centroids
resident in HBM; `value` is points per second over the timed steps.  The same run also times one
Train() (rotation + 1 GEMM-only iteration + pruned iterations, data resident in HBM) and reports
seconds per iteration and the per-stage device times next to their rooflines; with --host-pointers it
repeats Assign and Train on host pointers (`host_pointers`: the transfer-inclusive times, never `value`).
The CPU baseline is
the CPU oracle (OpenMP + BLAS restatement of the reference path) on a bounded prefix of the same
points, on the host cores of the same box.

Prints one JSON line.  Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--n N --d D --k K]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBPS = 8000.0


# L2 <-> fabric bytes of one exact search (the two gemm_argmin_kernel launches of an Assign pass), from two rocprofv3 --pmc passes (FETCH_SIZE, then
# WRITE_SIZE, KiB per dispatch) scaled by what the same counters read for a copy kernel of known size
# (FETCH_SIZE x 1.943, WRITE_SIZE x 1.000); counters cannot be read from inside this process, so the figure is
# kept per workload shape (n, d, k) and is null for shapes that were not profiled.
MEASURED_TRAFFIC_BYTES = {
    (1_000_000, 1024, 10_000): int(((31_523_194 + 2_005_616) * 1.943 + 609_375 + 7_812) * 1024),
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--n", type=int, default=1_000_000)
    ap.add_argument("--d", type=int, default=1024)
    ap.add_argument("--k", type=int, default=10_000)
    ap.add_argument("--train-iters", type=int, default=10)
    ap.add_argument("--cpu-assign-points", type=int, default=131072)
    ap.add_argument("--cpu-train-points", type=int, default=65536)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-train", action="store_true")
    ap.add_argument("--host-pointers", action="store_true",
                    help="also run the transfer-inclusive leg (Assign and Train called with host pointers); off by "
                         "default so that a kernel trace of the default command holds the resident launches only")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain row-copy kernel of known size (1 GiB read + 1 GiB write) three times; "
                         "used to scale the FETCH_SIZE / WRITE_SIZE hardware counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every box of this build has a single MI355X and the hot path "
              "is built and measured on one device (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    from superkmeans_amd import _capi

    if args.copy_calibration:
        ctx = _capi.Context(0)
        rows, width = 1 << 18, 1024
        src, dst = ctx.empty((rows, width)), ctx.empty((rows, width))
        index = ctx.array(np.arange(rows, dtype=np.uint64))
        _capi.check(ctx.lib.skm_fill_u32(ctx.handle, src.ptr, 0x3f800000, rows * width))
        for _ in range(3):
            _capi.check(ctx.lib.skm_gather_rows(ctx.handle, src.ptr, width, index.ptr, rows, dst.ptr, None, None))
        ctx.sync()
        print(json.dumps({"copy_calibration": "gather_rows_kernel", "bytes_read": rows * width * 4 + rows * 8,
                          "bytes_written": rows * width * 4, "launches": 3}))
        ctx.close()
        return

    n, d, k = args.n, args.d, args.k
    cfg = dict(iters=args.train_iters, sampling_fraction=1.0, early_termination=0, seed=42, suppress_warnings=1)
    km = _capi.KMeans(k, d, **cfg)
    ctx, lib = km.ctx, km.lib

    # ---- synthetic points, resident in HBM ----
    dX = ctx.empty((n, d))
    _capi.check(lib.skm_synth_gaussian_mixture(ctx.handle, dX.ptr, n, d, 0, k, 1234, 5678, 1.0, 0.3, 0.25, 1))
    ctx.sync()

    # ---- Train (device-resident data), per-stage device timers ----
    train = None
    centroids = None
    if not args.no_train:
        ctx.prof_enable(True)
        ctx.prof_reset()
        km.set_prune_accounting(False)
        t0 = time.perf_counter()
        centroids = km.train_device(dX, n)
        ctx.sync()
        train_s = time.perf_counter() - t0
        prof = ctx.prof()
        ctx.prof_enable(False)
        stats = km.stats()
        n_gemm = sum(1 for s in stats if s.is_gemm_only)
        n_pruned = len(stats) - n_gemm
        ms = lambda name: prof.get(name, (0.0, 0))[0]
        calls = lambda name: prof.get(name, (0.0, 0))[1]
        # A second, untimed Train of an identical object only to count the pairs entering each pruning step.
        km2 = _capi.KMeans(k, d, **cfg)
        km2.set_prune_accounting(True)
        km2.train_device(dX, n)
        acct = km2.prune_accounting()
        km2.close()
        _, V = _capi.dimension_split(d)
        prune_bytes = 0.0
        for row, s in zip(acct, [s for s in stats if not s.is_gemm_only]):
            pairs_blocks = float(sum(int(x) for x in row[1:-1]))
            pairs_tail = float(row[-1])
            prune_bytes += 4.0 * (n * (d - s.partial_d) + 64.0 * pairs_blocks + (V - s.partial_d) * pairs_tail) + 8.0 * n
        partial_flops = sum(2.0 * n * k * s.partial_d for s in stats if not s.is_gemm_only)
        stage = {}

        def add_stage(name, bound, work, t_ms, unit_peak):
            if t_ms <= 0:
                return
            ach = work / (t_ms * 1e-3) / (1e12 if bound == "mfma" else 1e9)
            stage[name] = {"bound": bound, "ms": round(t_ms, 3), "achieved": round(ach, 2),
                           "peak": unit_peak, "unit": "TFLOP/s" if bound == "mfma" else "GB/s",
                           "frac": round(ach / unit_peak, 4)}

        add_stage("rotation", "mfma", 2.0 * (n + k) * d * d, ms("rotator"), PEAK_FP32_MFMA_TFLOPS)
        add_stage("full_distance_gemm", "mfma", 2.0 * n * k * d * n_gemm, ms("search/1st_blas"), PEAK_FP32_MFMA_TFLOPS)
        # the dense redo of overflowing points is part of the same two stages
        add_stage("partial_distance_gemm", "mfma", partial_flops, ms("search/blas") + ms("search/overflow/blas"),
                  PEAK_FP32_MFMA_TFLOPS)
        add_stage("prune", "hbm", prune_bytes, ms("search/seed") + ms("search/pdx") + ms("search/overflow/pdx"),
                  PEAK_HBM_GBPS)
        add_stage("update", "hbm", len(stats) * (4.0 * n * d + 8.0 * n + 4.0 * k * d + 4.0 * k), ms("update_centroids"), PEAK_HBM_GBPS)
        add_stage("pdx_relayout", "hbm", calls("consolidate/pdxify") * (2.0 * 4 * k * d + 4.0 * k * V), ms("consolidate/pdxify"), PEAK_HBM_GBPS)
        iter_ms = ms("search") + ms("update_centroids") + ms("consolidate/pdxify") + ms("consolidate/splitting") + \
            ms("compute_cost") + ms("shift") + ms("norms_calc")
        gemm_iter_ms = ms("search/1st_blas") + ms("search/merge")
        train = {
            "train_s_end_to_end": round(train_s, 4),
            "iters": len(stats),
            "train_s_per_iter_mean": round(train_s / max(1, len(stats)), 4),
            "train_s_per_gemm_only_iter_search": round(gemm_iter_ms * 1e-3 / max(1, n_gemm), 4),
            "train_s_per_pruned_iter_search": round((ms("search") - gemm_iter_ms) * 1e-3 / max(1, n_pruned), 4),
            "device_ms_all_iteration_stages": round(iter_ms, 2),
            "final_objective": stats[-1].objective,
            "partial_d": [s.partial_d for s in stats],
            "not_pruned_pct": [round(s.not_pruned_pct, 5) for s in stats],
            "stages": stage,
        }

    if centroids is None:
        centroids = dX.download(k)  # first k points as centroids
    dC = ctx.array(centroids)
    dOut = ctx.empty(n, np.uint32)

    # ---- Assign steps: W warm-up, K timed; device timers give the GEMM kernel's launch duration ----
    for _ in range(args.warmup):
        km.assign_device(dX, dC, n, k, dOut)
    ctx.sync()
    ctx.prof_enable(True)
    ctx.prof_reset()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        km.assign_device(dX, dC, n, k, dOut)
    ctx.sync()
    elapsed = time.perf_counter() - t0
    prof = ctx.prof()
    ctx.prof_enable(False)
    ms_per_step = elapsed * 1e3 / args.steps
    value = n * args.steps / elapsed
    gemm_ms, gemm_calls = prof.get("search/1st_blas", (0.0, 0))
    gemm_avg_ms = gemm_ms / max(1, gemm_calls)
    launches_per_step = gemm_calls / max(1, args.steps)
    flops_per_launch = 2.0 * n * k * d / max(1.0, launches_per_step)
    achieved = flops_per_launch / (gemm_avg_ms * 1e-3) / 1e12 if gemm_avg_ms > 0 else 0.0
    roofline = {"kernel": "gemm_argmin_kernel", "bound": "mfma", "achieved": round(achieved, 2),
                "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
                "traffic": MEASURED_TRAFFIC_BYTES.get((n, d, k)), "avg_launch_ms": round(gemm_avg_ms, 3), "flops_per_launch": flops_per_launch}
    if 0 < k % 256 <= 128 and k > 256:
        # the exact search is then two launches of the same kernel; avg_launch_ms is their sum
        roofline["launches"] = (f"256x256 tiles over the first {k - k % 256} centroids + {32 * ((k % 256 + 31) // 32)}x128 tiles over the last "
                                f"{k % 256}")
    gpu_assign = dOut.download()

    # ---- PCIe-inclusive leg (reported beside `value`, never as it): the same calls on host pointers ----
    host_pointers = None
    if args.host_pointers:
        Xhost = dX.download()
        km.assign(Xhost[: min(n, 4096)], centroids)  # buffers of the host path touched once
        t0 = time.perf_counter()
        host_assign = km.assign(Xhost, centroids)
        host_assign_s = time.perf_counter() - t0
        host_pointers = {"assign_ms": round(host_assign_s * 1e3, 1), "assign_points_per_s": round(n / host_assign_s, 1),
                         "assign_equals_resident": bool(np.array_equal(host_assign, gpu_assign)),
                         "note": "pageable host rows, uploaded in 256 MiB slabs on a transfer stream while the "
                                 "previous slab is searched"}
        if not args.no_train:
            kmh = _capi.KMeans(k, d, **cfg)
            t0 = time.perf_counter()
            host_centroids = kmh.train(Xhost)
            host_pointers["train_s_end_to_end"] = round(time.perf_counter() - t0, 4)
            host_pointers["train_equals_resident"] = bool(np.array_equal(host_centroids, centroids))
            kmh.close()
        del Xhost

    # ---- CPU baseline: the oracle on a bounded prefix of the same points ----
    cpu = None
    if not args.no_cpu:
        from oracle import oracle as O

        O.load()
        O.set_threads(0)
        cores = O.get_threads()
        m = min(n, args.cpu_assign_points)
        Xh = dX.download(m)
        ok = O.KMeans(k, d, sampling_fraction=1.0, suppress_warnings=1)
        t0 = time.perf_counter()
        oa = ok.assign(Xh, centroids)
        cpu_assign_s = time.perf_counter() - t0
        agree = float(np.mean(oa == gpu_assign[:m]))
        cpu = {"value": round(m / cpu_assign_s, 1), "unit": "points/s", "cores": int(cores), "kind": "port",
               "sample": f"Assign of the first {m} of the {n} points against the same {k} centroids, "
                         f"{cpu_assign_s:.2f} s, BLAS={os.path.basename(O.blas_name())}",
               "assign_agreement_with_gpu": agree}
        mt = min(n, args.cpu_train_points)
        if mt >= k and not args.no_train:
            okt = O.KMeans(k, d, iters=3, sampling_fraction=1.0, early_termination=0, suppress_warnings=1)
            t0 = time.perf_counter()
            okt.train(Xh[:mt] if mt <= m else dX.download(mt))
            cpu_train_s = time.perf_counter() - t0
            cpu["train_sample"] = (f"Train (rotation + 1 GEMM-only + 2 pruned iterations) on the first {mt} points, "
                                   f"k={k}: {cpu_train_s:.2f} s end to end")
            cpu["train_s_end_to_end_on_sample"] = round(cpu_train_s, 3)

    out = {
        "metric": "assign_points_per_s",
        "value": round(value, 1),
        "unit": "points/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"SuperKMeans Assign (+ Train {args.train_iters} iters) fp32, n={n}, d={d}, k={k}, "
                               "seeded Gaussian mixture with 1/sqrt(j+1) variance decay, rows L2-normalised, resident in HBM"},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "train": train,
        "host_pointers": host_pointers,
    }
    print(json.dumps(out))
    km.close()


if __name__ == "__main__":
    main()
