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

--config selects one of the five benchmark configurations (default C2, the headline; its JSON line keeps the same
keys): C1 n=100,000 d=768 k=1,000 (25 iterations), C2, C3 n=10,000,000 d=1024 k=10,000 (Assign only), C4 hierarchical
n=10,000,000 d=1024 k=65,536, C5 n=2,000,000 d=1536 k=4,096 (low intrinsic dimension, heavy tails).  Every
configuration reports Assign points/s, Train seconds end to end and per iteration, the stage table and the CPU
baseline on a bounded sample; the transfer-inclusive leg runs by default where the host copy of the points is at most
16 GB (C1, C2, C5) and on request (--host-pointers) for the 41 GB configurations.

The headline run (no --config) adds three things to the same JSON line, none of them inside the timed steps:
`train.pruned_vs_exact_agreement` (how often the last pruned iteration of the Train kept the exact nearest centroid: the
device over all points, the CPU oracle on a sample of the same state), `assign_training_points` (the pruned
AssignTrainingPoints on host rows for sampling_fraction 1.0 and for the reference's default configuration, with its
agreement with Assign and the share of points whose candidate list overflowed) and `other_configs` (Assign and the
Train stage table of C1 and C5, without CPU or transfer legs).

Prints one JSON line.  Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C2] [--n N --d D --k K]
"""
import hashlib
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBPS = 8000.0


def kernel_sources_hash():
    """Identifies the device code of this tree: sha256 over the kernel sources and the headers they include."""
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "superkmeans_amd", "csrc")
    files = [os.path.join(csrc, f) for f in sorted(os.listdir(csrc)) if f.endswith((".hip", ".h"))]
    files.append(os.path.join(ROOT, "include", "skm_hip.h"))
    for f in files:
        with open(f, "rb") as fh:
            h.update(os.path.basename(f).encode() + b"\0" + fh.read())
    return h.hexdigest()[:16]


# Counter figures cannot be read from inside this process: they are recorded here from the rocprofv3 --pmc runs whose
# summaries are under profiles/ (FETCH_SIZE and WRITE_SIZE in KiB per dispatch, scaled by what the same counters read for a
# copy kernel of known size: FETCH_SIZE x 1.943, WRITE_SIZE x 1.000), per workload shape.  Every entry names the summary it
# comes from and the kernel_sources_hash() of the tree that was profiled; the figure is reported only while the tree
# still hashes to that value (otherwise the JSON carries null and the reason), so it cannot outlive the kernels it describes.
MEASURED_SOURCES_HASH = "011ebb84c588c41e"
MEASURED_TRAFFIC_BYTES = {
    # the two gemm_argmin_kernel launches of an Assign pass
    (1_000_000, 1024, 10_000): (int(((31_436_956 + 2_006_114) * 1.943 + 609_375 + 7_812) * 1024),
                                "profiles/gemm_argmin_kernel_assign_n1M_d1024_k10k_hbm_traffic.md"),
}
# every seed_distance_kernel and list-walk launch of one Train of (n, d, k, iterations)
MEASURED_PRUNE_TRAFFIC_BYTES = {
    (1_000_000, 1024, 10_000, 10): (int((49_811_612 * 1.943 + 1_760_127) * 1024),
                                    "profiles/gemm_argmin_kernel_assign_n1M_d1024_k10k_hbm_traffic.md"),
    (2_000_000, 1536, 4_096, 10): (int((881_240_000 * 1.943 + 3_441_701) * 1024),
                                   "profiles/train_n2M_d1536_k4096_kernel_stats_list_walk_traffic.md"),
}


def measured(table, key):
    """(bytes, provenance) of a counter figure, or (None, why not)."""
    if key not in table:
        return None, "shape not profiled"
    value, source = table[key]
    now = kernel_sources_hash()
    if now != MEASURED_SOURCES_HASH:
        return None, f"kernel sources changed since {source} was taken (profiled {MEASURED_SOURCES_HASH}, now {now})"
    return value, f"{source} @ kernel sources {MEASURED_SOURCES_HASH}"


# name -> (n, d, k, Train iterations, hierarchical, description of the generator)
CONFIGS = {
    "C1": (100_000, 768, 1_000, 25, False, "1,000 centres ~ N(0, I), point = centre + 0.3 N(0, I)"),
    "C2": (1_000_000, 1024, 10_000, 10, False, "seeded Gaussian mixture with 1/sqrt(j+1) variance decay"),
    "C3": (10_000_000, 1024, 10_000, 0, False, "fixed centroids ~ N(0, I) normalised, point = centroid + 0.5 N(0, I)"),
    "C4": (10_000_000, 1024, 65_536, 0, True, "two-level mixture: 256 coarse centres, 65,536 fine centres at sigma 0.2, "
                                               "point noise 0.1"),
    "C5": (2_000_000, 1536, 4_096, 10, False, "rank-64 Gaussian latent through a fixed linear map + Student-t(3) noise"),
}


def generate_points(_capi, lib, ctx, name, dX, n, d, k):
    """Fills dX (n x d, device) with the configuration's seeded synthetic rows (L2-normalised)."""
    if name == "C1":
        _capi.check(lib.skm_synth_gaussian_mixture(ctx.handle, dX.ptr, n, d, 0, k, 101, 102, 1.0, 0.3, 0.0, 1))
    elif name == "C3":
        _capi.check(lib.skm_synth_gaussian_mixture(ctx.handle, dX.ptr, n, d, 0, k, 77, 78, 1.0, 0.5, 0.0, 1))
    elif name == "C4":
        _capi.check(lib.skm_synth_two_level_mixture(ctx.handle, dX.ptr, n, d, 0, 256, 65_536, 9, 0.2, 0.1))
    elif name == "C5":
        _capi.check(lib.skm_synth_low_rank(ctx.handle, dX.ptr, n, d, 0, 64, 21, 0.05))
    else:
        _capi.check(lib.skm_synth_gaussian_mixture(ctx.handle, dX.ptr, n, d, 0, k, 1234, 5678, 1.0, 0.3, 0.25, 1))


def stage_table(n, d, k, ks, hierarchical, stats, acct, prof, V):
    """Per-stage device time of one Train next to the roofline that bounds the stage."""
    ms = lambda name: prof.get(name, (0.0, 0))[0]
    calls = lambda name: prof.get(name, (0.0, 0))[1]
    n_gemm = sum(1 for s in stats if s.is_gemm_only)
    # Algorithmic bytes of the pruning stage: the point row and its previous centroid for the seed distance, 8 bytes per
    # candidate pair of the lists, 256 bytes of centroid block per visited (pair, 64-dimension block), the [d', V) tail
    # of the centroid per pair that reaches it, and of the point's own row what the walks read: one 256-byte slice per
    # visited (pair, block) at most (survivors of one point share the slice) and never more than the row's tail.
    prune_bytes, blocks_visited = 0.0, 0.0
    for row, s in zip(acct, [s for s in stats if not s.is_gemm_only]):
        pairs_blocks = float(sum(int(x) for x in row[1:-1]))
        pairs_tail = float(row[-1])
        x_tails = min(4.0 * n * (d - s.partial_d), 4.0 * (64.0 * pairs_blocks + (V - s.partial_d) * pairs_tail))
        prune_bytes += 4.0 * n * d + 8.0 * float(row[0]) + x_tails + \
            4.0 * (64.0 * pairs_blocks + (V - s.partial_d) * pairs_tail) + 8.0 * n
        blocks_visited += pairs_blocks
    partial_flops = sum(2.0 * n * k * s.partial_d for s in stats if not s.is_gemm_only)  # flat runs only
    stage = {}

    def add_stage(name, bound, work, t_ms, unit_peak):
        if t_ms <= 0:
            return
        ach = work / (t_ms * 1e-3) / (1e12 if bound == "mfma" else 1e9)
        stage[name] = {"bound": bound, "ms": round(t_ms, 3), "achieved": round(ach, 2),
                       "peak": unit_peak, "unit": "TFLOP/s" if bound == "mfma" else "GB/s",
                       "frac": round(ach / unit_peak, 4)}

    add_stage("rotation", "mfma", 2.0 * (n + ks) * d * d, ms("rotator"), PEAK_FP32_MFMA_TFLOPS)
    add_stage("full_distance_gemm", "mfma", 2.0 * n * ks * d * n_gemm, ms("search/1st_blas"), PEAK_FP32_MFMA_TFLOPS)
    # the second pass over points whose candidate list overflowed is part of the same two stages
    add_stage("partial_distance_gemm", "mfma", partial_flops, ms("search/blas") + ms("search/overflow/blas"),
              PEAK_FP32_MFMA_TFLOPS)
    add_stage("prune", "hbm", prune_bytes,
              ms("search/seed") + ms("search/pdx") + ms("search/overflow/seed") + ms("search/overflow/pdx"), PEAK_HBM_GBPS)
    add_stage("update", "hbm", len(stats) * (4.0 * n * d + 8.0 * n + 4.0 * ks * d + 4.0 * ks), ms("update_centroids"), PEAK_HBM_GBPS)
    if not hierarchical:
        add_stage("pdx_relayout", "hbm", calls("consolidate/pdxify") * (2.0 * 4 * k * d + 4.0 * k * V), ms("consolidate/pdxify"), PEAK_HBM_GBPS)
    if "prune" in stage:
        p = stage["prune"]
        # Two rates.  Algorithmic bytes / time counts every 256-byte gather of a centroid block, most of which the
        # caches serve: a rate of useful bytes that can exceed the HBM peak.  Counter bytes / time is what leaves the
        # L2s: that one is `frac` whenever the counters of these kernel sources are on record (otherwise `frac` stays
        # the algorithmic rate and `frac_is` says so).  `ns_per_pair_block` is the unit that tracks the walk's progress.
        p["algorithmic_bytes"] = prune_bytes
        p["algorithmic_achieved"] = p["achieved"]
        p["algorithmic_frac"] = p["frac"]
        if blocks_visited > 0:
            p["pair_blocks_visited"] = blocks_visited
            p["ns_per_pair_block"] = round(p["ms"] * 1e6 / blocks_visited, 4)
        value, source = measured(MEASURED_PRUNE_TRAFFIC_BYTES, (n, d, k, len(stats)))
        p["measured_bytes"] = value
        p["measured_from"] = source
        if value:
            p["achieved"] = round(value / (p["ms"] * 1e-3) / 1e9, 2)
            p["frac"] = round(p["achieved"] / PEAK_HBM_GBPS, 4)
            p["frac_is"] = "counter bytes (FETCH_SIZE, WRITE_SIZE of every launch of the stage) / time / HBM peak"
        else:
            p["frac_is"] = "algorithmic bytes / time / HBM peak (block gathers are mostly cache hits): no counter figure for this shape and these sources"
        p["measured_frac"] = p["frac"] if value else None
    return stage


def run_config(args, name, n, d, k, train_iters, hierarchical, generator, steps, warmup, with_cpu, with_host, with_extras,
               with_agreement=False):
    """One configuration: Train (first and second object of the process, stage table), timed Assign steps, and on
    request the transfer-inclusive leg, the CPU baseline and the headline extras.  Returns the JSON object."""
    from superkmeans_amd import _capi

    no_train = args.no_train or (train_iters == 0 and not hierarchical)
    if hierarchical:
        cfg = dict(early_termination=0, seed=42, suppress_warnings=1)  # 3 + 5 + 0 iterations, the reference's defaults
        if args.n_threads is not None:
            cfg["n_threads"] = args.n_threads
    else:
        cfg = dict(iters=max(1, train_iters), sampling_fraction=1.0, early_termination=0, seed=42, suppress_warnings=1)
    def new_object():
        obj = _capi.KMeans(k, d, hierarchical=hierarchical, **cfg)
        _capi.check(obj.lib.skm_ctx_set_walk_kernel(obj.ctx.handle, args.walk_kernel))
        _capi.check(obj.lib.skm_ctx_set_walk_launches(obj.ctx.handle, args.walk_launches))
        return obj

    km = new_object()
    ctx, lib = km.ctx, km.lib

    # ---- synthetic points, resident in HBM ----
    dX = ctx.empty((n, d))
    generate_points(_capi, lib, ctx, name, dX, n, d, k)
    ctx.sync()

    # ---- Train (device-resident data), per-stage device timers ----
    train = None
    centroids = None
    extras = {}
    if not no_train:
        km.set_prune_accounting(False)
        t0 = time.perf_counter()
        centroids = km.train_device(dX, n)
        ctx.sync()
        train_s = time.perf_counter() - t0
        # hierarchical: the owner object's timers cover the mesoclustering and the refinement; the fine clusterings
        # run on helper objects with their own contexts and show up as the rest of the end-to-end time
        phase_stats = {nm: km.stats(which) for which, nm in ((1, "mesoclustering"), (2, "fineclustering"), (3, "refinement"))} \
            if hierarchical else None
        stats = (phase_stats["mesoclustering"] + phase_stats["refinement"]) if hierarchical else km.stats()
        n_gemm = sum(1 for s in stats if s.is_gemm_only)
        n_pruned = len(stats) - n_gemm
        # A second, untimed Train of an identical object only to count the pairs entering each pruning step.
        acct = []
        if n_pruned and not hierarchical:
            km2 = new_object()
            km2.set_prune_accounting(True)
            km2.train_device(dX, n)
            acct = km2.prune_accounting()
            km2.close()
        # The timed Train above is the first of the process: it pays for every device allocation (and its kernels for
        # the first touch of fresh device memory).  A third, identical object finds the blocks in the library's
        # per-device cache: its end-to-end time is reported beside the first, and its per-stage device timers (with the
        # event pairs they add around every stage) make the stage table.
        km3 = new_object()
        km3.set_prune_accounting(False)
        t0 = time.perf_counter()
        km3.train_device(dX, n)
        km3.ctx.sync()
        train_warm_s = time.perf_counter() - t0
        km3.close()
        km4 = new_object()
        km4.set_prune_accounting(False)
        km4.ctx.prof_enable(True)
        km4.ctx.prof_reset()
        km4.train_device(dX, n)
        km4.ctx.sync()
        prof = km4.ctx.prof()
        km4.close()
        ms = lambda nm: prof.get(nm, (0.0, 0))[0]
        _, V = _capi.dimension_split(d)
        # the owner object of a hierarchical Train searches among the sqrt(k) mesocluster centroids
        ks = int(round(k ** 0.5)) if hierarchical else k
        stage = stage_table(n, d, k, ks, hierarchical, stats, acct, prof, V)
        iter_ms = ms("search") + ms("update_centroids") + ms("consolidate/pdxify") + ms("consolidate/splitting") + \
            ms("compute_cost") + ms("shift") + ms("norms_calc")
        gemm_iter_ms = ms("search/1st_blas") + ms("search/merge")
        train = {
            "train_s_end_to_end": round(train_s, 4),
            "train_s_end_to_end_second_object": round(train_warm_s, 4),
            "iters": len(stats),
            "train_s_per_iter_mean": round(train_s / max(1, len(stats)), 4),
            "train_s_per_gemm_only_iter_search": round(gemm_iter_ms * 1e-3 / max(1, n_gemm), 4),
            "train_s_per_pruned_iter_search": round((ms("search") - gemm_iter_ms) * 1e-3 / max(1, n_pruned), 4),
            "device_ms_all_iteration_stages": round(iter_ms, 2),
            "final_objective": stats[-1].objective,
            "partial_d": [s.partial_d for s in stats],
            "not_pruned_pct": [round(s.not_pruned_pct, 5) for s in stats],
            "stages": stage,
            "stages_from": "an identical Train of a later object of the process (device blocks from the library's cache), "
                           "with per-stage device timers on; the end-to-end times above are taken without timers",
        }
        if hierarchical:
            train["phases"] = {nm: {"iterations": len(v), "final_objective": (v[-1].objective if v and nm != "fineclustering" else None)}
                               for nm, v in phase_stats.items()}
            train["owner_device_ms"] = round(iter_ms + ms("rotator"), 2)
            train["fine_phase_and_host_s"] = round(train_s - (iter_ms + ms("rotator")) * 1e-3, 4)
        if (with_extras or with_agreement) and not hierarchical and n_pruned and len(stats) >= 2:
            train["pruned_vs_exact_agreement"] = pruned_vs_exact(args, _capi, km, dX, n, d, k, cfg, stats,
                                                                 oracle_sample=with_extras and not args.no_cpu)

    if centroids is None and name == "C3":
        # the fixed, seeded centroids of the Assign-only configuration: the generator's own centres
        dC3 = ctx.empty((k, d))
        _capi.check(lib.skm_synth_gaussian_mixture(ctx.handle, dC3.ptr, k, d, 0, 0, 0, 79, 0.0, 1.0, 0.0, 1))
        centroids = dC3.download()
        dC3.free()
    if centroids is None:
        centroids = dX.download(k)  # first k points as centroids
    dC = ctx.array(centroids)
    dOut = ctx.empty(n, np.uint32)

    # ---- Assign steps: W warm-up, K timed; device timers give the GEMM kernel's launch duration ----
    for _ in range(warmup):
        km.assign_device(dX, dC, n, k, dOut)
    ctx.sync()
    ctx.prof_enable(True)
    ctx.prof_reset()
    t0 = time.perf_counter()
    for _ in range(steps):
        km.assign_device(dX, dC, n, k, dOut)
    ctx.sync()
    elapsed = time.perf_counter() - t0
    prof = ctx.prof()
    ctx.prof_enable(False)
    ms_per_step = elapsed * 1e3 / steps
    value = n * steps / elapsed
    gemm_ms, gemm_calls = prof.get("search/1st_blas", (0.0, 0))
    gemm_avg_ms = gemm_ms / max(1, gemm_calls)
    launches_per_step = gemm_calls / max(1, steps)
    flops_per_launch = 2.0 * n * k * d / max(1.0, launches_per_step)
    achieved = flops_per_launch / (gemm_avg_ms * 1e-3) / 1e12 if gemm_avg_ms > 0 else 0.0
    traffic, traffic_from = measured(MEASURED_TRAFFIC_BYTES, (n, d, k))
    roofline = {"kernel": "gemm_argmin_kernel", "bound": "mfma", "achieved": round(achieved, 2),
                "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
                "traffic": traffic, "traffic_from": traffic_from, "avg_launch_ms": round(gemm_avg_ms, 3),
                "flops_per_launch": flops_per_launch}
    if 0 < k % 256 <= 128 and k > 256:
        # the exact search is then two launches of the same kernel; avg_launch_ms is their sum
        roofline["launches"] = (f"256x256 tiles over the first {k - k % 256} centroids + {32 * ((k % 256 + 31) // 32)}x128 tiles over the last "
                                f"{k % 256}")
    gpu_assign = dOut.download()

    # ---- PCIe-inclusive leg (reported beside `value`, never as it): the same calls on host pointers ----
    host_pointers = None
    atp = None
    if with_host:
        Xhost = dX.download()
        km.assign(Xhost[: min(n, 4096)], centroids)  # buffers of the host path touched once
        t0 = time.perf_counter()
        host_assign = km.assign(Xhost, centroids)
        host_assign_s = time.perf_counter() - t0
        host_pointers = {"assign_ms": round(host_assign_s * 1e3, 1), "assign_points_per_s": round(n / host_assign_s, 1),
                         "assign_equals_resident": bool(np.array_equal(host_assign, gpu_assign)),
                         "note": "pageable host rows, uploaded in 256 MiB slabs on a transfer stream while the "
                                 "previous slab is searched"}
        if not no_train:
            kmh = _capi.KMeans(k, d, hierarchical=hierarchical, **cfg)
            t0 = time.perf_counter()
            host_centroids = kmh.train(Xhost)
            host_pointers["train_s_end_to_end"] = round(time.perf_counter() - t0, 4)
            host_pointers["train_equals_resident"] = bool(np.array_equal(host_centroids, centroids))
            kmh.close()
        if with_extras and not no_train and not hierarchical:
            atp = assign_training_points_legs(_capi, km, Xhost, centroids, gpu_assign, n, d, k)
        del Xhost

    # ---- CPU baseline: the oracle on a bounded prefix of the same points ----
    cpu = cpu_baseline(args, dX, n, d, k, centroids, gpu_assign, no_train or hierarchical) if with_cpu else None

    out = {
        "metric": "assign_points_per_s",
        "value": round(value, 1),
        "unit": "points/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{name}: {'Hierarchical' if hierarchical else ''}SuperKMeans Assign"
                               + ("" if no_train else f" (+ Train {'3+5+0' if hierarchical else train_iters} iters)")
                               + f" fp32, n={n}, d={d}, k={k}, {generator}, rows L2-normalised, resident in HBM"},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "train": train,
        "host_pointers": host_pointers,
    }
    if atp is not None:
        out["assign_training_points"] = atp
    km.close()
    return out


def pruned_vs_exact(args, _capi, km, dX, n, d, k, cfg, stats, oracle_sample):
    """How often the last pruned iteration of the Train kept the exact nearest centroid (ADSampling prunes with a
    probabilistic bound).  Train is deterministic: a run with one iteration less gives the rotated centroids and the
    assignments the last iteration started from; the exact search among those centroids is the truth.  The CPU oracle
    runs its own pruned search from the same state on a sample."""
    ctx, lib = km.ctx, km.lib
    last = stats[-1]
    prev_cfg = dict(cfg, iters=len(stats) - 1, unrotate_centroids=0)
    kp = _capi.KMeans(k, d, **prev_cfg)
    C_prev = kp.train_device(dX, n)
    a_prev = kp.assignments(n)
    kp.close()
    a_last = km.assignments(n)
    Q, _ = _capi.pruner_tables(d, 1.5, 42)
    dQ, dR = ctx.array(Q), ctx.empty((n, d))
    _capi.check(lib.skm_rotate(ctx.handle, dX.ptr, n, d, dQ.ptr, dR.ptr))
    dC, xn, cn = ctx.array(C_prev), ctx.empty(n), ctx.empty(k)
    a_exact, d_exact = ctx.empty(n, np.uint32), ctx.empty(n)
    _capi.check(lib.skm_norms(ctx.handle, dR.ptr, n, d, d, xn.ptr))
    _capi.check(lib.skm_norms(ctx.handle, dC.ptr, k, d, d, cn.ptr))
    _capi.check(lib.skm_assign_full(ctx.handle, dR.ptr, n, dC.ptr, k, d, xn.ptr, cn.ptr, a_exact.ptr, d_exact.ptr))
    ae = a_exact.download()
    out = {"iteration": int(last.iteration), "partial_d": int(last.partial_d),
           "gpu_pruned_equals_exact": round(float(np.mean(ae == a_last)), 6),
           "points": n}
    if oracle_sample:
        from oracle import oracle as O

        O.load()
        O.set_threads(0)
        m = min(n, 2048)
        ids = np.sort(np.random.default_rng(11).choice(n, m, replace=False))
        rows = np.empty((m, d), dtype=np.float32)
        for j, i in enumerate(ids):
            _capi.check(lib.skm_download(ctx.handle, rows[j].ctypes.data, dR.offset(int(i) * d), d * 4))
        oi, _, _ = O.find_nn_pruned(rows, C_prev, a_prev[ids], int(last.partial_d), O.ratios(d, 1.5))
        bi, _, _ = O.brute_force(rows, C_prev)
        out["oracle_sample"] = {"points": int(m), "oracle_pruned_equals_exact": round(float(np.mean(oi == bi)), 6),
                                "gpu_pruned_equals_exact": round(float(np.mean(a_last[ids] == bi)), 6),
                                "gpu_equals_oracle": round(float(np.mean(a_last[ids] == oi)), 6)}
    for a in (dQ, dR, dC, xn, cn, a_exact, d_exact):
        a.free()
    return out


def assign_training_points_legs(_capi, km, Xhost, centroids, exact_assign, n, d, k):
    """AssignTrainingPoints (the pruned assignment of the training points, superkmeans.h:397-564) on host rows: for the
    object trained on all points (seeds are the training assignments) and for the reference's default configuration
    (sampling_fraction 0.3, early termination: most points start from a meso-centroid's representative)."""
    legs = []

    def leg(obj, label, C, exact):
        ctx = obj.ctx
        ctx.prof_enable(True)
        ctx.prof_reset()
        t0 = time.perf_counter()
        got = obj.assign_training_points(Xhost, C)
        took = time.perf_counter() - t0
        prof = ctx.prof()
        ctx.prof_enable(False)
        over = obj.training_overflow()
        ms = lambda nm: round(prof.get(nm, (0.0, 0))[0], 2)
        legs.append({"config": label, "ms_end_to_end_from_host_rows": round(took * 1e3, 1),
                     "points_per_s": round(n / took, 1),
                     "equals_exact_assign": round(float(np.mean(got == exact)), 6),
                     "overflow_fraction": round(over / n, 4),
                     "device_ms": {"pruned_search": ms("search"), "seed": ms("search/seed"), "partial_gemm": ms("search/blas"),
                                   "list_walk": ms("search/pdx"), "second_pass": ms("search/overflow")}})

    leg(km, "sampling_fraction 1.0 (the Train above)", centroids, exact_assign)
    kd = _capi.KMeans(k, d, suppress_warnings=1)  # the reference's defaults: 10 iterations, 0.3, early termination
    t0 = time.perf_counter()
    Cd = kd.train(Xhost)
    train_ms = (time.perf_counter() - t0) * 1e3
    exact_d = kd.assign(Xhost, Cd)
    leg(kd, "reference defaults (sampling_fraction 0.3, early termination)", Cd, exact_d)
    legs[-1]["train_ms_from_host_rows"] = round(train_ms, 1)
    legs[-1]["train_iterations"] = len(kd.stats())
    kd.close()
    return legs


def cpu_baseline(args, dX, n, d, k, centroids, gpu_assign, no_train):
    from oracle import oracle as O

    O.load()
    O.set_threads(0)
    cores = O.get_threads()
    # a bounded sample: at most the work of 131,072 points against 10,000 centroids of 1,024 dimensions
    m = max(1024, min(n, args.cpu_assign_points, int(2.7e12 / (2.0 * k * d))))
    Xh = dX.download(m)
    ok = O.KMeans(k, d, sampling_fraction=1.0, suppress_warnings=1)
    cpu_assign_s = None
    for _ in range(2):  # the host share of the box is noisy: the better of two runs
        t0 = time.perf_counter()
        oa = ok.assign(Xh, centroids)
        took = time.perf_counter() - t0
        cpu_assign_s = took if cpu_assign_s is None else min(cpu_assign_s, took)
    agree = float(np.mean(oa == gpu_assign[:m]))
    cpu = {"value": round(m / cpu_assign_s, 1), "unit": "points/s", "cores": int(cores), "kind": "port",
           "sample": f"Assign of the first {m} of the {n} points against the same {k} centroids, best of two runs "
                     f"{cpu_assign_s:.2f} s, oracle built with g++ -O3 -march=x86-64-v3 -fopenmp, "
                     f"BLAS={os.path.basename(O.blas_name())}",
           "assign_agreement_with_gpu": agree}
    mt = min(n, args.cpu_train_points)
    if mt >= 4 * k and not no_train:
        # Train on a prefix large enough to keep the points-per-cluster regime in range; one iteration (rotation + the
        # exact search) and three (two pruned ones more), so that the two kinds of iteration are told apart
        Xt = Xh[:mt] if mt <= m else dX.download(mt)
        times = {}
        for iters in (1, 3):
            okt = O.KMeans(k, d, iters=iters, sampling_fraction=1.0, early_termination=0, suppress_warnings=1)
            t0 = time.perf_counter()
            okt.train(Xt)
            times[iters] = time.perf_counter() - t0
        cpu["train_sample"] = (f"Train on the first {mt} points, k={k}: 1 iteration (rotation + exact search + update) "
                               f"{times[1]:.2f} s, 3 iterations {times[3]:.2f} s")
        cpu["train_s_end_to_end_on_sample"] = round(times[3], 3)
        cpu["train_s_first_iteration_with_rotation_on_sample"] = round(times[1], 3)
        cpu["train_s_per_pruned_iter_on_sample"] = round((times[3] - times[1]) / 2.0, 3)
        cpu["train_sample_points"] = int(mt)
    return cpu


def compact(result):
    """What `other_configs` keeps of a configuration's result."""
    t = result["train"] or {}
    return {"workload": result["config"]["workload"], "assign_points_per_s": result["value"],
            "assign_ms": result["ms_per_step"], "assign_roofline_frac": result["roofline"]["frac"],
            "train_s_end_to_end": t.get("train_s_end_to_end"),
            "train_s_end_to_end_second_object": t.get("train_s_end_to_end_second_object"),
            "iters": t.get("iters"), "partial_d": t.get("partial_d"), "not_pruned_pct": t.get("not_pruned_pct"),
            "pruned_vs_exact_agreement": t.get("pruned_vs_exact_agreement"),
            "stages": {nm: dict({"ms": s["ms"], "frac": s["frac"], "bound": s["bound"]},
                                **({"frac_is": s["frac_is"]} if "frac_is" in s else {}))
                       for nm, s in t.get("stages", {}).items()}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", choices=sorted(CONFIGS), default=None)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--n", type=int, default=None)
    ap.add_argument("--d", type=int, default=None)
    ap.add_argument("--k", type=int, default=None)
    ap.add_argument("--train-iters", type=int, default=None)
    ap.add_argument("--cpu-assign-points", type=int, default=131072)
    ap.add_argument("--cpu-train-points", type=int, default=262144)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-train", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="headline run without the agreement, AssignTrainingPoints and other_configs legs")
    ap.add_argument("--host-pointers", action="store_true",
                    help="run the transfer-inclusive leg (Assign and Train called with host pointers) also where the "
                         "host copy of the points exceeds 16 GB")
    ap.add_argument("--no-host-pointers", action="store_true",
                    help="skip the transfer-inclusive leg, so that a kernel trace of the command holds the resident "
                         "launches only")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain row-copy kernel of known size (1 GiB read + 1 GiB write) three times; "
                         "used to scale the FETCH_SIZE / WRITE_SIZE hardware counters")
    ap.add_argument("--walk-kernel", type=int, default=0,
                    help="skm_ctx_set_walk_kernel for every Train of the run (0 automatic, 1 one point per wavefront, "
                         "2 / 3 four / eight points pooled per wavefront); for profiles that compare the walks")
    ap.add_argument("--walk-launches", type=int, default=1,
                    help="skm_ctx_set_walk_launches for every Train of the run (the pooled walk split into that many "
                         "launches over ranges of centroid batches); for the profile that compares one launch with one per batch")
    ap.add_argument("--n-threads", type=int, default=None,
                    help="hierarchical configurations: number of mesoclusters fine-clustered concurrently (the config's "
                         "n_threads; default 8 helper objects with a host thread and a stream each)")
    ap.add_argument("--print-kernel-hash", action="store_true",
                    help="print kernel_sources_hash() of this tree (what MEASURED_SOURCES_HASH must hold) and exit")
    args = ap.parse_args()
    if args.print_kernel_hash:
        print(kernel_sources_hash())
        return
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

    headline = args.config is None and args.n is None and args.d is None and args.k is None
    name = args.config or "C2"
    cn, cd, ck, citers, hierarchical, generator = CONFIGS[name]
    n, d, k = args.n or cn, args.d or cd, args.k or ck
    train_iters = args.train_iters if args.train_iters is not None else citers
    host_leg = not args.no_host_pointers and (args.host_pointers or 4.0 * n * d <= 16e9)
    extras = headline and not args.no_extras
    out = run_config(args, name, n, d, k, train_iters, hierarchical, generator, args.steps, args.warmup,
                     with_cpu=not args.no_cpu, with_host=host_leg, with_extras=extras)
    if extras and not args.no_train:
        # the other two flat configurations, briefly: Assign and the Train stage table (no CPU or transfer legs)
        others = {}
        for other in ("C1", "C5"):
            on, od, okk, oiters, ohier, ogen = CONFIGS[other]
            _capi.check(_capi.load().skm_device_cache_trim(0))
            others[other] = compact(run_config(args, other, on, od, okk, oiters, ohier, ogen, steps=2, warmup=1,
                                               with_cpu=False, with_host=False, with_extras=False, with_agreement=True))
        out["other_configs"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
