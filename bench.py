#!/usr/bin/env python3
"""Benchmark of the tree-learner path on one MI355X.

Default workload (configuration 2 of the benchmark plan): LBRegressor squared error,
Tree(max_depth=8, split_samples=256), X 10,000,000 x 100 f32. One step is one
boosting round: gradient step, BuildTreeTask, PredictTask of the new tree and
the prediction update, all with inputs resident in HBM.

Prints ONE JSON line. `roofline` describes the histogram kernels (HIP events on
the stream of the call, summed over the timed rounds); `cpu_baseline` is the
restated CPU variant of the reference timed on the host cores of this machine
on a row sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "legate-boost_amd"))
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--config", type=int, default=2, choices=[1, 2, 3, 4, 5])
    ap.add_argument("--rows", type=int, default=0, help="override the number of rows (0 = the configuration's)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--reference-flow", action="store_true",
                    help="update the training predictions with a PredictTask per round (as the reference loop does) instead of the row->leaf map that BuildTreeTask can return")
    ap.add_argument("--hist-cache-bytes", type=int, default=0,
                    help="bytes of histograms BuildTreeTask keeps (0 = the reference's 1e9, build_tree.cu:1004); a larger "
                         "cache builds the same trees and lets deeper levels derive siblings by subtraction")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--only-timed", action="store_true",
                    help="run the warm-up and the timed rounds only (no per-class breakdown rounds, no rounds in the other "
                         "flow, no CPU baseline, no other configurations): what a profiler run wants, every launch of "
                         "the process then belongs to the rounds the printed figures describe")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="default run only: leave out the short legs of configurations 3, 4 and 5 that follow the headline")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain 4 GiB device copy five times (to scale rocprofv3's FETCH_SIZE / "
                         "WRITE_SIZE counters against a kernel of known traffic)")
    return ap.parse_args()


def cpu_baseline_build(X_sample, y_sample, max_depth, split_samples, lr, full_rows, seconds, n_outputs_classes=0):
    """Rounds/s of the restated CPU variant of the reference on a row sample, at P = the host threads of this
    GPU's share of the machine and at P = 1, each scaled to the full row count (the work of a round is linear
    in the rows: binning, histograms and the position update all walk them once per level)."""
    import numpy as np

    import cpu_variant_lib as cv

    # a one-GPU box gives its job 16 host threads whatever os.cpu_count() reports
    cores = max(1, min(16, os.cpu_count() or 1))
    n = X_sample.shape[0]
    k = n_outputs_classes or 1

    def run(n_threads, budget, min_rounds):
        pred = np.zeros((n, k)) if n_outputs_classes else np.full((n, 1), y_sample.mean())
        rounds = 0
        t0 = time.perf_counter()
        while True:
            if n_outputs_classes:
                e = np.exp(pred - pred.max(axis=1, keepdims=True))
                p = e / e.sum(axis=1, keepdims=True)
                g = p.copy()
                g[np.arange(n), y_sample.astype(np.int64)] -= 1.0
                g *= lr
                h = np.maximum(p * (1 - p), 1e-8)
            else:
                g = (pred - y_sample.reshape(-1, 1)) * lr
                h = np.ones((n, 1))
            leaf, feat, split, gain, hess = cv.build_tree(X_sample, g, h, max_depth=max_depth,
                                                          split_samples=split_samples, seed=rounds, n_threads=n_threads)
            pred += cv.predict(X_sample, [(leaf, feat, split)], k, n_threads=n_threads)
            rounds += 1
            dt = time.perf_counter() - t0
            if rounds >= min_rounds and dt >= budget:
                return rounds, dt

    rounds_p, dt_p = run(cores, seconds * 0.4, 2)
    rounds_1, dt_1 = run(1, 0.0, 1)
    scale = n / full_rows
    return {
        "value": rounds_p / dt_p * scale,
        "unit": "rounds/s",
        "cores": cores,
        "kind": "port",
        "sample": ("all %d rows" % n if n == full_rows else "first %d of %d rows" % (n, full_rows))
                  + "; %d threads: %d rounds in %.1f s; 1 thread: %d round(s) in %.1f s" % (cores, rounds_p, dt_p, rounds_1, dt_1)
                  + ("" if n == full_rows else "; both scaled to the full rows by %d/%d (a round's work is linear in "
                                               "the rows)" % (n, full_rows)),
        "single_thread": {"value": rounds_1 / dt_1 * scale, "unit": "rounds/s", "cores": 1},
        "host_cpu_count": os.cpu_count(),
    }


def source_tag():
    """Identifies the kernels a profile was taken on: the first 12 hex digits of the SHA-256 of lbt_histogram.hip."""
    import hashlib

    path = os.path.join(ROOT, "legate-boost_amd", "csrc", "lbt_histogram.hip")
    return hashlib.sha256(open(path, "rb").read()).hexdigest()[:12]


def measured_traffic(workload, rows, features):
    """HBM bytes per launch from rocprofv3 counter runs of this command, kept as text under profiles/.

    Lines of the form `<kernel> traffic_bytes_per_launch=<number> workload=<name> rows=<n> features=<f>
    source=<tag>`; only those taken on the same workload and on the kernel source as it is now apply
    (a counter run cannot be made from inside this program). Returns {} when none do."""
    out = {}
    path = os.path.join(ROOT, "profiles", "hbm_traffic_%s.txt" % workload)
    if not os.path.exists(path):
        return out
    tag = source_tag()
    for line in open(path):
        parts = line.split()
        if len(parts) < 2 or "traffic_bytes_per_launch=" not in line:
            continue
        kv = dict(p.split("=", 1) for p in parts[1:] if "=" in p)
        if (kv.get("workload") == workload and int(kv.get("rows", -1)) == rows
                and int(kv.get("features", -1)) == features and kv.get("source") == tag):
            out[parts[0]] = float(kv["traffic_bytes_per_launch"])
            if "algorithmic_bytes_per_launch" in kv:
                # the algorithmic bytes of the very launches the counters were read on
                out[parts[0] + ":ratio"] = float(kv["traffic_bytes_per_launch"]) / float(kv["algorithmic_bytes_per_launch"])
    return out


def bench_training(args, cfg=None, steps=None, warmup=None, light=False):
    """One training configuration. light: a short leg that follows the headline in the default run:
    the timed rounds only (no second flow, no per-class breakdown, no CPU baseline) and a compact
    result. args.only_timed runs the same rounds and returns the full result."""
    compact = light
    light = light or args.only_timed
    import numpy as np
    import torch

    from lbtree import _lib, datasets, ops

    cfg = args.config if cfg is None else cfg
    steps = args.steps if steps is None else steps
    warmup = args.warmup if warmup is None else warmup
    lr = 0.1
    n_classes = 0
    rows_override = 0 if light else args.rows
    if cfg == 1:
        Xh, yh = datasets.config1()
        X, y = ops.as_device(Xh), ops.as_device(yh, torch.float64)
        depth, S, name = 6, 256, "cfg1"
    elif cfg == 2:
        rows = rows_override or 10_000_000
        X, y = datasets.config2(rows, 100)
        depth, S, name = 8, 256, "cfg2"
    elif cfg == 3:
        rows = rows_override or 2_000_000
        X, y = datasets.config3(rows, 200, 8)
        depth, S, name, n_classes = 8, 256, "cfg3", 8
    else:
        rows = rows_override or 1_000_000
        X, y = datasets.config4(rows, 50)
        depth, S, name = 12, 512, "cfg4"
    n, f = X.shape
    k = n_classes or 1
    rs = np.random.RandomState(0)
    if n_classes:
        prob = torch.bincount(y.to(torch.int64), minlength=k).to(torch.float64) / n
        pred = torch.log(prob).reshape(1, -1).repeat(n, 1).contiguous()
        label = y.to(torch.int64)
        ar = torch.arange(n, device=X.device)
    else:
        pred = torch.full((n, 1), float(y.mean()), dtype=torch.float64, device=X.device)
        yc = y.reshape(-1, 1)

    gh = (torch.empty_like(pred), torch.empty_like(pred))
    sums = torch.empty((2, int(_lib.lib.lbt_abs_sum_chunks(n, k))), dtype=torch.float64, device=X.device)

    def one_round(reference_flow=args.reference_flow, cache=args.hist_cache_bytes):
        seed = int(rs.randint(0, 2**31))
        if reference_flow:
            # the caller's steps as separate array operations and a traversal of X per round
            if n_classes:
                p = torch.softmax(pred, dim=1)
                g = p.clone()
                g[ar, label] -= 1.0
                g *= lr
                h = torch.clamp(p * (1.0 - p), min=1e-8)
            else:
                g = (pred - yc) * lr
                h = torch.ones_like(pred)
            r = ops.build_tree(X, g, h, max_depth=depth, split_samples=S, seed=seed, hist_cache_bytes=cache)
            pred.add_(ops.predict(X, [(r.leaf_value, r.feature, r.split_value)], k))
        else:
            # gradient step in one pass, which also leaves the first level of the quantiser's absolute
            # sums; the prediction update takes the rows' leaves from the build: same values as
            # PredictTask on the training rows (checked bit for bit in the tests)
            g, h, part = ops.weighted_gradient("log_loss" if n_classes else "squared_error", y if n_classes else yc,
                                               pred, None, lr, out=gh, sums=sums)
            r = ops.build_tree(X, g, h, max_depth=depth, split_samples=S, seed=seed, row_leaf=True, wait=False,
                               abs_sum_chunks=part, hist_cache_bytes=cache)
            ops.add_leaf_values(pred, r.leaf_value, r.row_leaf)
        return r

    def loss():
        if n_classes:
            return float(torch.nn.functional.cross_entropy(pred, label))
        return float(((pred[:, 0] - y) ** 2).mean())

    loss0 = loss()
    for _ in range(warmup):
        one_round()
    torch.cuda.synchronize()
    # the timed rounds carry HIP events around the two histogram-stage kernels only (18 events
    # per round); the per-class breakdown comes from two further, untimed rounds
    _lib.profile_reset()
    _lib.profile_enable(2)
    t0 = time.perf_counter()
    for _ in range(steps):
        one_round()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    prof = _lib.profile_get()
    loss1 = loss()
    _lib.profile_reset()
    prof_all = None
    other_rate = None
    other_steps = max(2, min(steps, 5))
    if not light:
        _lib.profile_enable(1)
        for _ in range(2):
            one_round()
        torch.cuda.synchronize()
        _lib.profile_enable(0)
        prof_all = _lib.profile_get()
        # the other flow of a round, in the same run and on the same model: the reference loop's own
        # steps (gradient as separate array operations, BuildTreeTask, PredictTask of the new tree)
        # when the timed rounds took the fused steps, and the other way round
        one_round(not args.reference_flow)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(other_steps):
            one_round(not args.reference_flow)
        torch.cuda.synchronize()
        other_rate = other_steps / (time.perf_counter() - t0)
    _lib.profile_enable(0)

    # The reference keeps 1e9 bytes of histograms (build_tree.cu:1004); a tree whose levels outgrow that
    # builds both children of every node from there on. With room for the whole tree (this GPU has 288 GB)
    # the same trees come out and every level derives siblings by subtraction: measured in the same run.
    whole_tree = (2 ** depth - 1) * k * f * S * 16
    whole_rate = None
    if whole_tree > (args.hist_cache_bytes or 1000000000) and not args.only_timed:
        one_round(cache=whole_tree)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(other_steps):
            one_round(cache=whole_tree)
        torch.cuda.synchronize()
        whole_rate = other_steps / (time.perf_counter() - t0)

    hist, binning = prof["histogram"], prof["binning"]
    elem = X.element_size()
    bin_bytes = 1 if S <= 256 else 2

    def gbps(byts, ms):
        return byts / (ms * 1e-3) / 1e9 if ms > 0 else 0.0

    # Algorithmic bytes of the histogram stage per level, the reference kernel's accounting:
    # every row of a built node reads its F feature values of X and its packed (grad, hess)
    # per output (gradients are quantised once per tree, 8 bytes per pair), every row of the
    # level's nodes its (node, row) pair, every built histogram is written once.
    stage_bytes = 0.0
    pair_extra = 0.0
    levels = []
    for d, lv in enumerate(prof["levels"]):
        # the library's own figure prices a feature value at its cached width; what is left of it
        # after the row terms are the histograms written
        own_extra = n * f * bin_bytes * steps if (d == 0 and depth >= 2) else 0.0  # feature-major copy, root launch
        written = max(0.0, lv["bytes"] - own_extra - lv["built_instances"] * (f * bin_bytes + k * 8.0 + 8.0))
        ref_bytes = lv["built_instances"] * (f * elem + k * 8.0) + lv["instances"] * 8.0 + written
        stage_bytes += ref_bytes
        pair_extra += lv["built_instances"] * k * 8.0
        levels.append({"level": d, "ms": lv["ms"] / steps, "built_rows": lv["built_instances"] / steps,
                       "built_nodes": lv["built_nodes"] / steps,
                       "GB_cached_bins": lv["bytes"] / steps / 1e9, "GBps_cached_bins": gbps(lv["bytes"], lv["ms"]),
                       "GB_reference_accounting": ref_bytes / steps / 1e9})
    stage_ms = hist["ms"] + binning["ms"]
    # the root launch's own-format bytes include the feature-major copy of the bins it writes for the
    # position updates; the histogram itself does not need it
    copy_bytes = n * f * bin_bytes * steps if depth >= 2 else 0.0
    traffic = measured_traffic(name, n, f)
    hist_achieved = gbps(hist["bytes"], hist["ms"])
    out = {
        "metric": "boosting rounds/sec + histogram HBM GB/s (% peak), 10M×100 depth 8" if cfg == 2
        else "boosting rounds/sec + histogram HBM GB/s (%% peak), %s" % name,
        "value": steps / dt,
        "unit": "rounds/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": dt / steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int64",
        "data": "synthetic",
        "config": {
            "workload": "%s: %s, Tree(max_depth=%d, split_samples=%d), lr %.1f, X %dx%d f32, K=%d"
                        % (name, "LBClassifier softmax" if n_classes else "LBRegressor squared error", depth, S, lr,
                           n, f, k),
            "rows": n, "features": f, "outputs": k, "max_depth": depth, "split_samples": S,
            "hist_cache_bytes": args.hist_cache_bytes or 1000000000,
            "loss_before": loss0, "loss_after": loss1,
            "prediction_update": "PredictTask" if args.reference_flow else "row->leaf map from BuildTreeTask",
            # a round as the reference loop runs it (legateboost.py:254-275): gradient arithmetic as
            # array operations, BuildTreeTask, PredictTask of the new tree; measured in this run
            "reference_flow_rounds_per_s": steps / dt if args.reference_flow else other_rate,
            "fused_flow_rounds_per_s": other_rate if args.reference_flow else steps / dt,
            # the fractions below are averages over these boosting rounds (0-based) of one model: the rows a
            # level has to build (the smaller child of every split) change from round to round, and with them
            # the share of the fixed root level in a tree's histogram bytes
            "rounds_timed": [warmup, warmup + steps - 1],
            "other_flow_steps": other_steps,
            "rounds_per_s_with_histograms_of_the_whole_tree_cached": whole_rate,
            "whole_tree_histogram_bytes": whole_tree,
        },
        # the kernel with the largest share of a round: the histogram kernel on cached bins,
        # priced on the bytes of its own input format (one or two bytes per feature value)
        "roofline": {
            "bound": "hbm",
            "achieved": hist_achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": hist_achieved / HBM_PEAK_GBS,
            "frac_without_feature_major_copy": gbps(hist["bytes"] - copy_bytes, hist["ms"]) / HBM_PEAK_GBS,
            "traffic": traffic.get("binned_histogram_kernel"),
            # measured HBM bytes over algorithmic bytes, both of the profiled run's own launches
            "traffic_over_algorithmic": traffic.get("binned_histogram_kernel:ratio"),
            "traffic_source": "profiles/hbm_traffic_%s.txt (rocprofv3 FETCH_SIZE / WRITE_SIZE), applies when its "
                              "source tag equals %s" % (name, source_tag()),
            # the histogram stage of a tree (binning pass + every histogram launch) against the bytes
            # the reference's histogram kernel has to move for the same levels, with the quantised
            # gradient pair of a row and output priced at 8 bytes (rounded once per tree here) and
            # at the 16 bytes of the two doubles the reference kernel reads
            "frac_reference_accounting": gbps(stage_bytes, stage_ms) / HBM_PEAK_GBS,
            "frac_reference_accounting_pairs_at_16_bytes": gbps(stage_bytes + pair_extra, stage_ms) / HBM_PEAK_GBS,
            "kernel": "binned_histogram_kernel",
            "launches": hist["launches"],
            "avg_launch_ms": hist["ms"] / max(1, hist["launches"]),
            "bytes_per_launch": hist["bytes"] / max(1, hist["launches"]),
            "levels": levels,
            # the other kernel of the histogram stage: the root pass that bins X into the cache
            "binning_kernel": {
                "kernel": "bin_rows_kernel", "launches": binning["launches"],
                "avg_launch_ms": binning["ms"] / max(1, binning["launches"]),
                "bytes_per_launch": binning["bytes"] / max(1, binning["launches"]),
                "achieved": gbps(binning["bytes"], binning["ms"]),
                "frac": gbps(binning["bytes"], binning["ms"]) / HBM_PEAK_GBS,
                "traffic": traffic.get("bin_rows_kernel"),
                "traffic_over_algorithmic": traffic.get("bin_rows_kernel:ratio"),
            },
            # the whole histogram stage of a tree (both kernels) against the bytes the
            # reference's histogram kernel would have to move for the same levels
            "stage_reference_accounting": {
                "kernels": "bin_rows_kernel + binned_histogram_kernel",
                "ms_per_tree": stage_ms / steps, "GB_per_tree": stage_bytes / steps / 1e9,
                "achieved": gbps(stage_bytes, stage_ms), "frac": gbps(stage_bytes, stage_ms) / HBM_PEAK_GBS,
            },
        },
    }
    if compact:
        r = out["roofline"]
        return {"workload": out["config"]["workload"], "value": out["value"], "unit": "rounds/s", "steps": steps,
                "warmup": warmup, "ms_per_step": out["ms_per_step"],
                "rounds_per_s_with_histograms_of_the_whole_tree_cached": whole_rate,
                "roofline": {"kernel": r["kernel"], "frac": r["frac"], "avg_launch_ms": r["avg_launch_ms"],
                             "frac_reference_accounting": r["frac_reference_accounting"],
                             "stage_ms_per_tree": stage_ms / steps, "stage_GB_per_tree_reference_accounting": stage_bytes / steps / 1e9,
                             "binning_ms": r["binning_kernel"]["avg_launch_ms"],
                             "level_ms": [lv["ms"] for lv in levels]}}
    if light:
        return out
    # two rounds after the timed ones, every kernel class bracketed by events
    out["kernel_ms_per_round"] = {c: prof_all[c]["ms"] / 2 for c in _lib.PROF_CLASSES}
    if not args.no_cpu_baseline:
        # config 2 (the headline) on all of its rows; the wider configurations on a row sample
        ns = n if cfg <= 2 else min(n, 500_000)
        out["cpu_baseline"] = cpu_baseline_build(X[:ns].cpu().numpy(), y[:ns].cpu().numpy(), depth, S, lr, n,
                                                 args.cpu_seconds, n_classes)
    return out


def bench_predict(args, steps=None, warmup=None, light=False):
    import numpy as np
    import torch

    import cpu_variant_lib as cv
    from lbtree import _lib, datasets, ops

    steps = args.steps if steps is None else steps
    warmup = args.warmup if warmup is None else warmup
    rows = (0 if light else args.rows) or 20_000_000
    trees = datasets.config5_ensemble()
    X = datasets.config5_X(rows)
    for _ in range(max(1, warmup)):
        ops.predict(X, trees, 1)
    torch.cuda.synchronize()
    _lib.profile_reset()
    _lib.profile_enable(True)
    t0 = time.perf_counter()
    for _ in range(steps):
        out_t = ops.predict(X, trees, 1)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    _lib.profile_enable(False)
    byts = rows * (64 * 4 + 8)
    achieved = byts * steps / dt / 1e9
    if light:
        return {"workload": "cfg5: PredictTask, 1000 trees of depth 8, X %dx64 f32, out f64" % rows,
                "value": rows * steps / dt, "unit": "rows/s", "steps": steps, "warmup": max(1, warmup),
                "ms_per_step": dt / steps * 1e3, "node_steps_per_s": rows * 8000 * steps / dt,
                "roofline": {"kernel": "predict_tile_kernel", "bound": "hbm", "frac": achieved / HBM_PEAK_GBS,
                             "limited_by": "lds"}}
    out = {
        "metric": "PredictTask rows/s, 1000 trees depth 8, 20M×64",
        "value": rows * steps / dt,
        "unit": "rows/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": dt / steps * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f64", "data": "synthetic",
        "config": {"workload": "cfg5: PredictTask, 1000 trees of depth 8, X %dx64 f32, out f64" % rows,
                   "rows": rows, "trees": 1000, "row_trees_per_s": rows * 1000 * steps / dt,
                   "node_steps_per_s": rows * 8000 * steps / dt},
        # X read once and the output written once are all the HBM bytes this path needs (achieved /
        # peak / frac price those); what bounds the kernel is the LDS: every node step of a wave
        # is two LDS reads (node, feature value), which the counters put at 8.2 cycles each
        # (4.2 of issue, 3.4 of bank conflicts; profiles/predict_tile_kernel_cfg5_*.txt), 17 of
        # the 17.5 cycles a CU spends per wave-level node step
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None, "kernel": "predict_tile_kernel",
                     "limited_by": "lds",
                     "lds": {"wave_level_node_steps": rows * 8000 / 64,
                             "cycles_per_wave_level_node_step_and_cu":
                                 dt / steps * 2.4e9 / (rows * 8000 / 64 / 256),
                             "lds_reads_per_node_step": 2.1, "lds_cycles_per_read_measured": 8.2,
                             "clock_assumed_GHz": 2.4}},
    }
    if not args.no_cpu_baseline and not args.only_timed:
        cores = max(1, min(16, os.cpu_count() or 1))
        ns = 20000
        Xs = X[:ns].cpu().numpy()
        th = [(a.cpu().numpy(), b.cpu().numpy(), c.cpu().numpy()) for a, b, c in trees]
        t0 = time.perf_counter()
        reps = 0
        while True:
            ref = cv.predict(Xs, th, 1, n_threads=cores)
            reps += 1
            if time.perf_counter() - t0 > args.cpu_seconds:
                break
        dtc = time.perf_counter() - t0
        assert np.abs(ref - out_t[:ns].cpu().numpy()).max() <= 1e-5
        out["cpu_baseline"] = {"value": ns * reps / dtc, "unit": "rows/s", "cores": cores, "kind": "port",
                               "sample": "first %d rows, all 1000 trees, %d repetitions in %.1f s" % (ns, reps, dtc)}
    return out


def copy_calibration():
    import torch

    n = 1 << 30
    a = torch.empty(n, dtype=torch.float32, device="cuda").normal_()
    b = torch.empty_like(a)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        b.copy_(a)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / 5
    print(json.dumps({"copy_bytes_read": n * 4, "copy_bytes_written": n * 4, "ms": dt * 1e3,
                      "GBps_read_plus_write": 2 * n * 4 / dt / 1e9}))


def main():
    args = parse()
    if args.copy_calibration:
        copy_calibration()
        return
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (no collectives are built)"
              % args.gpus, file=sys.stderr)
        sys.exit(2)
    out = bench_predict(args) if args.config == 5 else bench_training(args)
    if args.config == 2 and not args.no_other_configs and not args.rows and not args.only_timed:
        # the other benchmark configurations in the same run, a few rounds each, so that their
        # rates are on record beside the headline's (each can also be run alone with --config)
        out["other_configs"] = other_configs(args)
    print(json.dumps(out))


def _release_device_memory():
    import gc

    import torch

    from lbtree import ops

    ops._workspace.clear()
    gc.collect()
    torch.cuda.empty_cache()


def other_configs(args):
    legs = {}
    _release_device_memory()
    for cfg in (3, 4):
        legs["cfg%d" % cfg] = bench_training(args, cfg=cfg, steps=5, warmup=2, light=True)
        _release_device_memory()
    legs["cfg5"] = bench_predict(args, steps=2, warmup=1, light=True)
    _release_device_memory()
    return legs


if __name__ == "__main__":
    main()
