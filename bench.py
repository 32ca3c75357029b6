#!/usr/bin/env python3
"""Benchmark of the boosting loop on one MI355X.

A step is one boosting iteration (gradients, one depth-8 tree, prediction update, training metric)
on the 10M x 28 dense binary-logistic configuration with 255 bins; data, cut points and the bin matrix
are resident in HBM before the timed region starts (the reference's "training time" span,
src/thundergbm/trainer.cu:42-50, also excludes them). Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import numpy as np  # noqa: E402


def measured_traffic_per_launch():
    """HBM bytes per k_hist_dense launch from the committed rocprofv3 --pmc summary (FETCH_SIZE and
    WRITE_SIZE runs, calibrated against a plain copy kernel); None when the summary is absent."""
    path = os.path.join(ROOT, "profiles", "k_hist_dense_config2_pmc.txt")
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch:"):
                return float(line.split(":")[1])
    except OSError:
        pass
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--rows", type=int, default=10_000_000)
    ap.add_argument("--depth", type=int, default=8)
    ap.add_argument("--profile-steps", type=int, default=5)
    ap.add_argument("--cpu-steps", type=int, default=2, help="boosting iterations of the CPU baseline (0 = skip)")
    ap.add_argument("--calibration-copy-mb", type=int, default=0,
                    help="also run 3 launches of a plain copy kernel of this many MiB (profiler counter calibration)")
    ap.add_argument("--cpu-rows", type=int, default=0, help="rows of the CPU baseline sample (0 = all rows)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build trains on one GPU; --gpus %d is not supported (no multi-GPU path exists)"
              % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch  # device synchronisation only; the library manages its own HBM buffers
    import datasets as D
    import thundergbm_amd as T

    assert torch.cuda.is_available(), "no GPU visible"
    T.load()
    t0 = time.perf_counter()
    X, y = D.config2(args.rows, seed=1)
    val, rp, col = D.dense_to_csr(X)
    n, F = X.shape
    del X
    t_gen = time.perf_counter() - t0
    total_rounds = args.warmup + args.steps + args.profile_steps
    t0 = time.perf_counter()
    s = T.Session(val, rp, col, y, depth=args.depth, n_trees=total_rounds, objective="binary:logistic",
                  learning_rate=0.1, max_num_bin=255, verbose=0)
    t_prep = time.perf_counter() - t0
    for _ in range(args.warmup):
        s.boost(1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        s.boost(1)  # returns after the GPU finished the iteration
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    value = args.steps / dt

    roofline = None
    if args.profile_steps > 0:
        s.set_profiling(True)
        for _ in range(args.profile_steps):
            s.boost(1)
        prof = s.profile()
        s.set_profiling(False)
        if prof["launches"] > 0 and prof["hist_ms"] > 0:
            achieved = prof["bytes"] / (prof["hist_ms"] * 1e-3) / 1e9
            roofline = {"bound": "hbm", "kernel": "k_hist_dense", "achieved": round(achieved, 2), "peak": 8000.0,
                        "unit": "GB/s", "frac": round(achieved / 8000.0, 4),
                        "traffic": measured_traffic_per_launch() if args.rows == 10_000_000 else None,
                        "bytes_per_launch": round(prof["bytes"] / prof["launches"], 1),
                        "avg_launch_us": round(prof["hist_ms"] * 1e3 / prof["launches"], 2),
                        "hist_ms_per_tree": round(prof["hist_ms"] / args.profile_steps, 4),
                        "rows_built_per_tree": prof["rows_built"] // args.profile_steps}
    metric_log = s.metric_log()
    s.close()
    if args.calibration_copy_mb > 0:
        T.load().tgbm_calibration_copy(args.calibration_copy_mb << 20, 3)

    cpu = None
    if args.cpu_steps > 0:
        import oracle_lib as O
        m = args.cpu_rows if args.cpu_rows > 0 else n
        crp = rp[: m + 1]
        nnz = int(crp[-1])
        o = O.Oracle(val[:nnz], crp, col[:nnz], y[:m], depth=args.depth, n_trees=args.cpu_steps,
                     objective="binary:logistic", learning_rate=0.1, max_num_bin=255).prepare()
        t0 = time.perf_counter()
        o.boost(args.cpu_steps)
        cdt = time.perf_counter() - t0
        cpu_value = args.cpu_steps / cdt * (m / n)  # iterations/s scaled to the full row count
        cpu = {"value": round(cpu_value, 4), "unit": "boosting iters/s", "cores": O.lib().orc_num_threads(),
               "kind": "port",
               "sample": "%d boosting iterations of the OpenMP oracle on %d of %d rows (linear in rows), "
                         "boost loop only" % (args.cpu_steps, m, n)}

    out = {
        "metric": "boosting iters/sec (depth 8, 255 bins, 1 GPU)", "value": round(value, 3),
        "unit": "boosting iters/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "config 2: %d rows x %d dense features, binary:logistic, depth %d, 255 bins"
                               % (n, F, args.depth),
                   "rows": n, "features": F, "depth": args.depth, "max_num_bin": 255, "learning_rate": 0.1},
        "roofline": roofline, "cpu_baseline": cpu,
        "aux": {"data_gen_s": round(t_gen, 2), "prep_s_upload_cuts_bins": round(t_prep, 3),
                "train_error_last": float(metric_log[-1]) if len(metric_log) else None},
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
