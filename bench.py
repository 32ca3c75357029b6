#!/usr/bin/env python3
"""Benchmark of the boosting loop on one MI355X.

A step is one boosting iteration (gradients, the trees of the round, prediction update, training metric);
data, cut points and the bin matrix are resident in HBM before the timed region starts (the reference's
"training time" span, src/thundergbm/trainer.cu:42-50, also excludes them). The K timed steps are one
boosting call of K rounds, as in a training run, bracketed by device synchronisations. Prints one JSON line.

The default workload is benchmark configuration 2 (10M x 28 dense, binary:logistic, depth 8, 255 bins), the one
the headline metric is quoted on; --config 1, 3, 4, 5 time the other configurations the same way.
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

# objective, depth, bins, learning rate, trees of the configuration, histogram kernel
CONFIGS = {
    1: dict(objective="reg:linear", depth=6, max_num_bin=255, learning_rate=0.1, n_trees=40,
            kernel="k_hist_dense", name="config 1: %d rows x %d dense features, reg:linear, depth %d, 255 bins"),
    2: dict(objective="binary:logistic", depth=8, max_num_bin=255, learning_rate=0.1, n_trees=100,
            kernel="k_hist_dense", name="config 2: %d rows x %d dense features, binary:logistic, depth %d, 255 bins"),
    3: dict(objective="reg:linear", depth=6, max_num_bin=255, learning_rate=0.1, n_trees=50,
            kernel="k_hist_dense", name="config 3: %d rows x %d dense features (5%% heavy-tailed), reg:linear, depth %d, 255 bins"),
    4: dict(objective="binary:logistic", depth=8, max_num_bin=63, learning_rate=0.1, n_trees=100,
            kernel="sparse histogram kernels", name="config 4: %d rows x %d features CSR (~40 per row, Zipf), binary:logistic, depth %d, 63 bins"),
    5: dict(objective="multi:softmax", depth=8, max_num_bin=255, learning_rate=0.1, n_trees=100,
            kernel="k_hist_dense", name="config 5: %d rows x %d features, 8-class softmax (8 trees per step), depth %d, 255 bins"),
}


KERNEL_SOURCES = ["thundergbm_amd/csrc/tree_kernels.hip", "thundergbm_amd/csrc/sparse_kernels.hip",
                  "thundergbm_amd/csrc/kernel_common.h", "thundergbm_amd/csrc/trainer.hip",
                  "thundergbm_amd/csrc/device_api.h"]
# counter summary of a configuration's histogram kernels under profiles/
PMC_SUMMARY = {1: "none", 2: "k_hist_dense_config2_pmc.txt", 3: "k_hist_dense_config3_pmc.txt",
               4: "sparse_level_pass_config4_pmc.txt", 5: "k_hist_dense_config5_pmc.txt"}


def kernel_sources_sha1():
    """Fingerprint of the histogram kernels' sources; the counter summaries under profiles/ carry the one they
    were measured with."""
    import hashlib
    h = hashlib.sha1()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def traffic_from_profile(config):
    """HBM bytes per histogram launch (for the sparse level pass: per level, i.e. its table, chunk-sum and sorted
    kernels together) from the committed rocprofv3 --pmc summary of this configuration (FETCH_SIZE
    and WRITE_SIZE runs, calibrated against a plain copy kernel), with where it comes from. The figure is only
    passed on when the summary was measured with the kernel sources as they are now; else it would be stale."""
    rel = os.path.join("profiles", PMC_SUMMARY[config])
    value = sha = None
    try:
        for line in open(os.path.join(ROOT, rel)):
            if line.startswith("traffic_bytes_per_launch:"):
                value = float(line.split(":")[1])
            if line.startswith("kernel_sources_sha1:"):
                sha = line.split(":")[1].strip()
    except OSError:
        return None, None
    if value is None:
        return None, None
    if sha != kernel_sources_sha1():
        return None, "%s was measured with other kernel sources (%s): not used" % (rel, sha)
    return value, "%s (kernel sources %s)" % (rel, sha[:12])


def make_data(config, rows):
    import datasets as D
    if config == 1:
        X, y = D.config1(rows or 10_000, 8, seed=0)
    elif config == 2:
        X, y = D.config2(rows or 10_000_000, seed=1)
    elif config == 3:
        X, y = D.config3(rows or 500_000, 2000, seed=2)
    elif config == 5:
        X, y = D.config5(rows or 1_000_000, seed=4)
    else:
        val, rp, col, y = D.config4(rows or 2_000_000, 100_000, 40, seed=3)
        return val, rp, col, y, len(rp) - 1, 100_000
    n, F = X.shape
    val, rp, col = D.dense_to_csr(X)
    return val, rp, col, y, n, F


def small_data_figures(T, torch):
    """Milliseconds per tree on the two small workloads of the reference (its CPU-runnable configuration 1 and its
    quick-start file): a tree there is a chain of dependent launches over a few thousand rows, so the figure is
    launch latency, not bandwidth. One training call of 40 trees each, after a warm-up session."""
    import datasets as D
    out = {}
    X, y = D.config1(10_000, 8, seed=0)
    cases = {"config1_10000x8_depth6": (D.dense_to_csr(X), y, dict(objective="reg:linear", learning_rate=0.1)),
             "a1a_1605x119_depth6": (None, None, dict(objective="reg:linear", learning_rate=1.0))}
    val, rp, col, ya = D.read_libsvm(D.A1A)
    cases["a1a_1605x119_depth6"] = ((val, rp, col), ya, cases["a1a_1605x119_depth6"][2])
    for name, ((v, r, c), yy, kw) in cases.items():
        for rep in range(2):  # the first session warms the code paths up
            s = T.Session(v, r, c, yy, depth=6, n_trees=40, max_num_bin=255, verbose=0, **kw)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            s.boost(40)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            s.close()
        out[name + "_ms_per_tree"] = round(dt / 40 * 1e3, 4)
    return out


def predict_figures(T, s, val, rp, col, lr, n_trees=40):
    """Wall time of the C ABI's prediction call on the training rows (host CSR in, raw scores out: the upload is
    inside; the traversal kernel's own time is in the kernel trace under profiles/)."""
    import ctypes as C
    L = T.load()
    model = C.c_void_p(s.export_model())
    out = np.zeros(s.n, np.float32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    best = None
    for _ in range(2):
        out[:] = 0
        t0 = time.perf_counter()
        L.tgbm_predict_raw(s.n, p(val), p(rp), p(col), model, n_trees, 1, lr, s.base_score, p(out))
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    L.model_free(C.byref(model))
    return {"rows": int(s.n), "trees": n_trees, "wall_s_host_buffers": round(best, 4),
            "rows_per_s": round(s.n / best, 1), "mean_raw_score": float(out.mean())}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", type=int, default=2, choices=sorted(CONFIGS))
    ap.add_argument("--rows", type=int, default=0, help="rows of the synthetic matrix (0 = the configuration's own)")
    ap.add_argument("--depth", type=int, default=0, help="tree depth (0 = the configuration's own)")
    ap.add_argument("--profile-steps", type=int, default=5)
    ap.add_argument("--cpu-steps", type=int, default=2, help="boosting iterations of the CPU baseline (0 = skip)")
    ap.add_argument("--full-run", type=int, default=1,
                    help="config 2: also time one training call of all the configuration's trees (0 = skip)")
    ap.add_argument("--small-data", type=int, default=1,
                    help="config 2: also time the two small workloads, 40 trees each (0 = skip, e.g. under a profiler)")
    ap.add_argument("--predict", type=int, default=1,
                    help="config 2 with --full-run: also time tgbm_predict_raw (host buffers in, scores out) on all rows "
                         "with 40 of the trees (0 = skip)")
    ap.add_argument("--calibration-copy-mb", type=int, default=0,
                    help="also run 3 launches of a plain copy kernel of this many MiB (profiler counter calibration)")
    ap.add_argument("--cpu-rows", type=int, default=0, help="rows of the CPU baseline sample (0 = a default per config)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build trains on one GPU; --gpus %d is not supported (no multi-GPU path exists)"
              % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch  # device synchronisation only; the library manages its own HBM buffers
    import thundergbm_amd as T

    assert torch.cuda.is_available(), "no GPU visible"
    T.load()
    cfg = CONFIGS[args.config]
    depth = args.depth or cfg["depth"]
    t0 = time.perf_counter()
    val, rp, col, y, n, F = make_data(args.config, args.rows)
    t_gen = time.perf_counter() - t0
    kw = dict(depth=depth, objective=cfg["objective"], learning_rate=cfg["learning_rate"],
              max_num_bin=cfg["max_num_bin"], verbose=0)
    total_rounds = args.warmup + args.steps + args.profile_steps
    t0 = time.perf_counter()
    s = T.Session(val, rp, col, y, n_trees=total_rounds, **kw)
    t_prep = time.perf_counter() - t0
    if args.warmup:
        s.boost(args.warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    s.boost(args.steps)  # K rounds enqueued back to back; returns after the GPU finished the last one
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    value = args.steps / dt

    roofline = None
    phases = None
    if args.profile_steps > 0:
        # (profiled iterations follow the timed ones: HIP events between the stages would perturb the timed region)
        s.set_profiling(True)
        s.boost(args.profile_steps)
        prof = s.profile()
        phases = s.phase_profile()
        s.set_profiling(False)
        if prof["launches"] > 0 and prof["hist_ms"] > 0:
            achieved = prof["bytes"] / (prof["hist_ms"] * 1e-3) / 1e9
            full_size = args.rows == 0 and args.depth == 0
            traffic, source = traffic_from_profile(args.config) if full_size else (None, None)
            roofline = {"bound": "hbm", "kernel": cfg["kernel"], "achieved": round(achieved, 2), "peak": 8000.0,
                        "unit": "GB/s", "frac": round(achieved / 8000.0, 4),
                        "traffic": traffic, "traffic_source": source,
                        "bytes_per_launch": round(prof["bytes"] / prof["launches"], 1),
                        "avg_launch_us": round(prof["hist_ms"] * 1e3 / prof["launches"], 2),
                        "hist_ms_per_step": round(prof["hist_ms"] / args.profile_steps, 4),
                        "rows_built_per_step": prof["rows_built"] // args.profile_steps,
                        "measured_on": "the %d iterations that follow the timed ones (iterations %d-%d of the run), "
                                       "HIP events on the trainer's stream around every stage" % (
                                           args.profile_steps, args.warmup + args.steps + 1, total_rounds)}
            for part in ("root", "below_root"):  # the root level streams its rows, the levels below gather theirs
                h = phases["hist"][part]
                if h["launches"] > 0 and h["ms"] > 0:
                    gbs = h["bytes"] / (h["ms"] * 1e-3) / 1e9
                    roofline[part] = {"launches": h["launches"], "bytes_per_launch": round(h["bytes"] / h["launches"], 1),
                                      "avg_launch_us": round(h["ms"] * 1e3 / h["launches"], 2),
                                      "achieved": round(gbs, 2), "frac": round(gbs / 8000.0, 4)}
    metric_log = s.metric_log()
    reorders = s.info("reorders_done")
    s.close()

    aux = {"phase_ms": None if phases is None else
           {k: round(v / max(1, phases["rounds"]), 4) for k, v in phases["phase_ms"].items()},
           "phase_ms_note": "milliseconds per iteration of the profiled iterations, by stage; their sum exceeds ms_per_step "
                            "by what the event records between the stages cost",
           "data_gen_s": round(t_gen, 2), "prep_s_upload_cuts_bins": round(t_prep, 3),
           "train_metric_last": float(metric_log[-1]) if len(metric_log) else None,
           "row_reorderings_before_or_inside_the_timed_steps": reorders}
    if args.config == 2 and args.full_run and args.rows == 0:
        # the whole configuration as one training call: every row re-ordering pass is inside the timed span
        s = T.Session(val, rp, col, y, n_trees=cfg["n_trees"], **kw)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        s.boost(cfg["n_trees"])
        torch.cuda.synchronize()
        t_full = time.perf_counter() - t0
        aux["iters_per_s_100_trees"] = round(cfg["n_trees"] / t_full, 2)
        aux["reorderings_in_100_trees"] = s.info("reorders_done")
        if args.predict:
            aux["predict"] = predict_figures(T, s, val, rp, col, cfg["learning_rate"])
        s.close()
    if args.config == 2 and args.small_data and args.rows == 0:
        aux["small_data"] = small_data_figures(T, torch)
    if args.calibration_copy_mb > 0:
        import ctypes
        cal = ctypes.CDLL(os.path.join(ROOT, "thundergbm_amd", "libtgbm_calibration.so"))
        cal.tgbm_calibration_copy.argtypes = [ctypes.c_size_t, ctypes.c_int]
        cal.tgbm_calibration_copy.restype = None
        cal.tgbm_calibration_copy(args.calibration_copy_mb << 20, 3)

    cpu = None
    if args.cpu_steps > 0:
        import oracle_lib as O
        default_rows = {1: n, 2: n, 3: 25_000, 4: 200_000, 5: 200_000}[args.config]
        m = min(n, args.cpu_rows if args.cpu_rows > 0 else default_rows)
        crp = rp[: m + 1]
        nnz = int(crp[-1])
        o = O.Oracle(val[:nnz], crp, col[:nnz], y[:m], depth=depth, n_trees=args.cpu_steps, objective=cfg["objective"],
                     learning_rate=cfg["learning_rate"], max_num_bin=cfg["max_num_bin"]).prepare()
        t0 = time.perf_counter()
        o.boost(args.cpu_steps)
        cdt = time.perf_counter() - t0
        cpu_value = args.cpu_steps / cdt * (m / n)  # iterations/s scaled to the full row count
        cpu = {"value": round(cpu_value, 4), "unit": "boosting iters/s", "cores": O.lib().orc_num_threads(),
               "kind": "port",
               "sample": "%d boosting iterations of the OpenMP oracle on the first %d of %d rows (scaled linearly "
                         "in rows), boost loop only" % (args.cpu_steps, m, n)}

    out = {
        "metric": "boosting iters/sec (depth %d, %d bins, 1 GPU)" % (depth, cfg["max_num_bin"]), "value": round(value, 3),
        "unit": "boosting iters/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": cfg["name"] % (n, F, depth), "rows": n, "features": F, "depth": depth,
                   "max_num_bin": cfg["max_num_bin"], "learning_rate": cfg["learning_rate"],
                   "objective": cfg["objective"]},
        "roofline": roofline, "cpu_baseline": cpu, "aux": aux,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
