"""Headline benchmark: histogram tree growing at 10.5M rows x 28 features,
256 bins, max_depth 8, logistic objective, on one MI355X.

A step is one boosting iteration (one tree: gradients, 8 histogram levels,
split scans, row partitions, leaf update) over the resident, already quantised
matrix.  Prints ONE JSON line.

  value        row*feature histogram updates per second over the whole step
               (rows actually accumulated into histograms x 28 / step time)
  ms_per_step  milliseconds per tree
  roofline     the dominant kernel (fused partition + histogram pass):
               algorithmic bytes of its launches / their summed duration (HIP
               events on the builder's stream), against 8 TB/s
  cpu_baseline the CPU checker (oracle/, OpenMP) on a bounded row sample of the
               same workload, timed on this host
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MEASURED_FUSED_TRAFFIC_BYTES = 709.9e6  # 323.5 MiB fetched + 351.6 MiB written per launch
HBM_PEAK = 8.0e12  # bytes/s, MI355X


def make_workload(rows, features=28, seed=0):
    """BASELINE config 2: features 0-20 ~ N(0,1), 21-27 log-normal(0,1); label ~
    Bernoulli(sigmoid(sum of 8 random depth-3 stump products + 0.5 N(0,1) + bias)),
    bias chosen for about 53 % positives."""
    rng = np.random.default_rng(seed)
    X = rng.standard_normal(size=(rows, features), dtype=np.float32)
    X[:, 21:] = np.exp(X[:, 21:])
    score = np.zeros(rows, dtype=np.float32)
    for _ in range(8):
        prod = np.ones(rows, dtype=bool)
        for _ in range(3):
            f = int(rng.integers(0, features))
            t = float(np.quantile(X[:200000, f], rng.uniform(0.3, 0.7)))
            prod &= X[:, f] > t
        score += prod
    score += 0.5 * rng.standard_normal(size=rows, dtype=np.float32)
    score -= np.float32(score.mean() - 0.12)
    y = (rng.random(rows, dtype=np.float32) < 1.0 / (1.0 + np.exp(-score))).astype(np.float32)
    return X, y


def config(max_depth=8, hist_size=256):
    return {"objective": 1, "method": 1,
            "internals": {"hist_size": hist_size, "double_precision": True,
                          "use_hist_subtraction_trick": True, "upload_features": True},
            "tree": {"max_depth": max_depth, "eta": 0.1, "lambda": 1.0, "min_child_weight": 1.0,
                     "min_leaf_size": 1, "colsample_bytree": 1.0, "colsample_bylevel": 1.0}}


def make_stream_workload(rows, features=128, seed=0):
    """BASELINE config 5 shape: uint8 bins, per column either U{0..255} or a
    Binomial(255, 0.3) look-alike (rounded normal), labels from a random depth-6
    tree on the bins with 10 % flips.  A base tile of at most 4M rows is generated
    and repeated (the content does not change what is measured: PCIe streaming)."""
    rng = np.random.default_rng(seed)
    base = min(rows, 1 << 22)
    tile = rng.integers(0, 256, size=(base, features), dtype=np.uint8)
    for f in range(0, features, 2):
        tile[:, f] = np.clip(np.rint(rng.normal(76.5, 7.3, size=base)), 0, 255).astype(np.uint8)
    reps = (rows + base - 1) // base
    bins = np.tile(tile, (reps, 1))[:rows]
    node = np.zeros(rows, dtype=np.int32)
    for level in range(6):
        nn = 1 << level
        fid = rng.integers(0, features, size=nn)
        thr = rng.integers(40, 200, size=nn)
        node = 2 * node + (bins[np.arange(rows), fid[node]] > thr[node])
    leaf_label = rng.integers(0, 2, size=64)
    y = leaf_label[node].astype(np.float32)
    flip = rng.random(rows) < 0.1
    y[flip] = 1.0 - y[flip]
    return bins, y


def stream_mode(args, arb):
    """Out-of-core leg: bins in pinned host memory, streamed block by block at
    every level (not the headline metric; prints its own JSON line)."""
    bins, y = make_stream_workload(args.stream_rows, args.stream_features)
    cfg = config(args.max_depth, 256)
    cfg["internals"]["upload_features"] = False
    cfg["internals"]["stream_block_rows"] = args.stream_block_rows
    data = arb.DMatrix(bins, y=y, quantized=True)
    del bins
    model = arb.Garden(cfg, data)
    model.grow_tree()      # first call packs the blocks into pinned memory
    model.synchronize()
    if args.stream_timing:
        model.enable_timing(True)
    s0 = model.rows_scanned()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        model.grow_tree()
    model.synchronize()
    dt = time.perf_counter() - t0
    scanned = model.rows_scanned() - s0
    passes = args.max_depth + 1    # one copy of every block per level + the leaf pass
    host_bytes = args.stream_rows * ((args.stream_features + 3) // 4 * 4)
    print(json.dumps({
        "metric": "streamed (out-of-core) tree growing, bins in pinned host memory",
        "sec_per_tree": dt / args.steps, "steps": args.steps,
        "rows": args.stream_rows, "features": args.stream_features, "block_rows": args.stream_block_rows,
        "host_bin_bytes": host_bytes, "passes_per_tree": passes,
        "h2d_GBps": host_bytes * passes * args.steps / dt / 1e9,
        "hist_updates_per_s": scanned * args.stream_features / dt,
        "phase_ms_per_tree": ({k: v / args.steps for k, v in model.timings().items() if k.endswith("_ms")}
                              if args.stream_timing else None)}))


def cpu_baseline(X, y, cfg, sample_rows, trees):
    """The CPU checker on the first `sample_rows` rows (same columns, same
    configuration), all host cores."""
    from oracle import oracle as orc
    cores = os.cpu_count() or 1
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        pass
    cores = min(cores, 16)
    ob = orc.Booster(X[:sample_rows], y=y[:sample_rows], config=cfg, threads=cores)
    t0 = time.perf_counter()
    ob.grow(trees)
    dt = time.perf_counter() - t0
    return {"value": ob.updates / dt, "unit": "row*feature hist updates/s", "cores": cores, "kind": "port",
            "sample": "first %d rows x %d features, %d trees, max_depth %d (%.1f s; quantisation not timed)"
                      % (sample_rows, X.shape[1], trees, cfg["tree"]["max_depth"], dt),
            "sec_per_tree_scaled_to_full_rows": dt / trees * (X.shape[0] / sample_rows)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=40)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--rows", type=int, default=10_500_000)
    ap.add_argument("--features", type=int, default=28)
    ap.add_argument("--max-depth", type=int, default=8)
    ap.add_argument("--hist-size", type=int, default=256)
    ap.add_argument("--cpu-rows", type=int, default=10_500_000)
    ap.add_argument("--cpu-trees", type=int, default=16)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--nan-frac", type=float, default=0.0,
                    help="stress variant: this fraction of the feature values is replaced by NaN (all land in "
                         "one bin per feature; needs --hist-size <= 255)")
    ap.add_argument("--mode", choices=["resident", "stream"], default="resident")
    ap.add_argument("--stream-rows", type=int, default=64_000_000)
    ap.add_argument("--stream-features", type=int, default=128)
    ap.add_argument("--stream-block-rows", type=int, default=1 << 22)
    ap.add_argument("--stream-timing", action="store_true")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MiB",
                    help="also run one device-to-device copy of this many MiB (a kernel of known traffic, "
                         "used to scale the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1")

    import arboretum_amd as arb
    if arb.device_count() < 1:
        sys.exit("bench.py: no HIP device; the benchmark needs an MI355X")

    if args.copy_probe:
        arb.copy_probe(args.copy_probe << 20)
    if args.mode == "stream":
        stream_mode(args, arb)
        return

    X, y = make_workload(args.rows, args.features)
    if args.nan_frac > 0:
        rng = np.random.default_rng(1)
        for f in range(args.features):
            X[rng.random(args.rows, dtype=np.float32) < args.nan_frac, f] = np.nan
    cfg = config(args.max_depth, args.hist_size)
    data = arb.DMatrix(X, y=y)
    t0 = time.perf_counter()
    data.quantize(args.hist_size)
    t_quant = time.perf_counter() - t0
    model = arb.Garden(cfg, data)
    model.labels_count = 1

    for _ in range(args.warmup):
        model.grow_tree()
    model.synchronize()
    # The timed region brackets only the dominant kernel with HIP events (two per launch), on
    # every fourth tree; the phase breakdown comes from a few more trees grown afterwards with
    # every phase bracketed (about 35 event records per tree, which costs 5 % of the tree time).
    model.enable_timing(3)
    scanned0 = model.rows_scanned()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        model.grow_tree()
    model.synchronize()
    dt = time.perf_counter() - t0
    scanned = model.rows_scanned() - scanned0
    tm_dominant = model.timings()
    phase_trees = min(args.steps, 10)
    model.enable_timing(1)
    for _ in range(phase_trees):
        model.grow_tree()
    model.synchronize()
    tm_after = model.timings()
    model.enable_timing(0)
    # phase times of the extra trees only; the dominant kernel's figures from the timed region
    tm = {k: tm_after[k] - tm_dominant[k] for k in tm_after}
    fused_ms_timed, fused_launches_timed = tm_dominant["hist_deep_ms"], tm_dominant["hist_deep_launches"]

    F = args.features
    updates = scanned * F
    row_bytes = F + 8  # uint8 bins of all features + one (g, h) pair: the algorithmic figure
    # what the kernels move: with 0/1 labels (this workload) the pair travels as one float
    moved_row_bytes = F + 4
    cell_bytes = 16    # one histogram cell as written by a workgroup (two 64-bit words)
    # Dominant kernel: the fused partition + histogram pass of levels 1..max_depth-2
    # (k_part_hist<true, 7, true, false, true>).  Algorithmic bytes of one launch: every row is
    # read once and written once in the children order, and the smaller child of
    # each parent gets one histogram written.
    fl = max(fused_launches_timed, 1)
    # parents whose smaller child got a histogram in the measured launches (levels 1..max_depth-2
    # of the sampled trees)
    launches_per_tree = max(args.max_depth - 2, 1)
    parents = sum(1 << (l - 1) for l in range(1, args.max_depth - 1)) * fl / launches_per_tree
    fused_bytes = fl * args.rows * 2 * row_bytes + parents * F * 256 * cell_bytes
    fused_s = fused_ms_timed * 1e-3
    achieved = fused_bytes / fused_s if fused_s > 0 else 0.0
    # root level (k_hist<true, 7>): reads every row, writes one histogram
    root_bytes = tm["hist_root_rows"] * row_bytes + phase_trees * F * 256 * cell_bytes
    root_s = tm["hist_root_ms"] * 1e-3
    # last level (k_part_hist<true, 7, false, false, true>): moves no rows; reads the split feature's quad
    # of every row and then the rows of the smaller children, which are spread over nearly every
    # 32-byte sector: counted as one full read of the rows (the counters show 387 MiB fetched)
    last_bytes = tm["fused_last_launches"] * args.rows * row_bytes
    last_s = tm["fused_last_ms"] * 1e-3

    # HBM bytes per launch of the dominant kernel from hardware counters: two rocprofv3 --pmc
    # runs of this file (FETCH_SIZE, WRITE_SIZE), scaled by the same counters over a copy of
    # known size (--copy-probe); summary and commands in profiles/hbm_traffic_config2_*.txt.
    # Only known for the default workload.
    default_workload = (args.rows, F, args.hist_size, args.max_depth) == (10500000, 28, 256, 8)
    traffic = MEASURED_FUSED_TRAFFIC_BYTES if default_workload else None

    def frac(b, t):
        return (b / t) / HBM_PEAK if t > 0 else 0.0

    other = {"k_part_hist<true,7,false,false,true> (last level)": {
        "frac_of_hbm": frac(last_bytes, last_s),
        "avg_launch_us": tm["fused_last_ms"] * 1e3 / max(tm["fused_last_launches"], 1)}}
    if tm["hist_root_launches"] > 0:
        other["k_hist<true,7> (root level)"] = {
            "frac_of_hbm": frac(root_bytes, root_s),
            "avg_launch_us": tm["hist_root_ms"] * 1e3 / tm["hist_root_launches"],
            "updates_per_s": tm["hist_root_rows"] * F / root_s if root_s > 0 else 0.0}
    else:
        # the last pass of a tree (leaf of every row, prediction update, next gradients)
        # also builds the root histogram of the next tree: rows read once (bins, y_hat, y),
        # leaf id, y_hat, g, h written
        final_bytes = phase_trees * (args.rows * (F + 8 + 16) + F * 256 * cell_bytes * 256)
        other["k_final_hist<7> (last pass of a tree + root histogram of the next)"] = {
            "frac_of_hbm": frac(final_bytes, tm["leaf_ms"] * 1e-3),
            "avg_launch_us": tm["leaf_ms"] * 1e3 / phase_trees,
            "updates_per_s": phase_trees * args.rows * F / (tm["leaf_ms"] * 1e-3) if tm["leaf_ms"] > 0 else 0.0}

    out = {
        "metric": "row*feature hist updates/s + sec/tree at 10M x 28 depth 8; % of HBM peak",
        "value": updates / dt,
        "unit": "row*feature hist updates/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt / args.steps * 1e3,
        "sec_per_tree": dt / args.steps,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int64",
        "data": "synthetic",
        "config": {"workload": "binary classification %d rows x %d dense fp32 features (BASELINE configs[1]), "
                               "%d bins, max_depth %d, logistic, eta 0.1, lambda 1, min_child_weight 1"
                               % (args.rows, F, args.hist_size, args.max_depth),
                   "rows": args.rows, "features": F, "bins": args.hist_size, "max_depth": args.max_depth},
        "roofline": {"bound": "hbm", "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK, "traffic": traffic,
                     "kernel": "k_part_hist<true,7,true,false,true> (fused partition + histogram, levels 1..%d)"
                               % (args.max_depth - 2),
                     "launches": int(fused_launches_timed),
                     "avg_launch_us": fused_ms_timed * 1e3 / fl,
                     "bytes_per_launch": fused_bytes / fl,
                     # (g, h) packed in 4 bytes: bytes the kernel needs to move per launch
                     "bytes_moved_per_launch": (fused_bytes - fl * args.rows * 2 * (row_bytes - moved_row_bytes)) / fl},
        "other_kernels": other,
        "tree_algorithmic_floor_frac_of_hbm": (2.9e9 / (dt / args.steps)) / HBM_PEAK,
        "phase_ms_per_tree": dict({k: v / phase_trees for k, v in tm.items() if k.endswith("_ms")},
                                  hist_deep_ms=fused_ms_timed / (fl / launches_per_tree)),
        "phase_trees": phase_trees,
        "quantise_s": t_quant,
    }
    if not args.no_cpu and args.cpu_trees > 0:
        out["cpu_baseline"] = cpu_baseline(X, y, cfg, min(args.cpu_rows, args.rows), args.cpu_trees)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
