#!/usr/bin/env python3
"""Exact top-k inside narrow timestamp windows (one GPU): the scan of the windows' rows on the matrix cores.

Base: the 1M x 128 mixture of the headline benchmark, timestamps in row order, so a window is an interval of row ids.
Queries: 10,000 per batch, each with its own window of `--selectivity` of the rows.  Per selectivity: wall time of a call
over a prepared base (`grab_scan_base_window_topk`: host tables, their upload, contraction, selection, exact re-scoring),
the one-shot call (`grab_window_scan_topk`, which also splits the base rows and allocates its scratch), the kernels' own
time, and whether ids and distance bits equal the exact filtered top-k (`grab_bruteforce_topk`).  Prints ONE JSON line;
progress goes to stderr.

    python bench_window_scan.py [--n 1000000] [--nq 10000] [--dim 128] [--selectivity 0.001 0.01 0.1] [--steps 10]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tests"))

import datasets  # noqa: E402
import grab_loader  # noqa: E402


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--n", type=int, default=1_000_000)
    ap.add_argument("--nq", type=int, default=10_000)
    ap.add_argument("--dim", type=int, default=128)
    ap.add_argument("--k", type=int, default=10)
    ap.add_argument("--selectivity", type=float, nargs="*", default=[0.001, 0.01, 0.03, 0.1])
    ap.add_argument("--steps", type=int, default=10)
    args = ap.parse_args()
    grab = grab_loader.load()
    if grab.device_count() < 1:
        print("needs a GPU: no HIP device is visible", file=sys.stderr)
        sys.exit(3)
    n, nq, dim, k = args.n, args.nq, args.dim, args.k
    data = datasets.mixture(n, dim, 1000, 10, 11)
    q = datasets.mixture(nq, dim, 1000, 10, 12)
    d_data, d_q = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(q)
    d_ts = grab.DeviceArray.from_numpy(np.arange(n, dtype=np.uint64))
    d_out = (grab.DeviceArray((nq, k), np.int64), grab.DeviceArray((nq, k), np.float32))
    t = time.perf_counter()
    base = grab.ScanBase(d_data, n, dim)
    grab.synchronize()
    t_base = time.perf_counter() - t
    rows = []
    for sel in args.selectivity:
        lo, hi = datasets.windows(n, nq, sel, 13)
        gt, gd, _ = grab.bruteforce_topk(d_data, n, dim, d_q, nq, k, filter_kind=grab.FILTER_RANGE, d_ts=d_ts,
                                         d_win_start=grab.DeviceArray.from_numpy(lo), d_win_end=grab.DeviceArray.from_numpy(hi))
        ids, dist, _ = base.window_topk(d_q, nq, k, lo, hi)
        redone = grab.last_knn_exact_rows()
        equal = bool(np.array_equal(ids, gt) and np.array_equal(dist.view(np.uint32), gd.view(np.uint32)))
        base.window_topk(d_q, nq, k, lo, hi, d_out=d_out)  # the base's scratch has grown to this size of call
        walls, kms = [], []
        for _ in range(args.steps):
            grab.synchronize()
            t = time.perf_counter()
            _, _, ms = base.window_topk(d_q, nq, k, lo, hi, want_ms=True, d_out=d_out)
            walls.append(time.perf_counter() - t)
            kms.append(ms)
        flop = grab.last_knn_bf16_flop() or grab.last_knn_stats()[0]
        grab.window_scan_topk(d_data, n, dim, d_q, nq, k, lo, hi, d_out=d_out)
        grab.synchronize()
        t = time.perf_counter()
        grab.window_scan_topk(d_data, n, dim, d_q, nq, k, lo, hi, d_out=d_out)
        one_shot = time.perf_counter() - t
        wall, kernel_ms = float(np.mean(walls)), float(np.mean(kms))
        row = {"selectivity": sel, "ms_per_batch": wall * 1e3, "qps": nq / wall, "contraction_and_selection_ms": kernel_ms,
               "recall_at_10": datasets.recall(ids, gt), "ids_and_distance_bits_equal_exact_filtered_topk": equal,
               "queries_redone_row_by_row": int(redone), "one_shot_ms_per_batch": one_shot * 1e3,
               "matrix_flop": flop, "matrix_tflops": flop / (kernel_ms * 1e-3) / 1e12,
               "matrix_pipe": "bf16 (rows split into two bf16 halves, three instructions a product)" if grab.last_knn_bf16_flop() > 0 else "fp32"}
        rows.append(row)
        log(f"[window scan] {row}")
    base.close()
    print(json.dumps({"workload": f"exact top-{k} inside per-query windows, {n} x {dim} mixture, {nq} queries per batch, "
                                  "timestamps in row order", "prepare_base_seconds": t_base, "rows": rows}), flush=True)


if __name__ == "__main__":
    main()
