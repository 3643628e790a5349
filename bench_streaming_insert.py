#!/usr/bin/env python3
"""Streaming insert + search on the 1M x 128 mixture set (one GPU).

Start from the first half of the set built from scratch, insert the rest in batches with
increasing timestamps (CagraIndex::insert semantics: 64 rows per inner step, each step sees
the rows of the steps before it), and after every batch run range queries whose window is
10 % of the current time span.  Reports insert vectors/s, mapped versus logical bytes of the
growable device buffers, and recall@10 beside that of an index built from scratch at the
same size (at the checkpoints).  Prints ONE JSON line; progress goes to stderr.

    python bench_streaming_insert.py [--n 1000000] [--start 500000] [--batch 10000] [--queries 1000]
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
    ap.add_argument("--start", type=int, default=500_000)
    ap.add_argument("--batch", type=int, default=10_000)
    ap.add_argument("--queries", type=int, default=1000)
    ap.add_argument("--dim", type=int, default=128)
    ap.add_argument("--degree", type=int, default=64)
    ap.add_argument("--itopk", type=int, default=64)
    ap.add_argument("--entry-samples-per-million", type=int, default=65536)
    ap.add_argument("--insert-hash-bitlen", type=int, default=14)
    ap.add_argument("--checkpoints", type=int, nargs="*", default=None, help="sizes at which a from-scratch index is built")
    args = ap.parse_args()

    grab = grab_loader.load()
    if grab.device_count() < 1:
        print("needs a GPU: no HIP device is visible", file=sys.stderr)
        sys.exit(3)
    n, n0, dim, deg, k = args.n, args.start, args.dim, args.degree, 10
    checkpoints = args.checkpoints if args.checkpoints is not None else [(n0 + n) // 2 // args.batch * args.batch, n]
    t0 = time.time()
    data = datasets.mixture(n, dim, 1000, 10, 11)
    ts = np.arange(n, dtype=np.uint64)  # increasing timestamps = insertion order
    log(f"[stream] data generated in {time.time() - t0:.1f}s")

    def make_index(rows):
        idx = grab.CagraIndex(dim, deg, vmm_max_bytes=4 << 30)
        idx.setBuildParams(128, deg)
        idx.setQueryParams(args.itopk, 4, 0, 50, 10)   # 1024-slot visited set: only in-window ids enter it
        # insert searches are unfiltered, 6 x 64 ids per iteration: the reference's 4096-slot table
        # (src/cagraIndex.cu:34-37) fills up after a dozen iterations and probing a nearly full table
        # dominates the insert; 16384 slots stay under half full for a whole search
        idx.setInsertParams(128, 6, 0, 50, args.insert_hash_bitlen)
        idx.set_flags(grab.FLAG_FILTER_FIRST)
        idx.set_entry_layer(max(1024, int(args.entry_samples_per_million * rows / 1e6)), 16)
        return idx

    def measure(idx, rows, seed):
        """Recall@10 and queries/s of `idx` on fresh queries with 10 % windows over [0, rows)."""
        q = datasets.mixture(args.queries, dim, 1000, 10, seed)
        ws, we = datasets.windows(rows, args.queries, 0.1, seed + 1)
        idx.query_range_batch(q, k, ws, we)  # warm: entry layer rebuilt for the new rows
        t = time.time()
        ids, _ = idx.query_range_batch(q, k, ws, we)
        dt = time.time() - t
        d_data, _, d_ts = idx.device_ptrs()
        gt, _, _ = grab.bruteforce_topk(d_data, rows, dim, grab.DeviceArray.from_numpy(q), args.queries, k,
                                        filter_kind=grab.FILTER_RANGE, d_ts=d_ts,
                                        d_win_start=grab.DeviceArray.from_numpy(ws), d_win_end=grab.DeviceArray.from_numpy(we))
        return datasets.recall(ids, gt), args.queries / dt, (q, ws, we, gt)

    idx = make_index(n0)
    idx.add(data[:n0], ts[:n0])
    tb = time.time()
    idx.build()
    build0 = time.time() - tb
    log(f"[stream] initial build of {n0} rows: {build0:.2f}s")
    rec0, qps0, _ = measure(idx, n0, 14)
    log(f"[stream] before inserts: recall@10 {rec0:.4f}")

    batches, insert_s = [], 0.0
    rows = n0
    b = 0
    while rows < n:
        cur = min(args.batch, n - rows)
        t = time.time()
        idx.insert(data[rows:rows + cur], ts[rows:rows + cur])
        dt = time.time() - t
        insert_s += dt
        rows += cur
        b += 1
        rec, qps, probe = measure(idx, rows, 14 + b)
        mapped = idx.mapped_bytes()
        logical = (rows * dim * 4, rows * deg * 4, rows * 8)
        row = {"batch": b, "rows": rows, "insert_vectors_per_s": cur / dt, "recall_at_10": rec, "query_qps_host_buffers": qps,
               "mapped_bytes": sum(mapped), "logical_bytes": sum(logical)}
        if rows in checkpoints:
            fresh = make_index(rows)
            fresh.add(data[:rows], ts[:rows])
            tb = time.time()
            fresh.build()
            row["from_scratch_build_s"] = time.time() - tb
            q, ws, we, gt = probe
            fresh.query_range_batch(q, k, ws, we)
            fids, _ = fresh.query_range_batch(q, k, ws, we)
            row["from_scratch_recall_at_10"] = datasets.recall(fids, gt)
            row["recall_drift"] = rec - row["from_scratch_recall_at_10"]
            fresh.close()
        batches.append(row)
        log(f"[stream] {row}")

    inserted = n - n0
    result = {
        "workload": f"streaming insert + range search, {n} x {dim} mixture, start {n0}, batches of {args.batch}, "
                    f"{args.queries} queries per batch with 10 % windows, itopk {args.itopk}, degree {deg}",
        "insert_vectors_per_s": inserted / insert_s,
        "insert_seconds_total": insert_s,
        "initial_build_s": build0,
        "recall_before_inserts": rec0,
        "recall_min": min(r["recall_at_10"] for r in batches),
        "recall_last": batches[-1]["recall_at_10"],
        "mapped_bytes_final": batches[-1]["mapped_bytes"],
        "logical_bytes_final": batches[-1]["logical_bytes"],
        "mapped_over_logical": batches[-1]["mapped_bytes"] / batches[-1]["logical_bytes"],
        "checkpoints": [r for r in batches if "recall_drift" in r],
        "batches": batches,
    }
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
