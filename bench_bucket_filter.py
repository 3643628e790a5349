#!/usr/bin/env python3
"""High-dimensional bucket-filtered search (one GPU): 768-d unit rows, inner product, label sets.

Base: unit-normalised N(0,1) rows, each with one of 64 bucket labels drawn Zipf(s = 1.1).  Queries:
unit-norm rows, each restricted to 1-4 random buckets (a 64-bit label set tested inside the traversal,
filter kind 2).  Graph degree 64 from intermediate degree 128, k 10, itopk 128, search width 4.
Seeds: itopk random rows that carry one of the query's labels, drawn on the host before the timed region
(`--entry-samples N`: the label-carrying rows nearest to the query among N sample rows instead, from the
entry-point layer, its time counted).  The rows are stored label by label and the graph is the bucket-partitioned
one unless `--partitioned 0`.  Ground truth: exact filtered top-10 on the GPU (`grab_bruteforce_topk`).  Reports build seconds, queries/s from the search kernel's own duration,
recall@10, and algorithmic bytes per second.  Prints ONE JSON line; progress goes to stderr.

    python bench_bucket_filter.py [--n 1000000] [--nq 10000] [--dim 768] [--itopk 128]
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


def label_seeds(labels, masks, n_labels, per_query, seed):
    """[nq, per_query] uint32: random distinct rows that carry one of the query's labels (0xFFFFFFFF pads short lists)."""
    rng = np.random.default_rng(seed)
    order = np.argsort(labels, kind="stable").astype(np.uint32)
    starts = np.searchsorted(labels[order], np.arange(n_labels + 1))
    out = np.full((masks.shape[0], per_query), 0xFFFFFFFF, np.uint32)
    for i, m in enumerate(masks):
        ls = [b for b in range(n_labels) if (int(m) >> b) & 1]
        sizes = np.array([starts[b + 1] - starts[b] for b in ls])
        total = int(sizes.sum())
        pick = rng.choice(total, size=min(per_query, total), replace=False)
        which = np.searchsorted(np.cumsum(sizes), pick, side="right")
        offs = pick - (np.cumsum(sizes) - sizes)[which]
        out[i, :pick.size] = order[starts[np.array(ls)[which]] + offs]
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--n", type=int, default=1_000_000)
    ap.add_argument("--nq", type=int, default=10_000)
    ap.add_argument("--dim", type=int, default=768)
    ap.add_argument("--degree", type=int, default=64)
    ap.add_argument("--intermediate", type=int, default=128)
    ap.add_argument("--labels", type=int, default=64)
    ap.add_argument("--itopk", type=int, nargs="*", default=[128])
    ap.add_argument("--width", type=int, default=4)
    ap.add_argument("--max-iter", type=int, default=50)
    ap.add_argument("--hash-bitlen", type=int, default=13)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--entry-samples", type=int, default=0,
                    help="> 0: seeds are the label-carrying rows nearest to the query among this many sample rows (the "
                         "entry-point layer, exact selection with the label test); 0: random label-carrying rows")
    ap.add_argument("--seeds", type=int, default=0, help="seeds per query from the entry layer (0: itopk, at most 256)")
    ap.add_argument("--decomposition", choices=["auto", "wave", "block"], default="auto",
                    help="one wave or one workgroup per query")
    ap.add_argument("--filter-first", type=int, default=0, help="1: test the label set before the visited-set insert")
    ap.add_argument("--partitioned", type=int, default=1,
                    help="1: rows are stored label by label and the graph is the bucket-partitioned one (CagraIndexOpt: local edges "
                         "stay inside a row's bucket, the last slots hold remote edges); 0: one global graph over rows in random order")
    ap.add_argument("--local-degree", type=int, default=48)
    args = ap.parse_args()

    grab = grab_loader.load()
    if grab.device_count() < 1:
        print("needs a GPU: no HIP device is visible", file=sys.stderr)
        sys.exit(3)
    n, nq, dim, deg, k = args.n, args.nq, args.dim, args.degree, 10
    t0 = time.time()
    data = datasets.unit_rows(n, dim, 20)
    labels = datasets.zipf_labels(n, args.labels, 1.1, 21)
    q = datasets.unit_rows(nq, dim, 22)
    masks = datasets.label_masks(nq, args.labels, 23)
    if args.partitioned:
        order = np.argsort(labels, kind="stable")
        data, labels = np.ascontiguousarray(data[order]), np.ascontiguousarray(labels[order])
    log(f"[bucket] data generated in {time.time() - t0:.1f}s")

    d_data = grab.DeviceArray.from_numpy(data)
    grab.synchronize()
    tb = time.time()
    if args.partitioned:
        sizes = [int(c) for c in np.bincount(labels, minlength=args.labels) if c > 0]
        bucket_of = np.repeat(np.arange(len(sizes), dtype=np.uint64), sizes)
        d_graph = grab.build_time_partitioned_graph(d_data, n, dim, grab.DeviceArray.from_numpy(bucket_of), sizes, deg,
                                                    args.local_degree, grab.METRIC_IP)
        grab.synchronize()
        knn_ms, t_knn, knn_pipe = None, None, None
    else:
        d_knn, knn_ms = grab.generate_knn_graph(d_data, n, dim, args.intermediate, grab.METRIC_IP, want_ms=True)
        knn_flop = grab.last_knn_stats()[0]  # the operations the contraction executed (about half of all pairs)
        knn_bf16 = grab.last_knn_bf16_flop()   # ... on bf16 instructions, three a product of the split rows
        knn_pipe = "bf16" if knn_bf16 > 0 else "fp32"
        knn_flop = knn_bf16 if knn_bf16 > 0 else knn_flop
        grab.synchronize()
        t_knn = time.time() - tb
        d_graph = grab.build_graph(d_data, n, d_knn, args.intermediate, deg)
        grab.synchronize()
        d_knn.free()
    t_build = time.time() - tb
    knn_tflops = knn_flop / (knn_ms * 1e-3) / 1e12 if knn_ms else None
    log(f"[bucket] build {t_build:.2f}s" + (f" (kNN {t_knn:.2f}s, contraction kernel {knn_ms:.0f} ms = {knn_tflops:.1f} TFLOP/s of {knn_pipe} instructions)" if knn_ms else
                                            f" (graph partitioned into {len(sizes)} buckets, {args.local_degree} local slots)"))

    d_q = grab.DeviceArray.from_numpy(q)
    d_labels, d_masks = grab.DeviceArray.from_numpy(labels), grab.DeviceArray.from_numpy(masks)
    t = time.time()
    gt, _, _ = grab.bruteforce_topk(d_data, n, dim, d_q, nq, k, metric=grab.METRIC_IP, filter_kind=grab.FILTER_MASK,
                                    d_labels=d_labels, d_masks=d_masks)
    log(f"[bucket] ground truth (exact filtered top-{k}) {1e3 * (time.time() - t):.0f} ms")
    passing = np.array([np.count_nonzero((int(m) >> labels.astype(np.uint64)) & np.uint64(1)) for m in masks[:200]])
    log(f"[bucket] rows passing a query's label set (first 200 queries): median {np.median(passing) / n:.3%}, "
        f"min {passing.min() / n:.3%}, max {passing.max() / n:.3%}")

    flags = {"auto": 0, "wave": grab.FLAG_WAVE_PER_QUERY, "block": grab.FLAG_BLOCK_PER_QUERY}[args.decomposition] | \
        (grab.FLAG_FILTER_FIRST if args.filter_first else 0)
    rows = []
    layer = None
    for itopk in args.itopk:
        n_seeds, entry_ms = itopk, None
        if args.entry_samples > 0:
            n_seeds = min(args.seeds if args.seeds else itopk, 256, itopk)
            if layer is None:
                layer = grab.EntryLayer(d_data, n, dim, args.entry_samples, d_labels=d_labels)
            d_seeds = grab.DeviceArray((nq, n_seeds), np.uint32)
            for _ in range(2):  # the second call is timed on the host (the call returns when the seeds are written)
                grab.synchronize()
                te = time.time()
                layer.select(d_q, nq, n_seeds, metric=grab.METRIC_IP, filter_kind=grab.FILTER_MASK, d_masks=d_masks, d_out=d_seeds)
                entry_ms = (time.time() - te) * 1e3
        else:
            d_seeds = grab.DeviceArray.from_numpy(label_seeds(labels, masks, args.labels, itopk, 24))
        run = lambda **kw: grab.search_ex(d_data, d_graph, n, dim, deg, d_q, nq, k, itopk, args.width, args.max_iter,
                                          args.hash_bitlen, n_seeds, 9, d_seeds=d_seeds, n_provided=n_seeds, metric=grab.METRIC_IP,
                                          filter_kind=grab.FILTER_MASK, d_labels=d_labels, d_masks=d_masks,
                                          flags=flags, **kw)
        ids, _, ctr, _ = run(want_counters=True)
        ms = []
        for _ in range(args.steps):
            ms.append(run(want_ms=True)[3])
        kernel_ms = float(np.mean(ms))
        # algorithmic bytes: query + seed rows + graph rows + one label byte per tested neighbour + child rows + results
        s, p, f, d = (int(ctr[:, i].sum()) for i in (1, 2, 3, 4))
        abytes = nq * 4 * dim + s * 4 * dim + p * 4 * deg + f * 1 + d * 4 * dim + nq * k * 12
        row = {"method": "graph", "itopk": itopk, "seeds": n_seeds, "entry_layer_ms": entry_ms, "kernel_ms": kernel_ms,
               "qps": nq / ((kernel_ms + (entry_ms or 0.0)) * 1e-3), "recall_at_10": datasets.recall(ids, gt),
               "algorithmic_bytes": abytes, "achieved_GBps": abytes / (kernel_ms * 1e-3) / 1e9,
               "frac_of_hbm_peak": abytes / (kernel_ms * 1e-3) / 8e12, "mean_iterations": float(ctr[:, 0].mean()),
               "rows_scored_per_query": (s + d) / nq}
        rows.append(row)
        log(f"[bucket] {row}")
        d_seeds.free()

    # The exact answer for the same queries: only the rows of a query's buckets are scanned, on the matrix cores (the rows
    # are stored bucket by bucket).  Wall time of the whole call: host-side set-up, transfers of the row tables, contraction,
    # exact re-scoring and the merge of a query's partial lists.
    if args.partitioned:
        offsets = np.searchsorted(labels, np.arange(args.labels + 1)).astype(np.uint64)
        d_out = (grab.DeviceArray((nq, k), np.int64), grab.DeviceArray((nq, k), np.float32))
        grab.bucket_scan_topk(d_data, n, dim, offsets, d_q, nq, k, masks, metric=grab.METRIC_IP, d_out=d_out)  # warm
        walls, kms = [], []
        for _ in range(args.steps):
            grab.synchronize()
            t = time.perf_counter()
            _, _, ms1 = grab.bucket_scan_topk(d_data, n, dim, offsets, d_q, nq, k, masks, metric=grab.METRIC_IP, want_ms=True, d_out=d_out)
            walls.append(time.perf_counter() - t)
            kms.append(ms1)
        flop, flop_bf16 = grab.last_knn_stats()[0], grab.last_knn_bf16_flop()
        on_bf16 = flop_bf16 > 0
        flop, peak = (flop_bf16, 2500.0) if on_bf16 else (flop, 157.3)
        wall, kernel_ms = float(np.mean(walls)), float(np.mean(kms))
        sids = d_out[0].numpy()
        row = {"method": "exact bucket scan", "itopk": None, "qps": nq / wall, "ms_per_batch": wall * 1e3, "kernel_ms": kernel_ms,
               "recall_at_10": datasets.recall(sids, gt), "ids_equal_exact_filtered_topk": bool(np.array_equal(sids, gt)),
               "flop": flop, "tflops": flop / (kernel_ms * 1e-3) / 1e12, "mfma_frac": flop / (kernel_ms * 1e-3) / 1e12 / peak,
               "mfma_pipe": "bf16 (rows split into two bf16 halves, three instructions a product)" if on_bf16 else "fp32"}
        rows.append(row)
        log(f"[bucket] {row}")
        # the same scan over a base prepared once: the rows' bf16 halves and the calls' scratch memory are kept
        tb0 = time.perf_counter()
        base = grab.ScanBase(d_data, n, dim, grab.METRIC_IP)
        grab.synchronize()
        t_base = time.perf_counter() - tb0
        for _ in range(2):
            base.bucket_topk(offsets, d_q, nq, k, masks, d_out=d_out)
        walls, kms = [], []
        for _ in range(args.steps):
            grab.synchronize()
            t = time.perf_counter()
            _, _, ms1 = base.bucket_topk(offsets, d_q, nq, k, masks, want_ms=True, d_out=d_out)
            walls.append(time.perf_counter() - t)
            kms.append(ms1)
        wall, kernel_ms = float(np.mean(walls)), float(np.mean(kms))
        sids = d_out[0].numpy()
        row = dict(row, method="exact bucket scan, prepared base", qps=nq / wall, ms_per_batch=wall * 1e3, kernel_ms=kernel_ms,
                   recall_at_10=datasets.recall(sids, gt), ids_equal_exact_filtered_topk=bool(np.array_equal(sids, gt)),
                   tflops=flop / (kernel_ms * 1e-3) / 1e12, mfma_frac=flop / (kernel_ms * 1e-3) / 1e12 / peak,
                   prepare_base_seconds=t_base)
        rows.append(row)
        log(f"[bucket] {row}")
        base.close()

    print(json.dumps({
        "workload": f"bucket-filtered search, {n} x {dim} unit rows, inner product, {args.labels} Zipf(1.1) labels, "
                    f"{nq} queries with 1-4 labels each, degree {deg}, k {k}, width {args.width}, "
                    + (f"graph partitioned by label ({args.local_degree} local slots)" if args.partitioned else "global graph"),
        "build_seconds": t_build, "knn_seconds": t_knn, "knn_kernel_ms": knn_ms, "knn_tflops": knn_tflops, "knn_pipe": knn_pipe,
        "search": rows}), flush=True)


if __name__ == "__main__":
    main()
