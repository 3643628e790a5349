#!/usr/bin/env python3
"""Headline benchmark: timestamp-range-filtered search on the 1M x 128 mixture set.

One step = one pass of the hot path over the query batch: seeds drawn per query on the
device from the query's window, then the filtered beam search, with dataset, graph,
timestamps, queries and windows already resident in HBM.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Everything goes through the C ABI of libgrab_anns.so (stateless device-pointer entry
points).  The CPU oracle is used only for the cpu_baseline object.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tests"))

import datasets  # noqa: E402
import grab_loader  # noqa: E402

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
MFMA_FP32_PEAK_TFLOPS = 157.3  # MI355X published dense fp32 matrix rate

# HBM bytes per launch of the two main kernels, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this script at its default configuration (summaries under profiles/).  Reported as
# roofline.traffic only when the run uses that configuration, otherwise null.
PMC_CONFIG = (1_000_000, 10_000, 128, 64, 64, 4, 50, 10, 0.10, 65536, 16, 1, False, 768, 16, 32)
PMC_TRAFFIC_BYTES = {"search": 718_879_000, "entry": 63_432_000}  # (FETCH_SIZE x 2.0 + WRITE_SIZE) KiB x 1024


def auto_bitlen(n_seeds, width, degree, selectivity, local_fraction=0.0):
    """Visited-set size when only in-window ids are inserted: 1.25x what 30 iterations can add.
    In a time-partitioned graph the local edges of a row stay in its bucket, hence mostly in the window."""
    need = 1.25 * (n_seeds + 30 * width * degree * max(selectivity, local_fraction))
    b = 8
    while (1 << b) < need:
        b += 1
    return min(b, 13)


def local_fraction(args):
    return args.local_degree / args.degree if args.partition_buckets > 0 else 0.0


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def algorithmic_bytes(ctr, nq, dim, degree, k, filter_word):
    """Per-launch algorithmic bytes: query + seed rows + graph rows + filter words + child rows + results."""
    s, p, f, d = (int(ctr[:, i].sum()) for i in (1, 2, 3, 4))
    return nq * 4 * dim + s * 4 * dim + p * 4 * degree + f * filter_word + d * 4 * dim + nq * k * 12


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--n", type=int, default=1_000_000)
    ap.add_argument("--nq", type=int, default=10_000)
    ap.add_argument("--dim", type=int, default=128)
    ap.add_argument("--degree", type=int, default=64)
    ap.add_argument("--intermediate", type=int, default=128)
    ap.add_argument("--k", type=int, default=10)
    ap.add_argument("--itopk", type=int, default=64)
    ap.add_argument("--entry-samples", type=int, default=65536,
                    help="rows of the entry-point layer that picks the seeds; 0 = seed like the reference (random ids of the window)")
    ap.add_argument("--seeds", type=int, default=16, help="seeds per query taken from the entry-point layer")
    ap.add_argument("--entry-groups", type=int, default=768,
                    help="k-means groups of the sample rows; > 0: only the groups of a query's nearest centroids are scored")
    ap.add_argument("--entry-nprobe", type=int, default=16, help="nearest centroids kept per query (<= 64)")
    ap.add_argument("--entry-min-rows", type=int, default=32, help="groups are walked until this many in-window rows were scored")
    ap.add_argument("--neighbor-timestamps", type=int, default=1,
                    help="with --read-timestamps: 1 = read them from rows laid out like the graph (grab_neighbor_timestamps)")
    ap.add_argument("--read-timestamps", action="store_true",
                    help="test each visited neighbour's timestamp (as the reference does) instead of its id against the "
                         "window's id interval; the two are the same thing when timestamps follow insertion order")
    ap.add_argument("--width", type=int, default=4)
    ap.add_argument("--max-iter", type=int, default=50)
    ap.add_argument("--hash-bitlen", type=int, default=0,
                    help="0: with --filter-first 1 the smallest table with 1.25x the slots of the ids that can pass the window "
                         "between two rebuilds (30 iterations), else 13")
    ap.add_argument("--filter-first", type=int, default=1,
                    help="1: test the window before the visited-set insert, so a small table serves a selective filter")
    ap.add_argument("--decomposition", choices=["auto", "wave", "block"], default="auto",
                    help="one wave or one workgroup per query (auto: wave for batches of 1024 queries or more)")
    ap.add_argument("--partition-buckets", type=int, default=0,
                    help="build the time-partitioned graph instead of the global one: this many equal buckets of consecutive "
                         "rows, local edges inside a bucket, remote edges in the last slots (0 = global graph)")
    ap.add_argument("--local-degree", type=int, default=48, help="local slots of a row in the time-partitioned graph")
    ap.add_argument("--selectivity", type=float, default=0.10)
    ap.add_argument("--centroids", type=int, default=1000)
    ap.add_argument("--cpu-queries", type=int, default=2000, help="queries of the CPU baseline sample")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--hnsw-rows", type=int, default=1_000_000,
                    help="rows of the CPU HNSW baseline (M 32, efConstruction 200, efSearch 128): a prefix of the base "
                         "(all of it by default, about 25 s to build on 16 threads); 0 skips it")
    ap.add_argument("--no-reference-seeding", action="store_true",
                    help="skip the comparison run seeded the way the reference seeds (keeps profiles to one search configuration)")
    ap.add_argument("--no-two-streams", action="store_true",
                    help="skip the run with two batches in flight (keeps profiles to launches that do not overlap)")
    ap.add_argument("--streams", type=int, default=2, help="batches in flight in that run")
    ap.add_argument("--sweep", action="store_true", help="also print the itopk / selectivity sweep to stderr")
    ap.add_argument("--calibrate-copy-mib", type=int, default=0,
                    help="also run one plain device copy of this many MiB (yardstick for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.hash_bitlen == 0:
        args.hash_bitlen = auto_bitlen(args.seeds if args.entry_samples else args.itopk, args.width, args.degree,
                                       args.selectivity, local_fraction(args)) if args.filter_first else 13

    if args.gpus != 1:
        print("bench.py measures one GPU: this index runs on a single MI355X and no multi-GPU figure is produced "
              f"(got --gpus {args.gpus})", file=sys.stderr)
        sys.exit(2)

    grab = grab_loader.load()
    if grab.device_count() < 1:
        print("bench.py needs a GPU: no HIP device is visible", file=sys.stderr)
        sys.exit(3)

    n, nq, dim, deg, k = args.n, args.nq, args.dim, args.degree, args.k
    t0 = time.time()
    data = datasets.mixture(n, dim, args.centroids, 10, 11)
    queries = datasets.mixture(nq, dim, args.centroids, 10, 12)
    ts = np.arange(n, dtype=np.uint64)
    ws, we = datasets.windows(n, nq, args.selectivity, 13)
    log(f"[bench] data generated in {time.time() - t0:.1f}s")

    # ---- build (resident in HBM afterwards) ----
    d_data = grab.DeviceArray.from_numpy(data)
    grab.synchronize()
    tb = time.time()
    if args.partition_buckets > 0:
        nb = args.partition_buckets
        sizes = [n * (b + 1) // nb - n * b // nb for b in range(nb)]
        bucket_of = np.repeat(np.arange(nb, dtype=np.uint64), sizes)
        d_graph = grab.build_time_partitioned_graph(d_data, n, dim, grab.DeviceArray.from_numpy(bucket_of), sizes, deg,
                                                    args.local_degree)
        knn_ms, t_knn, t_opt, knn_flop, knn_redone = 0.0, 0.0, 0.0, 0.0, 0
    else:
        d_knn, knn_ms = grab.generate_knn_graph(d_data, n, dim, args.intermediate, want_ms=True)
        knn_flop, knn_redone = grab.last_knn_stats()
        t_knn = time.time() - tb
        tb2 = time.time()
        d_graph = grab.build_graph(d_data, n, d_knn, args.intermediate, deg)
        t_opt = time.time() - tb2
        d_knn.free()
    build_s = time.time() - tb
    # the contraction computes the tiles on and above the diagonal plus a pass against a sample of the rows: the rate is
    # quoted on the operations it executes (the library's count), not on the 2 n^2 dim of all pairs
    knn_tflops = knn_flop / (knn_ms * 1e-3) / 1e12 if knn_ms else 0.0
    log(f"[bench] build {build_s:.2f}s (kNN {t_knn:.2f}s, contraction kernels {knn_ms:.0f} ms, {knn_flop:.3g} FLOP executed = "
        f"{knn_tflops:.1f} TFLOP/s, {knn_redone} rows redone by the plain pass; all pairs would be {2.0 * n * n * dim:.3g} FLOP; "
        f"optimise {t_opt:.2f}s)")

    d_q = grab.DeviceArray.from_numpy(queries)
    d_ts = grab.DeviceArray.from_numpy(ts)
    d_ws, d_we = grab.DeviceArray.from_numpy(ws), grab.DeviceArray.from_numpy(we)
    d_order = grab.DeviceArray.from_numpy(np.arange(n, dtype=np.uint32))  # timestamps are insertion order

    # ---- exact filtered ground truth on the GPU ----
    gt, _, gt_ms = grab.bruteforce_topk(d_data, n, dim, d_q, nq, k, filter_kind=grab.FILTER_RANGE, d_ts=d_ts,
                                        d_win_start=d_ws, d_win_end=d_we, want_ms=True)
    log(f"[bench] ground truth (exact filtered top-{k}) {gt_ms:.0f} ms")

    use_entry = args.entry_samples > 0
    n_prov = args.seeds if use_entry else args.itopk
    itopk_eff, n_seeds, _ = grab.search_plan(grab.WRAP_RANGE, k, args.itopk, args.width, deg, n_prov)
    layer = grab.EntryLayer(d_data, n, dim, args.entry_samples, d_ts=d_ts) if use_entry else None
    if use_entry and args.entry_groups > 0:
        tg = time.time()
        layer.build_groups(args.entry_groups, niter=10, seed=1)
        log(f"[bench] entry layer: {args.entry_groups} groups of the {layer.size} sample rows in {time.time() - tg:.2f}s")
    entry_ms_box = C.c_float(0.0)

    # outputs, seeds and the descriptor are allocated once: a step allocates nothing and
    # copies nothing over PCIe
    max_seeds = max(n_seeds, 256)
    d_seeds = grab.DeviceArray((nq, max_seeds), np.uint32)
    d_out_i = grab.DeviceArray((nq, k), np.int64)
    d_out_d = grab.DeviceArray((nq, k), np.float32)
    d_ctr = grab.DeviceArray((nq, 6), np.uint64)
    d_lo, d_hi = grab.DeviceArray((nq,), np.uint64), grab.DeviceArray((nq,), np.uint64)
    ms_box = C.c_float(0.0)
    id_filter = not args.read_timestamps
    # timestamps read per neighbour: optionally from rows laid out like the graph instead of scattered single words
    d_graph_ts = grab.neighbor_timestamps(d_graph, d_ts, n, deg) if (args.read_timestamps and args.neighbor_timestamps) else None
    search_flags = (grab.FLAG_FILTER_FIRST if args.filter_first else 0) | \
        {"auto": 0, "wave": grab.FLAG_WAVE_PER_QUERY, "block": grab.FLAG_BLOCK_PER_QUERY}[args.decomposition]

    lane0 = (None, layer, d_seeds, d_lo, d_hi, d_out_i, d_out_d)

    def one_pass(step, want_counters=False, want_ms=False, itopk=None, seeds_n=None, win=None, entry=None, bitlen=None,
                 asynchronous=False, lane=None):
        """One step: seeds from the entry layer (or sampled), then the search.  `asynchronous`: the call returns with the
        kernels queued.  `lane`: (stream, entry layer, seeds, id_lo, id_hi, out ids, out distances) of a second batch in
        flight; the default is the null stream and the buffers above."""
        stream, layer, d_seeds, d_lo, d_hi, d_out_i, d_out_d = lane if lane is not None else lane0
        it = itopk_eff if itopk is None else itopk
        sn = n_seeds if seeds_n is None else seeds_n
        w0, w1 = (d_ws, d_we) if win is None else win
        if entry is None:
            entry = use_entry and itopk is None
        if entry and args.entry_groups > 0:
            # seeds = nearest in-window sample rows among the groups of the query's nearest centroids
            grab.check(grab.lib.grab_entry_layer_select_grouped(layer.h, C.c_void_p(d_q.ptr), C.c_size_t(nq), C.c_int(grab.METRIC_L2),
                                                                C.c_void_p(w0.ptr), C.c_void_p(w1.ptr), C.c_uint64(0), C.c_uint64(0),
                                                                C.c_int(1), C.c_void_p(d_ts.ptr if id_filter else None), C.c_size_t(n),
                                                                C.c_void_p(d_lo.ptr), C.c_void_p(d_hi.ptr),
                                                                C.c_uint32(args.entry_nprobe), C.c_uint32(args.entry_min_rows),
                                                                C.c_uint32(sn), C.c_void_p(d_seeds.ptr),
                                                                C.pointer(entry_ms_box) if want_ms else None, stream))
        elif entry:
            # seeds = nearest in-window rows of the entry-point layer (MFMA contraction over the sample)
            grab.check(grab.lib.grab_entry_layer_select(layer.h, C.c_void_p(d_q.ptr), C.c_size_t(nq), C.c_int(grab.METRIC_L2),
                                                        C.c_int(grab.FILTER_RANGE), C.c_void_p(w0.ptr), C.c_void_p(w1.ptr),
                                                        C.c_uint64(0), C.c_uint64(0), C.c_int(1), None, C.c_uint32(sn),
                                                        C.c_void_p(d_seeds.ptr), C.pointer(entry_ms_box) if want_ms else None, None))
        else:
            # seeds as in the reference: random ids of the window
            grab.check(grab.lib.grab_sample_window_seeds(C.c_void_p(d_ts.ptr), C.c_void_p(d_order.ptr), C.c_size_t(n),
                                                         C.c_void_p(w0.ptr), C.c_void_p(w1.ptr), C.c_uint64(0), C.c_uint64(0),
                                                         C.c_int(1), C.c_size_t(nq), C.c_uint32(sn), C.c_uint64(1000 + step),
                                                         C.c_void_p(d_seeds.ptr), None))
        d = grab.SearchDesc()
        d.d_dataset, d.d_graph, d.num_dataset, d.dim = d_data.ptr, d_graph.ptr, n, dim
        d.graph_degree = d.active_degree = deg
        d.metric = grab.METRIC_L2
        d.d_queries, d.num_queries, d.k = d_q.ptr, nq, k
        d.itopk, d.search_width, d.max_iterations = it, args.width, args.max_iter
        d.hash_bitlen = args.hash_bitlen if bitlen is None else bitlen
        d.n_seeds, d.d_seeds, d.n_provided, d.rand_xor_mask = sn, d_seeds.ptr, sn, 0x5EED0000 + step
        if id_filter:
            # timestamps are insertion order: the window is an id interval (two binary searches per query);
            # the grouped seed selection has written the intervals already
            if not (entry and args.entry_groups > 0):
                grab.check(grab.lib.grab_windows_to_id_ranges(C.c_void_p(d_ts.ptr), C.c_size_t(n), C.c_void_p(w0.ptr),
                                                              C.c_void_p(w1.ptr), C.c_size_t(nq), C.c_void_p(d_lo.ptr),
                                                              C.c_void_p(d_hi.ptr), None))
            d.filter_kind = grab.FILTER_ID_RANGE
            d.d_win_start, d.d_win_end, d.per_query_window = d_lo.ptr, d_hi.ptr, 1
        else:
            d.filter_kind, d.d_ts = grab.FILTER_RANGE, d_ts.ptr
            d.d_graph_ts = d_graph_ts.ptr if d_graph_ts is not None else None
            d.d_win_start, d.d_win_end, d.per_query_window = w0.ptr, w1.ptr, 1
        d.flags = search_flags
        d.d_out_indices, d.d_out_dists = d_out_i.ptr, d_out_d.ptr
        d.d_counters = d_ctr.ptr if want_counters else None
        d.kernel_ms = C.pointer(ms_box) if want_ms else None
        d.stream = stream
        grab.check((grab.lib.grab_search_ex_async if asynchronous else grab.lib.grab_search_ex)(C.byref(d)))
        return ms_box.value if want_ms else None

    if args.calibrate_copy_mib:
        nb = args.calibrate_copy_mib << 20
        a, b = grab.DeviceArray((nb,), np.uint8), grab.DeviceArray((nb,), np.uint8)
        a.fill_bytes(1)
        grab.check(grab.lib.grab_device_copy(C.c_void_p(b.ptr), C.c_void_p(a.ptr), C.c_size_t(nb)))
        a.free()
        b.free()

    # the steps are queued one behind the other on one stream; the host waits once, after the last
    for w in range(args.warmup):
        one_pass(w, asynchronous=True)
    grab.synchronize()
    t1 = time.time()
    for s in range(args.steps):
        one_pass(100 + s, asynchronous=True)
    grab.synchronize()
    elapsed = time.time() - t1
    ids = d_out_i.numpy()
    ms_per_step = elapsed / args.steps * 1e3
    qps = nq / (elapsed / args.steps)
    rec = datasets.recall(ids, gt)

    # the same step with the host hand-over a caller with host buffers pays: queries and windows in, results out
    # (page-locked host buffers, synchronous copies); reported beside the headline value, never as it
    def pinned(arr):
        p = C.c_void_p()
        grab.check(grab.lib.grab_host_malloc(C.byref(p), C.c_size_t(arr.nbytes)))
        view = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(arr.nbytes,)).view(arr.dtype).reshape(arr.shape)
        view[...] = arr
        return p, view
    host_in = [pinned(x) for x in (queries, ws, we)]
    host_out = [pinned(np.empty((nq, k), np.int64)), pinned(np.empty((nq, k), np.float32))]
    # copies and kernels of a step are queued on the one stream, the host waits once per step for its results
    def handed_over(step):
        for dst, (hp, view) in zip((d_q, d_ws, d_we), host_in):
            grab.check(grab.lib.grab_copy_to_device_async(C.c_void_p(dst.ptr), hp, C.c_size_t(view.nbytes), None))
        one_pass(step, asynchronous=True)
        for src, (hp, view) in zip((d_out_i, d_out_d), host_out):
            grab.check(grab.lib.grab_copy_to_host_async(hp, C.c_void_p(src.ptr), C.c_size_t(view.nbytes), None))
        grab.synchronize()
    handed_over(199)
    tp = time.time()
    for s in range(5):
        handed_over(200 + s)
    pcie_qps = nq / ((time.time() - tp) / 5)
    assert np.array_equal(host_out[0][1], d_out_i.numpy())
    for hp, _ in host_in + host_out:
        grab.check(grab.lib.grab_host_free(hp))
    log(f"[bench] with host hand-over (5.3 MB in, 1.2 MB out per step over PCIe, page-locked host buffers, stream-ordered copies, one host wait per step): {pcie_qps:,.0f} QPS")

    # Two batches in flight: the same steps, alternating between two streams, each with its own entry layer, seed and
    # result buffers.  The end of one batch's search (its last queries leave most of the device idle) and the next
    # batch's entry layer (matrix and vector work, little memory traffic) then overlap.  Reported beside the headline
    # value, which stays the one-stream figure.
    two_lanes = None
    if use_entry and args.entry_groups > 0 and not args.no_two_streams:
        streams = []
        for _ in range(args.streams):
            p = C.c_void_p()
            grab.check(grab.lib.grab_stream_create(C.byref(p)))
            streams.append(p)
        lanes = [(streams[0], layer, d_seeds, d_lo, d_hi, d_out_i, d_out_d)]
        for st in streams[1:]:
            layer_b = grab.EntryLayer(d_data, n, dim, args.entry_samples, d_ts=d_ts)
            layer_b.build_groups(args.entry_groups, niter=10, seed=1)
            lanes.append((st, layer_b, grab.DeviceArray((nq, max_seeds), np.uint32), grab.DeviceArray((nq,), np.uint64),
                          grab.DeviceArray((nq,), np.uint64), grab.DeviceArray((nq, k), np.int64),
                          grab.DeviceArray((nq, k), np.float32)))
        for w in range(max(len(lanes), args.warmup)):
            one_pass(w, asynchronous=True, lane=lanes[w % len(lanes)])
        grab.synchronize()
        tl = time.time()
        for s in range(args.steps):
            one_pass(100 + s, asynchronous=True, lane=lanes[s % len(lanes)])
        grab.synchronize()
        el = time.time() - tl
        same = all(np.array_equal(ln[5].numpy(), ids) for ln in lanes)
        two_lanes = {"qps": nq * args.steps / el, "ms_per_step": el / args.steps * 1e3, "streams": len(lanes),
                     "results_equal_one_stream": bool(same)}
        log(f"[bench] {len(lanes)} batches in flight (one stream each): {two_lanes['qps']:,.0f} QPS, {two_lanes['ms_per_step']:.3f} ms per step, "
            f"results {'equal' if same else 'DIFFER from'} the one-stream run")
        for p in streams:
            grab.check(grab.lib.grab_stream_destroy(p))

    # kernel duration from HIP events on the kernel's stream, averaged over the same number of launches
    kms, ems, sms = [], [], []
    for s in range(args.steps):
        kms.append(one_pass(100 + s, want_ms=True))
        ems.append(entry_ms_box.value)
        sms.append(layer.last_select_ms if use_entry else 0.0)
    kernel_ms = float(np.mean(kms))
    entry_ms = float(np.mean(ems)) if use_entry else 0.0
    select_ms = float(np.mean(sms)) if use_entry else 0.0
    one_pass(100, want_counters=True)
    ctr = d_ctr.numpy()
    hash_full = int(ctr[:, 5].sum())
    abytes = algorithmic_bytes(ctr, nq, dim, deg, k, 8)  # F is zero when ids are tested instead of timestamps
    achieved = abytes / (kernel_ms * 1e-3) / 1e9
    # entry-point layer: one dot product per (query, sample row inside the query's window)
    entry_flops = 0.0
    if use_entry:
        S = layer.size
        sample_ts = ts[(np.arange(S, dtype=np.int64) * n // S)]
        cols = np.searchsorted(sample_ts, we, side="left").astype(np.int64) - np.searchsorted(sample_ts, ws, side="left")
        entry_flops = 2.0 * float(np.maximum(cols, 0).sum()) * dim
        if args.entry_groups > 0:
            entry_flops = 2.0 * nq * args.entry_groups * dim  # query x centroid
    entry_tflops = entry_flops / (entry_ms * 1e-3) / 1e12 if entry_ms else 0.0
    log(f"[bench] search: {qps:,.0f} QPS, recall@{k} {rec:.4f}, kernel {kernel_ms:.3f} ms, {abytes / nq / 1024:.1f} KiB/query "
        f"-> {achieved:.0f} GB/s; mean iters {ctr[:, 0].mean():.1f}, F {ctr[:, 3].mean():.0f}, D {ctr[:, 4].mean():.0f}, "
        f"visited-set overflows {hash_full}; entry layer: contraction {entry_ms:.3f} ms = {entry_tflops:.1f} TFLOP/s, "
        f"selection {select_ms:.3f} ms")

    # the same search seeded the way the reference seeds it (itopk random ids of the window), for comparison
    ref_seeding = None
    if use_entry and not args.no_reference_seeding:
        ie, sn, _ = grab.search_plan(grab.WRAP_RANGE, k, 256, args.width, deg, 256)
        one_pass(0, itopk=ie, seeds_n=sn)
        grab.synchronize()
        tt = time.time()
        for s in range(5):
            one_pass(s, itopk=ie, seeds_n=sn)
        grab.synchronize()
        ref_seeding = {"itopk": 256, "seeds_per_query": sn, "qps": nq / ((time.time() - tt) / 5),
                       "recall_at_10": datasets.recall(d_out_i.numpy(), gt)}
        log(f"[bench] reference seeding (random window ids, itopk 256): {ref_seeding}")

    sweep = None
    if args.sweep:
        sweep = []
        for sel in (0.01, 0.10, 0.50):
            s0, s1 = datasets.windows(n, nq, sel, 13)
            w = (grab.DeviceArray.from_numpy(s0), grab.DeviceArray.from_numpy(s1))
            g, _, _ = grab.bruteforce_topk(d_data, n, dim, d_q, nq, k, filter_kind=grab.FILTER_RANGE, d_ts=d_ts,
                                           d_win_start=w[0], d_win_end=w[1])
            for itk in (32, 64, 128, 256):
                for seeding in (("entry-layer", "reference") if use_entry else ("reference",)):
                    ent = seeding == "entry-layer"
                    ie, sn, _ = grab.search_plan(grab.WRAP_RANGE, k, itk, args.width, deg, args.seeds if ent else itk)
                    bl = auto_bitlen(sn, args.width, deg, sel, local_fraction(args)) if args.filter_first else 13
                    one_pass(0, itopk=ie, seeds_n=sn, win=w, entry=ent, bitlen=bl, want_counters=True)
                    overflow = int(d_ctr.numpy()[:, 5].sum())
                    grab.synchronize()
                    tt = time.time()
                    for s in range(5):
                        one_pass(s, itopk=ie, seeds_n=sn, win=w, entry=ent, bitlen=bl)
                    grab.synchronize()
                    row = {"selectivity": sel, "itopk": itk, "itopk_eff": ie, "seeding": seeding, "seeds": sn, "hash_bitlen": bl,
                           "qps": nq / ((time.time() - tt) / 5), "recall": datasets.recall(d_out_i.numpy(), g),
                           "visited_set_overflows": overflow}
                    sweep.append(row)
                    log(f"[sweep] {row}")

    cpu = None
    if not args.no_cpu:
        import oracle_binding as oracle
        graph = d_graph.numpy()
        m = min(args.cpu_queries, nq)
        threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
        tc = time.time()
        if use_entry:
            S = layer.size
            sid = (np.arange(S, dtype=np.int64) * n // S).astype(np.uint32)
            cid, _ = oracle.bruteforce_topk(data[sid], queries[:m], n_seeds, filter_kind=oracle.FILTER_RANGE, ts=ts[sid],
                                            win_start=ws[:m], win_end=we[:m], threads=threads)
            seeds = np.where(cid >= 0, sid[np.clip(cid, 0, S - 1)], 0xFFFFFFFF).astype(np.uint32)
        else:
            seeds = oracle.sample_window_seeds(ts, np.arange(n, dtype=np.uint32), n_seeds, 1100, win_start=ws[:m], win_end=we[:m])
        cids, _, _ = oracle.search(data, graph, queries[:m], k, itopk_eff, args.width, args.max_iter, args.hash_bitlen,
                                   n_seeds, 0x5EED0064, seeds=seeds, filter_kind=oracle.FILTER_RANGE, ts=ts,
                                   win_start=ws[:m], win_end=we[:m], flags=search_flags & 3, threads=threads)
        tcs = time.time() - tc
        mb = min(200, m)
        tbf = time.time()
        oracle.bruteforce_topk(data, queries[:mb], k, filter_kind=oracle.FILTER_RANGE, ts=ts, win_start=ws[:mb],
                               win_end=we[:mb], threads=threads)
        tbfs = time.time() - tbf
        cpu = {"value": m / tcs, "unit": "queries/s", "cores": threads, "kind": "port",
               "sample": f"first {m} of the {nq} queries, same graph/params/windows, CPU restatement of the reference "
                         f"search (OpenMP over queries); seeds = the exact nearest in-window sample rows, brute force "
                         f"over the sample included in the time (the GPU's grouped selection approximates these seeds)",
               "recall_at_k": datasets.recall(cids, gt[:m]),
               "exact_filtered_bruteforce_qps": mb / tbfs, "exact_bruteforce_sample": f"first {mb} queries"}
        log(f"[bench] cpu baseline: {cpu['value']:.0f} QPS on {threads} threads (recall {cpu['recall_at_k']:.4f}); "
            f"exact filtered brute force {cpu['exact_filtered_bruteforce_qps']:.1f} QPS")
        if args.hnsw_rows > 0:
            # HNSW as the configurations name it for FAISS (not installed: the published algorithm restated in
            # oracle/hnsw_baseline.cpp), on a prefix of the base with 10 % windows over that prefix, post-filtered
            import hnsw_binding
            hn = min(args.hnsw_rows, n)
            hq = min(1000, nq)
            hws, hwe = datasets.windows(hn, hq, args.selectivity, 17)
            hgt, _ = oracle.bruteforce_topk(data[:hn], queries[:hq], k, filter_kind=oracle.FILTER_RANGE, ts=ts[:hn],
                                            win_start=hws, win_end=hwe, threads=threads)
            hnsw = hnsw_binding.Hnsw(dim, 32, 200)
            th = time.time()
            hnsw.add(data[:hn], threads=threads)
            hbuild = time.time() - th
            th = time.time()
            hids, _ = hnsw.search_range(queries[:hq], k, ts[:hn], hws, hwe, ef=128, threads=threads)
            hsearch = time.time() - th
            cpu["hnsw"] = {"rows": hn, "M": 32, "ef_construction": 200, "ef_search": 128, "threads": threads,
                           "build_seconds": hbuild, "insert_vectors_per_s": hn / hbuild, "filtered_qps": hq / hsearch,
                           "recall_at_10": datasets.recall(hids, hgt), "queries": hq,
                           "filter": "post-filter, ef doubled until 10 results fall inside the window"}
            hnsw.close()
            log(f"[bench] cpu HNSW on the first {hn} rows: build {hbuild:.1f}s ({hn / hbuild:.0f} vectors/s), filtered "
                f"{hq / hsearch:.0f} QPS at recall {cpu['hnsw']['recall_at_10']:.4f}")

    # Two kernels carry the step: the beam search (random row gathers: HBM-bound) and the entry
    # layer's contraction (fp32 MFMA-bound).  "roofline" describes the one with the longer launch.
    default_cfg = (n, nq, dim, deg, args.itopk, args.width, args.max_iter, args.hash_bitlen, args.selectivity, args.entry_samples,
                   args.seeds, args.filter_first, args.read_timestamps, args.entry_groups, args.entry_nprobe,
                   args.entry_min_rows) == PMC_CONFIG
    rl_search = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                 "traffic": PMC_TRAFFIC_BYTES["search"] if default_cfg else None,
                 "kernel": "search_wave_reg_kernel (id-interval filter)" if args.decomposition != "block" and nq >= 1024
                 else "search_kernel", "kernel_ms": kernel_ms, "algorithmic_bytes": abytes}
    rl_entry = {"bound": "mfma", "achieved": entry_tflops, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": entry_tflops / MFMA_FP32_PEAK_TFLOPS, "traffic": PMC_TRAFFIC_BYTES["entry"] if default_cfg else None,
                "kernel": "tile_topk_kernel (dense-store mode, entry-point layer%s)" % (": queries x centroids" if args.entry_groups > 0 else ""),
                "kernel_ms": entry_ms,
                "algorithmic_flops": entry_flops}
    roofline, roofline_secondary = (rl_search, rl_entry) if (kernel_ms >= entry_ms or not use_entry) else (rl_entry, rl_search)
    if not use_entry:
        roofline_secondary = None

    result = {
        "metric": "filtered QPS @ recall@10>=0.95 (1M x 128)",
        "value": qps,
        "unit": "queries/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"timestamp range-filtered search, {n} x {dim} fp32 Gaussian mixture ({args.centroids} centroids), "
                        f"{nq} queries, window selectivity {args.selectivity:g}, L2",
            "k": k, "itopk": args.itopk, "itopk_eff": itopk_eff, "search_width": args.width,
            "max_iterations": args.max_iter, "hash_bitlen": args.hash_bitlen, "graph_degree": deg,
            "intermediate_degree": args.intermediate, "seeds_per_query": n_seeds,
            "graph": (f"time-partitioned, {args.partition_buckets} buckets, local degree {args.local_degree}"
                      if args.partition_buckets > 0 else "global"),
            "seeding": ((f"entry-point layer, {args.entry_samples} sample rows"
                         + (f" in {args.entry_groups} k-means groups, {args.entry_nprobe} nearest centroids kept, groups walked "
                            f"until {args.entry_min_rows} in-window rows" if args.entry_groups > 0 else ""))
                        if use_entry else "random ids of the window (reference)"),
            "filter": ("id interval of the window (timestamps = insertion order)" if id_filter else "timestamp read per visited neighbour"),
        },
        "recall_at_10": rec,
        "recall_target_met": bool(rec >= 0.95),
        "build_seconds": build_s,
        "build": {"knn_seconds": t_knn, "knn_kernel_ms": knn_ms, "knn_tflops": knn_tflops, "knn_flop_executed": knn_flop,
                  "knn_flop_all_pairs": 2.0 * n * n * dim, "knn_rows_redone": knn_redone, "optimize_seconds": t_opt,
                  "mfma_fp32_peak_tflops": MFMA_FP32_PEAK_TFLOPS, "mfma_frac": knn_tflops / MFMA_FP32_PEAK_TFLOPS},
        "roofline": roofline,
        "roofline_secondary": roofline_secondary,
        "visited_set_overflows": hash_full,
        "pcie_inclusive_qps": pcie_qps,
        "two_batches_in_flight": two_lanes,
        "entry_layer": ({"samples": args.entry_samples, "groups": args.entry_groups, "nprobe": args.entry_nprobe,
                         "min_rows": args.entry_min_rows, "contraction_ms": entry_ms, "selection_ms": select_ms}
                        if use_entry else None),
        "reference_seeding": ref_seeding,
        "cpu_baseline": cpu,
    }
    if sweep is not None:
        result["sweep"] = sweep
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
