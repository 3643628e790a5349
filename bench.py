#!/usr/bin/env python3
"""Headline benchmark: timestamp-range-filtered search on the 1M x 128 mixture set.

One step = one pass of the hot path over one query batch: seeds drawn per query on the
device from the query's window, then the filtered beam search, with dataset, graph,
timestamps, queries and windows already resident in HBM.  Consecutive steps take different
pre-generated batches (queries and windows), so that a step does not find in the 256 MB
Infinity Cache what the step before it read.  Prints ONE JSON line.

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
MFMA_BF16_PEAK_TFLOPS = 2500.0  # ... and dense bf16

# HBM bytes per launch of the two main kernels come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script
# at its default configuration (summaries under profiles/).  The figures live in a small tracked file beside those
# summaries, each with a digest of the kernel's source files and the configuration it was measured on:
# roofline.traffic is reported only while both still match, otherwise null - a figure cannot outlive its kernel.
# `python bench.py --record-traffic search=BYTES entry=BYTES` rewrites the file (no GPU needed).
PMC_CONFIG = (1_000_000, 10_000, 128, 64, 64, 4, 50, 10, 0.10, 65536, "list", 32, 1, False, 768, 16, 16, 8)
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "pmc_hbm_traffic_bytes.txt")
# the files that hold device code of the two kernels (common.hpp holds host-side helpers only)
KERNEL_SOURCES = {"search": ("search_wave.hip", "search_internal.hpp", "device_utils.hpp"),
                  "entry": ("entry_probe.hip", "entry_layer.hpp", "device_utils.hpp")}


def source_digest(kernel):
    import hashlib
    h = hashlib.sha256()
    for f in KERNEL_SOURCES[kernel]:
        with open(os.path.join(ROOT, "grab-anns_amd", "csrc", f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def config_digest(cfg=PMC_CONFIG):
    import hashlib
    return hashlib.sha256(repr(tuple(cfg)).encode()).hexdigest()[:12]


def load_traffic(cfg):
    """{kernel: bytes per launch} for the kernels whose recorded figure matches today's sources and `cfg`."""
    out = {"search": None, "entry": None}
    try:
        lines = open(TRAFFIC_FILE).read().splitlines()
    except OSError:
        return out
    for ln in lines:
        p = ln.split()
        if len(p) == 4 and not ln.startswith("#") and p[0] in out:
            if p[1] == source_digest(p[0]) and p[2] == config_digest(cfg):
                out[p[0]] = int(p[3])
    return out


def record_traffic(pairs):
    rows = ["# HBM bytes per launch by rocprofv3 --pmc: (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0) KiB x 1024, the factors being what the",
            "# same counters read for a plain device copy of known size.  Written by `python bench.py --record-traffic`;",
            "# bench.py reports a figure as roofline.traffic only while the digests still match.",
            "# kernel  sha256[:16] of " + " / ".join("+".join(v) for v in KERNEL_SOURCES.values()) + "  sha256[:12] of the configuration  bytes"]
    for pair in pairs:
        name, val = pair.split("=")
        rows.append(f"{name} {source_digest(name)} {config_digest()} {int(val)}")
    with open(TRAFFIC_FILE, "w") as f:
        f.write("\n".join(rows) + "\n")


def auto_bitlen(n_seeds, width, degree, selectivity, local_fraction=0.0):
    """Visited-set size when only in-window ids are inserted: 1.25x what 30 iterations can add.
    In a time-partitioned graph the local edges of a row stay in its bucket, hence mostly in the window."""
    need = 1.25 * (n_seeds + 30 * width * degree * max(selectivity, local_fraction))
    b = 8
    while (1 << b) < need:
        b += 1
    return min(b, 13)


def entry_seeds(args):
    """Seeds per query that the entry layer hands to the headline search."""
    ts_filter = args.read_timestamps and args.neighbor_timestamps < 2
    return args.seeds if (args.entry_mode == "scored" or args.entry_groups == 0 or ts_filter) else args.entry_list


def default_shape(args):
    """The configuration's own shape (side benchmarks only ride along with it, not with experiments)."""
    return (args.n, args.nq, args.dim, args.partition_buckets, args.read_timestamps) == (1_000_000, 10_000, 128, 0, False)


def local_fraction(args):
    return args.local_degree / args.degree if args.partition_buckets > 0 else 0.0


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def algorithmic_bytes(ctr, nq, dim, degree, k, filter_word):
    """Per-launch algorithmic bytes: query + seed rows + graph rows + filter words + child rows + results."""
    s, p, f, d = (int(ctr[:, i].sum()) for i in (1, 2, 3, 4))
    return nq * 4 * dim + s * 4 * dim + p * 4 * degree + f * filter_word + d * 4 * dim + nq * k * 12


MAX_LINE_CHARS = 6000  # the last stdout line is read back from a tail of limited length


def _r(x, digits=4):
    """Numbers of the short line: floats to `digits` significant digits, everything else as it is."""
    if isinstance(x, bool) or x is None or isinstance(x, (int, str)):
        return x
    if isinstance(x, float):
        y = float(f"{x:.{digits}g}")
        return int(y) if abs(y) >= 1e5 and y == int(y) else y
    if isinstance(x, dict):
        return {k: _r(v, digits) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [_r(v, digits) for v in x]
    return x


def _pick(d, keys):
    return {k: d[k] for k in keys if d is not None and k in d}


def compact_line(full):
    """The ONE stdout line: the contract's fields, roofline, cpu_baseline and one terse row per other configuration.
    `full` is everything the run measured (written to stderr and gpurun_out/bench_detail.json).  Text fields are
    short on purpose, trajectories and per-batch lists stay out: the line must stay well under MAX_LINE_CHARS."""
    cfg = full["config"]
    sp = full.get("ms_per_step_spread") or {}
    out = {k: full[k] for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step")}
    out.update({"ms_per_step_min": sp.get("min"), "ms_per_step_median": sp.get("median"), "ms_per_step_max": sp.get("max"),
                "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": full["dtype"], "data": "synthetic"})
    out["config"] = {"workload": cfg["workload_short"]}
    out["config"].update(_pick(cfg, ("k", "itopk", "search_width", "max_iterations", "hash_bitlen", "graph_degree",
                                     "seeds_per_query", "graph", "seeding_short", "filter_short")))
    out.update(_pick(full, ("recall_at_10", "recall_target_met", "build_seconds")))
    b = full.get("build") or {}
    out["build"] = _pick(b, ("knn_seconds", "knn_kernel_ms", "knn_tflops", "mfma_peak_tflops", "mfma_frac", "knn_pipe",
                             "knn_rows_redone", "knn_rows_not_proven_redone_exactly", "optimize_seconds"))
    for key in ("roofline", "roofline_secondary"):
        rl = full.get(key)
        out[key] = None if rl is None else _pick(rl, ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel_short",
                                                      "kernel_ms", "algorithmic_bytes", "algorithmic_flops"))
    cpu = full.get("cpu_baseline")
    if cpu is not None:
        c = _pick(cpu, ("value", "unit", "cores", "kind", "sample_short", "recall_at_k", "gpu_ids_equal_cpu_same_seeds",
                        "gpu_counters_equal_cpu_same_seeds", "exact_filtered_bruteforce_qps"))
        c["sample"] = c.pop("sample_short", "")
        h = cpu.get("hnsw")
        if h:
            c["hnsw"] = _pick(h, ("rows", "build_seconds", "filtered_qps", "recall_at_10", "threads"))
        out["cpu_baseline"] = c
    else:
        out["cpu_baseline"] = None
    out.update(_pick(full, ("visited_set_overflows", "pcie_inclusive_qps", "partitioned_build_seconds")))
    hd = full.get("handle")
    if hd:
        out["handle_qps"] = hd.get("qps")
        out["handle"] = _pick(hd, ("ms_per_call", "recall_at_10", "buffers", "one_shot_qps", "scan_sel1_qps", "scan_sel1_ids_equal_exact"))
    tl = full.get("two_batches_in_flight")
    if tl:
        out["two_streams"] = _pick(tl, ("qps", "ms_per_step", "streams", "results_equal_one_stream"))
    rs = full.get("reference_seeding")
    if rs:
        out["reference_seeding"] = _pick(rs, ("itopk", "qps", "recall_at_10"))
    # one terse entry per other configuration; the sweep as lists of values under `columns`
    allrows = full.get("configs") or []
    if allrows:
        cols = ("graph_short", "selectivity", "itopk", "qps", "recall_at_10")
        out["configs"] = {
            "cfg3_sweep": {"columns": ["graph", "selectivity", "itopk", "qps", "recall_at_10"],
                           "rows": [[r.get(c) for c in cols] for r in allrows if r.get("cfg") == "cfg3"]},
            "cfg3_other": [_pick(r, ("max_iterations", "listed_seeds", "qps", "recall_at_10", "kernel_ms", "frac_of_hbm_peak"))
                           for r in allrows if r.get("cfg") == "cfg3 op"],
            "cfg2": [_pick(r, ("seeding_short", "itopk", "qps", "recall_at_10")) for r in allrows if r.get("cfg") == "cfg2 unfiltered"],
            "cfg3_exact_scan": {"columns": ["selectivity", "qps", "recall_at_10", "ids_equal_exact"],
                                "rows": [[r.get(c) for c in ("selectivity", "qps", "recall_at_10", "ids_equal_exact_filtered_topk")]
                                         for r in allrows if r.get("cfg") == "cfg3 scan"]},
            "visited_set_overflows": sum(int(r.get("visited_set_overflows") or 0) for r in allrows)}
    else:
        out["configs"] = None
    side = full.get("configs_other_benchmarks") or {}
    c4 = side.get("cfg4_streaming_insert")
    if c4:
        out["cfg4"] = c4 if "error" in c4 else dict(
            _pick(c4, ("insert_vectors_per_s", "initial_build_s", "recall_before_inserts", "recall_min", "recall_last",
                       "mapped_over_logical")),
            checkpoints=[_pick(r, ("rows", "recall_at_10", "from_scratch_recall_at_10", "recall_drift"))
                         for r in c4.get("checkpoints", [])])
    c5 = side.get("cfg5_bucket_filter_1Mx768")
    if c5:
        out["cfg5"] = c5 if "error" in c5 else dict(
            {k: v for k, v in _pick(c5, ("build_seconds", "knn_pipe", "knn_tflops")).items() if v is not None},
            search=[_pick(r, ("method", "itopk", "qps", "recall_at_10", "kernel_ms", "frac_of_hbm_peak", "mfma_frac"))
                    for r in c5.get("search", [])])
    line = json.dumps(_r(out), separators=(",", ":"))
    assert len(line) < MAX_LINE_CHARS, f"bench line is {len(line)} characters; the limit is {MAX_LINE_CHARS}"
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--settle-ms", type=float, default=40.0,
                    help="untimed steps are run for this long before the warm-up, until the device holds its clock")
    ap.add_argument("--batches", type=int, default=8,
                    help="distinct pre-generated query/window batches that the steps rotate through")
    ap.add_argument("--repeats", type=int, default=5,
                    help="blocks of --steps steps that are timed; `value` is the first, the spread over all is reported")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the rows of the other configurations (1 % / 50 % windows, longer lists, unfiltered search, "
                         "time-partitioned graph)")
    ap.add_argument("--no-side-benches", action="store_true",
                    help="skip bench_streaming_insert.py (cfg4) and bench_bucket_filter.py (cfg5), which run as child processes "
                         "after the headline and whose JSON lines are embedded in this one")
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
    ap.add_argument("--entry-min-rows", type=int, default=16, help="groups are walked until this many in-window rows were met")
    ap.add_argument("--entry-mode", choices=["list", "fused", "scored"], default="list",
                    help="list: the in-window rows of the groups of the nearest centroids are listed and the search scores them "
                         "all as seeds (grab_entry_layer_list_grouped); fused: the search kernel writes that list itself "
                         "(grab_entry_layer_probe + grab_search_desc.entry_layer); scored: the walk scores the rows and hands "
                         "over the --seeds nearest (grab_entry_layer_select_grouped)")
    ap.add_argument("--entry-list", type=int, default=32, help="list / fused: at most this many listed rows per query (<= 64)")
    ap.add_argument("--neighbor-timestamps", type=int, default=1,
                    help="with --read-timestamps: 0 = d_ts[neighbour], a scattered 8-byte read per test; 1 = 8-byte timestamps "
                         "in rows laid out like the graph (grab_neighbor_timestamps); 2 = 4-byte places in timestamp order in "
                         "rows laid out like the graph (grab_neighbor_ranks, interval test on the place); 3 = d_rank[neighbour], "
                         "a scattered 4-byte read per test")
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
    ap.add_argument("--knn-fp32", action="store_true",
                    help="build the kNN graph with fp32 matrix instructions only (default: bf16 halves where they apply; same graph)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--hnsw-rows", type=int, default=1_000_000,
                    help="rows of the CPU HNSW baseline (M 32, efConstruction 200, efSearch 128): a prefix of the base "
                         "(all of it by default, about 25 s to build on 16 threads); 0 skips it")
    ap.add_argument("--no-reference-seeding", action="store_true",
                    help="skip the comparison run seeded the way the reference seeds (keeps profiles to one search configuration)")
    ap.add_argument("--no-handle", action="store_true", help="skip the run through the index handle with host pointers")
    ap.add_argument("--no-two-streams", action="store_true",
                    help="skip the run with two batches in flight (keeps profiles to launches that do not overlap)")
    ap.add_argument("--streams", type=int, default=2, help="batches in flight in that run")
    ap.add_argument("--sweep", action="store_true", help="also print the itopk / selectivity sweep to stderr")
    ap.add_argument("--calibrate-copy-mib", type=int, default=0,
                    help="also run one plain device copy of this many MiB (yardstick for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--record-traffic", nargs="+", metavar="KERNEL=BYTES",
                    help="write profiles/pmc_hbm_traffic_bytes.txt for today's kernel sources and the default configuration, then exit")
    args = ap.parse_args()
    if args.record_traffic:
        record_traffic(args.record_traffic)
        return
    if args.hash_bitlen == 0:
        args.hash_bitlen = auto_bitlen(entry_seeds(args) if args.entry_samples else args.itopk, args.width, args.degree,
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
    ts = np.arange(n, dtype=np.uint64)
    # batch 0 is the configuration's query set (seeds 12 / 13); the others are further draws of the same kind
    B = max(1, args.batches)
    h_q = [datasets.mixture(nq, dim, args.centroids, 10, 12 + 100 * b) for b in range(B)]
    h_win = [datasets.windows(n, nq, args.selectivity, 13 + 100 * b) for b in range(B)]
    queries, (ws, we) = h_q[0], h_win[0]
    log(f"[bench] data generated in {time.time() - t0:.1f}s ({B} batches of {nq} queries)")

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
        knn_ms, t_knn, t_opt, knn_flop, knn_redone, knn_exact_rows, knn_flop_bf16 = 0.0, 0.0, 0.0, 0.0, 0, 0, 0.0
    else:
        if args.knn_fp32:
            grab.knn_allow_bf16(False)
        d_knn, knn_ms = grab.generate_knn_graph(d_data, n, dim, args.intermediate, want_ms=True)
        knn_flop, knn_redone = grab.last_knn_stats()
        knn_flop_bf16 = grab.last_knn_bf16_flop()
        knn_exact_rows = grab.last_knn_exact_rows()
        t_knn = time.time() - tb
        tb2 = time.time()
        d_graph = grab.build_graph(d_data, n, d_knn, args.intermediate, deg)
        t_opt = time.time() - tb2
        d_knn.free()
    build_s = time.time() - tb
    # the contraction computes the tiles on and above the diagonal plus a pass against a sample of the rows: the rate is
    # quoted on the operations it executes (the library's count), not on the 2 n^2 dim of all pairs
    # Where the symmetric pass and its bounds run on the bf16 pipe (three instructions a product of the split rows), the
    # rate is quoted on those operations against that pipe's peak; the fp32 instructions left are the redone rows
    knn_on_bf16 = knn_flop_bf16 > 0.0
    knn_tflops = (knn_flop_bf16 if knn_on_bf16 else knn_flop) / (knn_ms * 1e-3) / 1e12 if knn_ms else 0.0
    knn_peak = MFMA_BF16_PEAK_TFLOPS if knn_on_bf16 else MFMA_FP32_PEAK_TFLOPS
    log(f"[bench] build {build_s:.2f}s (kNN {t_knn:.2f}s, contraction kernels {knn_ms:.0f} ms, "
        f"{knn_flop_bf16 if knn_on_bf16 else knn_flop:.3g} {'bf16' if knn_on_bf16 else 'fp32'} FLOP executed = "
        f"{knn_tflops:.1f} TFLOP/s, {knn_redone} rows redone by the plain pass, {knn_exact_rows} rows not proven by their candidates and redone exactly; all pairs would be {2.0 * n * n * dim:.3g} FLOP; "
        f"optimise {t_opt:.2f}s)")

    d_ts = grab.DeviceArray.from_numpy(ts)
    d_order = grab.DeviceArray.from_numpy(np.arange(n, dtype=np.uint32))  # timestamps are insertion order
    d_qs = [grab.DeviceArray.from_numpy(x) for x in h_q]
    d_wins = [(grab.DeviceArray.from_numpy(a), grab.DeviceArray.from_numpy(b)) for a, b in h_win]
    d_q, (d_ws, d_we) = d_qs[0], d_wins[0]

    # ---- exact filtered ground truth on the GPU, every batch ----
    gts, gt_ms = [], 0.0
    for b in range(B):
        g, _, ms1 = grab.bruteforce_topk(d_data, n, dim, d_qs[b], nq, k, filter_kind=grab.FILTER_RANGE, d_ts=d_ts,
                                         d_win_start=d_wins[b][0], d_win_end=d_wins[b][1], want_ms=True)
        gts.append(g)
        gt_ms += ms1
    gt = gts[0]
    log(f"[bench] ground truth (exact filtered top-{k}) {gt_ms / B:.0f} ms per batch")

    use_entry = args.entry_samples > 0
    n_prov = entry_seeds(args) if use_entry else args.itopk
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
    new_outs = lambda: [(grab.DeviceArray((nq, k), np.int64), grab.DeviceArray((nq, k), np.float32)) for _ in range(B)]
    outs0 = new_outs()  # one result buffer per batch, so that the recall of the timed steps themselves is what is reported
    d_ctr = grab.DeviceArray((nq, 6), np.uint64)
    d_lo, d_hi = grab.DeviceArray((nq,), np.uint64), grab.DeviceArray((nq,), np.uint64)
    ms_box = C.c_float(0.0)
    rank_mode = args.read_timestamps and args.neighbor_timestamps >= 2   # the interval is tested on the row's place in timestamp order
    id_filter = not args.read_timestamps or rank_mode
    # timestamps are insertion order here, so a row's place in timestamp order is its id: the table is the identity,
    # which the kernel cannot know - it reads it like any other
    d_rank = grab.DeviceArray.from_numpy(np.arange(n, dtype=np.uint32)) if rank_mode else None
    # timestamps read per neighbour: optionally from rows laid out like the graph instead of scattered single words
    d_graph_ts = grab.neighbor_timestamps(d_graph, d_ts, n, deg) if (args.read_timestamps and args.neighbor_timestamps == 1) else None
    d_graph_rank = grab.neighbor_ranks(d_graph, d_rank, n, deg) if (rank_mode and args.neighbor_timestamps == 2) else None
    search_flags = (grab.FLAG_FILTER_FIRST if args.filter_first else 0) | \
        {"auto": 0, "wave": grab.FLAG_WAVE_PER_QUERY, "block": grab.FLAG_BLOCK_PER_QUERY}[args.decomposition]

    d_groups0 = grab.DeviceArray((nq, max(1, args.entry_nprobe)), np.uint32)
    lane0 = (None, layer, d_seeds, d_lo, d_hi, outs0, d_groups0)

    def one_pass(step, want_counters=False, want_ms=False, itopk=None, seeds_n=None, win=None, entry=None, bitlen=None,
                 asynchronous=False, lane=None, batch=None, graph=None, flags=None, count=None, wins=None, unfiltered=False,
                 given_seeds=None, max_iter=None, list_n=None):
        """One step: seeds from the entry layer (or sampled), then the search.  `asynchronous`: the call returns with the
        kernels queued.  `batch`: which pre-generated batch (default: step modulo the number of batches).  `lane`:
        (stream, entry layer, seeds, id_lo, id_hi, result buffers per batch) of another batch in flight; the default is
        the null stream and the buffers above.  `count`: only the first `count` queries of the batch.  `wins`: other
        windows, one pair of device arrays per batch.  `unfiltered`: no filter at all (cfg2).  `given_seeds`: a device
        array [count, seeds_n] used instead of any selection.  `max_iter`: another iteration limit.  `list_n`: the
        headline's way of seeding with another number of listed rows per query."""
        stream, layer, d_seeds, d_lo, d_hi, outs = lane[:6] if lane is not None else lane0[:6]
        d_groups = (lane if lane is not None else lane0)[6]
        fused = False
        b = step % B if batch is None else batch
        d_q = d_qs[b]
        d_out_i, d_out_d = outs[b]
        nq = args.nq if count is None else count
        it = itopk_eff if itopk is None else itopk
        sn = n_seeds if seeds_n is None else seeds_n
        if list_n is not None:
            sn = list_n
        w0, w1 = (d_wins[b] if wins is None else wins[b]) if win is None else win
        if entry is None:
            entry = use_entry and itopk is None
        if given_seeds is not None:
            d_seeds = given_seeds
            if id_filter and not unfiltered:
                grab.check(grab.lib.grab_windows_to_id_ranges(C.c_void_p(d_ts.ptr), C.c_size_t(n), C.c_void_p(w0.ptr),
                                                              C.c_void_p(w1.ptr), C.c_size_t(nq), C.c_void_p(d_lo.ptr),
                                                              C.c_void_p(d_hi.ptr), None))
        elif unfiltered:
            if entry:
                # nearest sample rows, no window: one window that covers every timestamp, no id intervals asked
                grab.check(grab.lib.grab_entry_layer_select_grouped(layer.h, C.c_void_p(d_q.ptr), C.c_size_t(nq), C.c_int(grab.METRIC_L2),
                                                                    None, None, C.c_uint64(0), C.c_uint64(2**63), C.c_int(0), None,
                                                                    C.c_size_t(0), None, None, C.c_uint32(args.entry_nprobe),
                                                                    C.c_uint32(args.entry_min_rows), C.c_uint32(sn),
                                                                    C.c_void_p(d_seeds.ptr), None, stream))
        elif entry and args.entry_groups > 0:
            mode = args.entry_mode if (seeds_n is None and id_filter) else "scored"   # the rows of other configurations
            if mode == "fused" and rank_mode:
                mode = "list"
            if mode == "fused":
                # nearest centroids now; the search kernel turns the window into the id interval and lists the seeds itself
                grab.check(grab.lib.grab_entry_layer_probe(layer.h, C.c_void_p(d_q.ptr), C.c_size_t(nq), C.c_int(grab.METRIC_L2),
                                                           C.c_uint32(args.entry_nprobe), C.c_void_p(d_groups.ptr),
                                                           C.pointer(entry_ms_box) if want_ms else None, stream))
                fused = True
            else:
                # seeds = in-window sample rows of the groups of the query's nearest centroids: listed, or scored and the
                # nearest kept
                fn = grab.lib.grab_entry_layer_list_grouped if mode == "list" else grab.lib.grab_entry_layer_select_grouped
                grab.check(fn(layer.h, C.c_void_p(d_q.ptr), C.c_size_t(nq), C.c_int(grab.METRIC_L2),
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
        d.d_dataset, d.d_graph, d.num_dataset, d.dim = d_data.ptr, (d_graph if graph is None else graph).ptr, n, dim
        d.graph_degree = d.active_degree = deg
        d.metric = grab.METRIC_L2
        d.d_queries, d.num_queries, d.k = d_q.ptr, nq, k
        d.itopk, d.search_width, d.max_iterations = it, args.width, args.max_iter if max_iter is None else max_iter
        d.hash_bitlen = args.hash_bitlen if bitlen is None else bitlen
        d.n_seeds, d.d_seeds, d.n_provided, d.rand_xor_mask = sn, d_seeds.ptr, sn, 0x5EED0000 + b   # seeds that a short list leaves open are drawn with it: one value per batch, so that a batch's result does not depend on the step that ran it
        if unfiltered:
            d.filter_kind = grab.FILTER_NONE
            if not entry and given_seeds is None:
                d.d_seeds, d.n_provided = None, 0   # the reference's formula ids (src/index/compute_distance.cuh:176)
        elif id_filter:
            # timestamps are insertion order: the window is an id interval (two binary searches per query);
            # the grouped seed selection has written the intervals already
            if given_seeds is None and not (entry and args.entry_groups > 0):
                grab.check(grab.lib.grab_windows_to_id_ranges(C.c_void_p(d_ts.ptr), C.c_size_t(n), C.c_void_p(w0.ptr),
                                                              C.c_void_p(w1.ptr), C.c_size_t(nq), C.c_void_p(d_lo.ptr),
                                                              C.c_void_p(d_hi.ptr), None))
            d.filter_kind = grab.FILTER_ID_RANGE
            d.d_win_start, d.d_win_end, d.per_query_window = d_lo.ptr, d_hi.ptr, 1
            if rank_mode:
                d.d_rank = d_rank.ptr
                d.d_graph_rank = d_graph_rank.ptr if d_graph_rank is not None else None
            if fused:
                d.d_win_start, d.d_win_end, d.d_ts = w0.ptr, w1.ptr, d_ts.ptr   # timestamps: the kernel works out the interval
                d.entry_layer, d.d_entry_groups = layer.h, d_groups.ptr
                d.entry_nprobe, d.entry_min_rows = args.entry_nprobe, args.entry_min_rows
                d.d_seeds, d.n_provided = None, 0
        else:
            d.filter_kind, d.d_ts = grab.FILTER_RANGE, d_ts.ptr
            d.d_graph_ts = d_graph_ts.ptr if d_graph_ts is not None else None
            d.d_win_start, d.d_win_end, d.per_query_window = w0.ptr, w1.ptr, 1
        d.flags = (search_flags & ~grab.FLAG_FILTER_FIRST if unfiltered else search_flags) if flags is None else flags
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

    # The device takes some tens of milliseconds of continuous work to settle at the clock it then holds (blocks of 20
    # steps right after an idle phase read 0.190, 0.188, 0.185, 0.184, 0.182 ms): the same untimed steps run for
    # --settle-ms before the warm-up, whatever --warmup says.
    settle_steps = 0
    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
        for w in range(16):
            one_pass(settle_steps + w, asynchronous=True)
        grab.synchronize()
        settle_steps += 16
    # the steps are queued one behind the other on one stream; the host waits once, after the last
    for w in range(args.warmup):
        one_pass(w, asynchronous=True)
    grab.synchronize()
    block_ms = []
    for r in range(max(1, args.repeats)):
        t1 = time.perf_counter()
        for s in range(args.steps):
            one_pass(r * args.steps + s, asynchronous=True)   # batch = step modulo the number of batches
        grab.synchronize()
        block_ms.append((time.perf_counter() - t1) / args.steps * 1e3)
    ms_per_step = block_ms[0]   # `value`: the first block of exactly --steps steps
    qps = nq / (ms_per_step * 1e-3)
    ids_by_batch = [outs0[b][0].numpy() for b in range(B)]
    ids = ids_by_batch[0]
    recalls = [datasets.recall(ids_by_batch[b], gts[b]) for b in range(min(B, args.steps * max(1, args.repeats)))]
    rec = float(np.mean(recalls))
    spread = {"blocks": len(block_ms), "min": float(np.min(block_ms)), "median": float(np.median(block_ms)),
              "max": float(np.max(block_ms)), "all": [round(x, 5) for x in block_ms]}
    log(f"[bench] ms per step over {len(block_ms)} blocks of {args.steps} steps: min {spread['min']:.4f} median {spread['median']:.4f} "
        f"max {spread['max']:.4f}; recall@{k} per batch {[round(x, 4) for x in recalls]}")

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
        one_pass(step, asynchronous=True, batch=0)
        for src, (hp, view) in zip(outs0[0], host_out):
            grab.check(grab.lib.grab_copy_to_host_async(hp, C.c_void_p(src.ptr), C.c_size_t(view.nbytes), None))
        grab.synchronize()
    handed_over(199)
    tp = time.time()
    for s in range(5):
        handed_over(200 + s)
    pcie_qps = nq / ((time.time() - tp) / 5)
    assert np.array_equal(host_out[0][1], outs0[0][0].numpy())
    for hp, _ in host_in + host_out:
        grab.check(grab.lib.grab_host_free(hp))
    log(f"[bench] with host hand-over (5.3 MB in, 1.2 MB out per step over PCIe, page-locked host buffers, stream-ordered copies, one host wait per step): {pcie_qps:,.0f} QPS")

    # The same batches through the index handle, the reference's calling convention: CagraIndex with host pointers to
    # ordinary pageable memory in, results to pageable memory out, one call per batch (query_range_batch: the
    # per-query-window extension of query_range).  The handle cuts the batch into chunks that overlap on its streams.
    # Reported beside the headline value, never as it.
    handle = None
    if use_entry and args.entry_groups > 0 and id_filter and default_shape(args) and not args.no_handle:
        th = time.time()
        idx = grab.CagraIndex(dim, deg, vmm_max_bytes=4 << 30)
        idx.setBuildParams(args.intermediate, deg)
        idx.setQueryParams(args.itopk, args.width, 0, args.max_iter, args.hash_bitlen)
        idx.set_flags(grab.FLAG_FILTER_FIRST)
        idx.set_entry_layer(args.entry_samples, args.seeds)
        idx.set_entry_groups(args.entry_groups, args.entry_nprobe, args.entry_min_rows)
        idx.set_entry_list(args.entry_list if args.entry_mode == "list" else 0)
        idx.add(data, ts)
        idx.build()
        h_ids, h_dist = np.empty((nq, k), np.int64), np.empty((nq, k), np.float32)

        def handle_call(b):
            grab.check(grab.lib.grab_index_search_range_batch(
                idx.h, h_q[b].ctypes.data_as(C.c_void_p), C.c_size_t(nq), C.c_int(k), h_win[b][0].ctypes.data_as(C.c_void_p),
                h_win[b][1].ctypes.data_as(C.c_void_p), h_ids.ctypes.data_as(C.c_void_p), h_dist.ctypes.data_as(C.c_void_p)))

        def handle_rate(calls):
            for b in range(min(B, 3)):
                handle_call(b)
            t = time.perf_counter()
            for c in range(calls):
                handle_call(c % B)
            return nq / ((time.perf_counter() - t) / calls)
        hq = handle_rate(4 * B)
        hrec = []
        for b in range(min(B, 4)):
            handle_call(b)
            hrec.append(datasets.recall(h_ids, gts[b]))
        idx.set_batch_chunk(0)
        hq_one = handle_rate(2 * B)
        # 1 % windows through the handle's exact scan (CagraIndex::scan_range_batch), same host buffers
        narrow = [datasets.windows(n, nq, 0.01, 13 + 100 * b) for b in range(B)]

        def scan_call(b):
            grab.check(grab.lib.grab_index_scan_range_batch(
                idx.h, h_q[b].ctypes.data_as(C.c_void_p), C.c_size_t(nq), C.c_int(k), narrow[b][0].ctypes.data_as(C.c_void_p),
                narrow[b][1].ctypes.data_as(C.c_void_p), h_ids.ctypes.data_as(C.c_void_p), h_dist.ctypes.data_as(C.c_void_p)))
        for b in range(min(B, 3)):
            scan_call(b)
        t = time.perf_counter()
        for c in range(2 * B):
            scan_call(c % B)
        scan_qps = nq / ((time.perf_counter() - t) / (2 * B))
        scan_call(0)
        gt_narrow = grab.bruteforce_topk(d_data, n, dim, d_qs[0], nq, k, filter_kind=grab.FILTER_RANGE, d_ts=d_ts,
                                         d_win_start=grab.DeviceArray.from_numpy(narrow[0][0]),
                                         d_win_end=grab.DeviceArray.from_numpy(narrow[0][1]))[0]
        handle = {"qps": hq, "ms_per_call": nq / hq * 1e3, "recall_at_10": float(np.mean(hrec)), "one_shot_qps": hq_one,
                  "buffers": "pageable host memory", "batches_in_rotation": B, "setup_seconds": time.time() - th,
                  "scan_sel1_qps": scan_qps, "scan_sel1_ids_equal_exact": bool(np.array_equal(h_ids, gt_narrow))}
        idx.close()
        log(f"[bench] index handle, host pointers (CagraIndex::query_range_batch, {B} host batches in rotation): {hq:,.0f} QPS "
            f"({handle['ms_per_call']:.3f} ms per call), recall@{k} {handle['recall_at_10']:.4f}; undivided call {hq_one:,.0f} QPS; "
            f"1 % windows through scan_range_batch {scan_qps:,.0f} QPS, ids equal the exact filtered top-k: {handle['scan_sel1_ids_equal_exact']}")

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
        lanes = [(streams[0], layer, d_seeds, d_lo, d_hi, new_outs(), d_groups0)]
        for st in streams[1:]:
            layer_b = grab.EntryLayer(d_data, n, dim, args.entry_samples, d_ts=d_ts)
            layer_b.build_groups(args.entry_groups, niter=10, seed=1)
            lanes.append((st, layer_b, grab.DeviceArray((nq, max_seeds), np.uint32), grab.DeviceArray((nq,), np.uint64),
                          grab.DeviceArray((nq,), np.uint64), new_outs(), grab.DeviceArray((nq, max(1, args.entry_nprobe)), np.uint32)))
        for w in range(max(len(lanes), args.warmup)):
            one_pass(w, asynchronous=True, lane=lanes[w % len(lanes)])
        grab.synchronize()
        lane_ms = []
        for r in range(max(1, args.repeats)):
            tl = time.perf_counter()
            for s in range(args.steps):
                one_pass(r * args.steps + s, asynchronous=True, lane=lanes[s % len(lanes)])
            grab.synchronize()
            lane_ms.append((time.perf_counter() - tl) / args.steps * 1e3)
        # every (lane, batch) pair that ran must have produced the one-stream result
        same, differing = True, []
        for st in range(min(args.steps, B * len(lanes))):
            got = lanes[st % len(lanes)][5][st % B][0].numpy()
            if not np.array_equal(got, ids_by_batch[st % B]):
                same = False
                differing.append((st % len(lanes), st % B, int((got != ids_by_batch[st % B]).any(axis=1).sum())))
        if differing:
            log(f"[bench] (stream, batch, queries that differ): {differing}")
        two_lanes = {"qps": nq / (float(np.median(lane_ms)) * 1e-3), "ms_per_step": float(np.median(lane_ms)),
                     "ms_per_step_min": float(np.min(lane_ms)), "ms_per_step_max": float(np.max(lane_ms)),
                     "blocks": len(lane_ms), "streams": len(lanes), "results_equal_one_stream": bool(same)}
        log(f"[bench] {len(lanes)} batches in flight (one stream each): {two_lanes['qps']:,.0f} QPS, {two_lanes['ms_per_step']:.3f} ms per step, "
            f"results {'equal' if same else 'DIFFER from'} the one-stream run")
        for p in streams:
            grab.check(grab.lib.grab_stream_destroy(p))

    # kernel duration from HIP events on the kernel's stream, averaged over the same number of launches
    kms, ems, sms = [], [], []
    for s in range(args.steps):
        kms.append(one_pass(s, want_ms=True))
        ems.append(entry_ms_box.value)
        sms.append(layer.last_select_ms if use_entry else 0.0)
    kernel_ms = float(np.mean(kms))
    entry_ms = float(np.mean(ems)) if use_entry else 0.0
    select_ms = float(np.mean(sms)) if use_entry else 0.0
    # algorithmic bytes of each batch from the kernel's own work counters; a launch is charged its own batch's bytes
    batch_bytes, hash_full = [], 0
    for b in range(B):
        one_pass(b, want_counters=True, batch=b)
        ctr = d_ctr.numpy()
        hash_full += int(ctr[:, 5].sum())
        batch_bytes.append(algorithmic_bytes(ctr, nq, dim, deg, k, 4 if rank_mode else 8))  # F is zero when ids are tested
    abytes = float(np.mean([batch_bytes[s % B] for s in range(args.steps)]))
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
        f"-> {achieved:.0f} GB/s; iters mean {ctr[:, 0].mean():.1f} p50 {np.percentile(ctr[:, 0], 50):.0f} p90 {np.percentile(ctr[:, 0], 90):.0f} "
        f"p99 {np.percentile(ctr[:, 0], 99):.0f} max {ctr[:, 0].max()}, F {ctr[:, 3].mean():.0f}, D {ctr[:, 4].mean():.0f}, "
        f"visited-set overflows {hash_full}; entry layer: centroid ranking {entry_ms:.3f} ms = {entry_tflops:.1f} TFLOP/s of fp32-equivalent products (bf16 halves), "
        f"group walk {select_ms:.3f} ms")

    # the same search seeded the way the reference seeds it (itopk random ids of the window), for comparison
    ref_seeding = None
    if use_entry and not args.no_reference_seeding:
        ie, sn, _ = grab.search_plan(grab.WRAP_RANGE, k, 256, args.width, deg, 256)
        one_pass(0, itopk=ie, seeds_n=sn)
        grab.synchronize()
        tt = time.time()
        for s in range(B):
            one_pass(s, itopk=ie, seeds_n=sn)
        grab.synchronize()
        ref_seeding = {"itopk": 256, "seeds_per_query": sn, "qps": nq / ((time.time() - tt) / B),
                       "recall_at_10": float(np.mean([datasets.recall(outs0[b][0].numpy(), gts[b]) for b in range(B)]))}
        log(f"[bench] reference seeding (random window ids, itopk 256): {ref_seeding}")

    # ---- rows of the other configurations (outside the timed headline): cfg3 at 1 % and 50 %, longer lists at the
    # headline's selectivity, cfg2 (unfiltered), and narrow windows on the time-partitioned graph.  Each row: 5 steps
    # over 5 batches' queries after one warm-up, recall over those batches.
    def windows_for(sel):
        hw = [datasets.windows(n, nq, sel, 13 + 100 * b) for b in range(B)]
        dw = [(grab.DeviceArray.from_numpy(a), grab.DeviceArray.from_numpy(c)) for a, c in hw]
        g = [grab.bruteforce_topk(d_data, n, dim, d_qs[b], nq, k, filter_kind=grab.FILTER_RANGE, d_ts=d_ts,
                                  d_win_start=dw[b][0], d_win_end=dw[b][1])[0] for b in range(min(B, 5))]
        host_windows[sel] = hw
        return dw, g

    host_windows = {args.selectivity: h_win}

    def timed_row(label, gt_list, rounds=1, **kw):
        nb = len(gt_list)
        one_pass(0, batch=0, want_counters=True, **kw)
        overflow = int(d_ctr.numpy()[:, 5].sum())
        grab.synchronize()
        tt = time.perf_counter()
        for rnd in range(rounds):   # short steps are timed over several rounds of the batches
            for b in range(nb):
                one_pass(b, batch=b, asynchronous=True, **kw)
        grab.synchronize()
        el = (time.perf_counter() - tt) / (nb * rounds)
        r = float(np.mean([datasets.recall(outs0[b][0].numpy(), gt_list[b]) for b in range(nb)]))
        row = dict(label, qps=nq / el, ms_per_step=el * 1e3, recall_at_10=r, visited_set_overflows=overflow)
        if label.get("cfg") == "cfg3 op":
            # the search kernel of this operating point against the memory roofline, as for the headline: algorithmic
            # bytes from the kernel's counters, duration from HIP events on its stream
            ab = algorithmic_bytes(d_ctr.numpy(), nq, dim, deg, k, 4 if rank_mode else 8)
            km = float(np.mean([one_pass(b, batch=b % nb, want_ms=True, **kw) for b in range(10)]))
            row.update(kernel_ms=km, algorithmic_bytes=ab, frac_of_hbm_peak=ab / (km * 1e-3) / 8e12)
        log(f"[configs] {row}")
        return row

    configs, partitioned_build_s = None, None
    if not args.no_configs and use_entry and args.entry_groups > 0 and not args.read_timestamps and args.partition_buckets == 0:
        configs = []
        per_sel = {}
        for sel in (0.01, 0.50):
            per_sel[sel] = windows_for(sel)
        per_sel[args.selectivity] = (d_wins, gts[:min(B, 5)])
        for sel in (0.01, args.selectivity, 0.50):
            dw, g = per_sel[sel]
            for itk in (64, 128, 256):
                if sel == args.selectivity and itk == args.itopk:
                    continue   # the headline itself
                ie, sn, _ = grab.search_plan(grab.WRAP_RANGE, k, itk, args.width, deg, args.seeds)
                bl = auto_bitlen(sn, args.width, deg, sel)
                configs.append(timed_row({"cfg": "cfg3", "graph_short": "global", "selectivity": sel, "itopk": itk,
                                          "hash_bitlen": bl, "seeding": "entry layer"}, g, itopk=ie, seeds_n=sn, bitlen=bl,
                                         entry=True, wins=dw))
        # The headline keeps CagraIndex's iteration limit of 50 (src/cagraIndex.cu:28).  Where the same search stands with
        # the limit of the reference's own search test (10, tests/test_cagra_hotpotqa.cpp:238), and with 16 listed seeds
        # a query instead of 32 - same graph, itopk, width and degree; recall stays above 0.95:
        if id_filter and args.entry_mode == "list":
            dw, g = per_sel[args.selectivity]
            for mi, ln in ((10, None), (10, 16)):
                configs.append(timed_row({"cfg": "cfg3 op", "graph_short": "global",
                                          "selectivity": args.selectivity, "itopk": args.itopk, "max_iterations": mi,
                                          "listed_seeds": n_seeds if ln is None else ln, "hash_bitlen": args.hash_bitlen,
                                          "seeding": "entry layer"}, g, rounds=8, max_iter=mi, list_n=ln, wins=dw))
        # cfg2: unfiltered search, the parameters of cagra::search (itopk 64, width 4, itopk/4 formula seeds, 8192 slots)
        gt_all = [grab.bruteforce_topk(d_data, n, dim, d_qs[b], nq, k)[0] for b in range(min(B, 5))]
        ie, sn, _ = grab.search_plan(grab.WRAP_SEARCH, k, 64, args.width, deg, 0)
        configs.append(timed_row({"cfg": "cfg2 unfiltered", "graph_short": "global", "itopk": 64, "hash_bitlen": 13,
                                  "seeding": "reference (itopk/4 formula ids)", "seeding_short": "reference formula ids"},
                                 gt_all, unfiltered=True, itopk=ie, seeds_n=sn, bitlen=13, entry=False))
        ie, sn, _ = grab.search_plan(grab.WRAP_SEARCH_OPT, k, 64, args.width, deg, 32)
        configs.append(timed_row({"cfg": "cfg2 unfiltered", "graph_short": "global", "itopk": 64, "hash_bitlen": 13,
                                  "seeding": "entry layer, 32 nearest sample rows", "seeding_short": "entry layer 32"},
                                 gt_all, unfiltered=True, itopk=ie, seeds_n=32, bitlen=13, entry=True))
        # the time-partitioned graph (100 buckets of consecutive rows, 48 local + 16 remote slots), which is what answers
        # narrow windows
        tpb = time.time()
        nbk = 100
        sizes = [n * (b + 1) // nbk - n * b // nbk for b in range(nbk)]
        d_pgraph = grab.build_time_partitioned_graph(d_data, n, dim, grab.DeviceArray.from_numpy(
            np.repeat(np.arange(nbk, dtype=np.uint64), sizes)), sizes, deg, 48)
        grab.synchronize()
        t_part = time.time() - tpb
        partitioned_build_s = t_part
        for sel in (0.01, args.selectivity, 0.50):
            dw, g = per_sel[sel]
            for itk in (64, 128, 256):
                ie, sn, _ = grab.search_plan(grab.WRAP_RANGE, k, itk, args.width, deg, args.seeds)
                bl = auto_bitlen(sn, args.width, deg, sel, 48 / deg)
                configs.append(timed_row({"cfg": "cfg3", "graph_short": f"part{nbk}x48", "graph":
                                          f"time-partitioned, {nbk} buckets, 48 local slots (build {t_part:.2f} s)",
                                          "selectivity": sel, "itopk": itk, "hash_bitlen": bl, "seeding": "entry layer"},
                                         g, itopk=ie, seeds_n=sn, bitlen=bl, entry=True, graph=d_pgraph, wins=dw))
        d_pgraph.free()
        # The exact answer instead of a graph search (timestamps are in row order, so a window is an interval of row ids):
        # the intervals scanned on the matrix cores over a base prepared once.  Wall time of the call - host tables,
        # their upload, contraction, selection, exact re-scoring - over the same batches.
        if id_filter:
            tsb = time.time()
            scan_base = grab.ScanBase(d_data, n, dim)
            grab.synchronize()
            t_scan_base = time.time() - tsb
            for sel in (0.001, 0.01, args.selectivity, 0.50):
                if sel not in per_sel:
                    per_sel[sel] = windows_for(sel)
                g = per_sel[sel][1]
                hw = host_windows[sel]
                for b in range(len(g)):   # warm: the base's scratch grows to this size of call
                    scan_base.window_topk(d_qs[b], nq, k, hw[b][0], hw[b][1], d_out=outs0[b])
                grab.synchronize()
                tt = time.perf_counter()
                for b in range(len(g)):
                    scan_base.window_topk(d_qs[b], nq, k, hw[b][0], hw[b][1], d_out=outs0[b])
                el = (time.perf_counter() - tt) / len(g)
                got = [outs0[b][0].numpy() for b in range(len(g))]
                row = {"cfg": "cfg3 scan", "method": "exact window scan", "selectivity": sel, "qps": nq / el, "ms_per_step": el * 1e3,
                       "recall_at_10": float(np.mean([datasets.recall(got[b], g[b]) for b in range(len(g))])),
                       "ids_equal_exact_filtered_topk": bool(all(np.array_equal(got[b], g[b]) for b in range(len(g)))),
                       "queries_redone_row_by_row": int(grab.last_knn_exact_rows()), "prepare_base_seconds": t_scan_base}
                configs.append(row)
                log(f"[configs] {row}")
            scan_base.close()

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
                    one_pass(0, itopk=ie, seeds_n=sn, win=w, entry=ent, bitlen=bl, want_counters=True, batch=0)
                    overflow = int(d_ctr.numpy()[:, 5].sum())
                    grab.synchronize()
                    tt = time.time()
                    for s in range(5):
                        one_pass(s, itopk=ie, seeds_n=sn, win=w, entry=ent, bitlen=bl, batch=0)
                    grab.synchronize()
                    row = {"selectivity": sel, "itopk": itk, "itopk_eff": ie, "seeding": seeding, "seeds": sn, "hash_bitlen": bl,
                           "qps": nq / ((time.time() - tt) / 5), "recall": datasets.recall(outs0[0][0].numpy(), g),
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
        cids, _, cctr = oracle.search(data, graph, queries[:m], k, itopk_eff, args.width, args.max_iter, args.hash_bitlen,
                                   n_seeds, 0x5EED0000, seeds=seeds, filter_kind=oracle.FILTER_RANGE, ts=ts,
                                   win_start=ws[:m], win_end=we[:m], flags=search_flags & 3, threads=threads)
        tcs = time.time() - tc
        # like for like: the GPU on exactly this sample with exactly these seeds, and the GPU's own (grouped) seeds on
        # the same queries
        d_given = grab.DeviceArray.from_numpy(np.ascontiguousarray(seeds))
        one_pass(100, batch=0, count=m, given_seeds=d_given, want_counters=True)
        gpu_same = outs0[0][0].numpy()[:m].copy()
        gpu_same_ctr = d_ctr.numpy()[:m].copy()
        one_pass(100, batch=0)
        gpu_own = outs0[0][0].numpy()[:m].copy()
        mb = min(200, m)
        tbf = time.time()
        oracle.bruteforce_topk(data, queries[:mb], k, filter_kind=oracle.FILTER_RANGE, ts=ts, win_start=ws[:mb],
                               win_end=we[:mb], threads=threads)
        tbfs = time.time() - tbf
        cpu = {"value": m / tcs, "unit": "queries/s", "cores": threads, "kind": "port",
               "sample_short": f"first {m} of {nq} queries, oracle search + exact seed selection, OpenMP",
               "sample": f"first {m} of the {nq} queries, same graph/params/windows, CPU restatement of the reference "
                         f"search (OpenMP over queries); seeds = the exact nearest in-window sample rows, brute force "
                         f"over the sample included in the time (the GPU's grouped selection approximates these seeds)",
               "recall_at_k": datasets.recall(cids, gt[:m]),
               "gpu_recall_same_queries_same_seeds": datasets.recall(gpu_same, gt[:m]),
               "gpu_ids_equal_cpu_same_seeds": bool(np.array_equal(gpu_same, cids)),
               "gpu_counters_equal_cpu_same_seeds": bool(np.array_equal(gpu_same_ctr[:, [0, 1, 2, 4]], cctr[:, [0, 1, 2, 4]])),
               "gpu_recall_same_queries_grouped_seeds": datasets.recall(gpu_own, gt[:m]),
               "exact_filtered_bruteforce_qps": mb / tbfs, "exact_bruteforce_sample": f"first {mb} queries"}
        log(f"[bench] same {m} queries, same seeds: recall CPU {cpu['recall_at_k']:.5f} / GPU {cpu['gpu_recall_same_queries_same_seeds']:.5f} "
            f"(ids equal: {cpu['gpu_ids_equal_cpu_same_seeds']}, counters equal: {cpu['gpu_counters_equal_cpu_same_seeds']}); GPU with its "
            f"grouped seeds on these queries {cpu['gpu_recall_same_queries_grouped_seeds']:.5f}")
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

    # cfg4 and cfg5 have benchmarks of their own; their JSON lines ride along so that one run records every configuration
    side = None
    if not (args.no_side_benches or args.no_configs) and default_shape(args):
        import subprocess
        side = {}
        for key, cmd in (("cfg4_streaming_insert", ["bench_streaming_insert.py"]),
                         ("cfg5_bucket_filter_1Mx768", ["bench_bucket_filter.py", "--itopk", "64", "128"])):
            ts0 = time.time()
            try:
                r = subprocess.run([sys.executable, "-u", os.path.join(ROOT, cmd[0])] + cmd[1:], stdout=subprocess.PIPE,
                                   stderr=subprocess.DEVNULL, timeout=600, check=True)
                side[key] = json.loads(r.stdout.decode().strip().splitlines()[-1])
            except Exception as e:  # a side run must not take the headline down with it
                side[key] = {"error": repr(e)}
            log(f"[bench] {cmd[0]}: {time.time() - ts0:.1f}s")

    # Two kernels carry the step: the beam search (random row gathers: HBM-bound) and the entry
    # layer's contraction (fp32 MFMA-bound).  "roofline" describes the one with the longer launch.
    traffic = load_traffic((n, nq, dim, deg, args.itopk, args.width, args.max_iter, args.hash_bitlen, args.selectivity,
                            args.entry_samples, args.entry_mode, args.entry_list, args.filter_first, args.read_timestamps,
                            args.entry_groups, args.entry_nprobe, args.entry_min_rows, B))
    rl_search = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                 "traffic": traffic["search"],
                 "kernel_short": "search_wave_reg_kernel" if args.decomposition != "block" and nq >= 1024 else "search_kernel",
                 "kernel": "search_wave_reg_kernel (id-interval filter)" if args.decomposition != "block" and nq >= 1024
                 else "search_kernel", "kernel_ms": kernel_ms, "algorithmic_bytes": abytes}
    rl_entry = {"bound": "mfma", "achieved": entry_tflops, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": entry_tflops / MFMA_FP32_PEAK_TFLOPS, "traffic": traffic["entry"],
                "kernel_short": "centroid_probe_kernel" if args.entry_groups > 0 else "tile_topk_kernel",
                "kernel": ("centroid_probe_kernel (entry-point layer: queries x centroids, selection in the accumulators)"
                           if args.entry_groups > 0 else "tile_topk_kernel (dense-store mode, entry-point layer)"),
                "kernel_ms": entry_ms,
                "algorithmic_flops": entry_flops}
    if args.entry_groups > 0:
        # the centroid ranking forms every fp32 product from bf16 halves: three bf16 matrix-instruction products each
        rl_entry.update({"achieved": 3.0 * entry_tflops, "peak": MFMA_BF16_PEAK_TFLOPS, "frac": 3.0 * entry_tflops / MFMA_BF16_PEAK_TFLOPS,
                         "executed_flops": 3.0 * entry_flops, "fp32_equivalent_tflops": entry_tflops,
                         "kernel": "centroid_probe_kernel (entry-point layer: queries x centroids from bf16 halves on "
                                   "v_mfma_f32_16x16x32_bf16, selection in the accumulators)"})
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
        "settling": {"ms": args.settle_ms, "untimed_steps": settle_steps},
        "ms_per_step": ms_per_step,
        "ms_per_step_spread": spread,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload_short": f"cfg3: timestamp range-filtered search, {n}x{dim} fp32 mixture, {nq} queries/step, "
                              f"{args.selectivity:g} windows, L2",
            "seeding_short": ((f"entry layer {args.entry_samples} samples/{args.entry_groups} groups/nprobe {args.entry_nprobe}/"
                               f"{args.entry_mode} {entry_seeds(args)}") if use_entry else "reference (random window ids)"),
            "filter_short": "place" if rank_mode else "id interval" if id_filter else "timestamp per neighbour",
            "workload": f"timestamp range-filtered search, {n} x {dim} fp32 Gaussian mixture ({args.centroids} centroids), "
                        f"{nq} queries, window selectivity {args.selectivity:g}, L2",
            "batches": f"{B} distinct pre-generated query/window batches, one per step in rotation",
            "k": k, "itopk": args.itopk, "itopk_eff": itopk_eff, "search_width": args.width,
            "max_iterations": args.max_iter, "hash_bitlen": args.hash_bitlen, "graph_degree": deg,
            "intermediate_degree": args.intermediate, "seeds_per_query": n_seeds,
            "graph": (f"time-partitioned, {args.partition_buckets} buckets, local degree {args.local_degree}"
                      if args.partition_buckets > 0 else "global"),
            "seeding": ((f"entry-point layer, {args.entry_samples} sample rows"
                         + (f" in {args.entry_groups} k-means groups, {args.entry_nprobe} nearest centroids kept, groups walked "
                            f"until {args.entry_min_rows} in-window rows; " + {"list": f"these rows (at most {args.entry_list}) are the seeds",
                                                                            "fused": f"these rows (at most {args.entry_list}) are the seeds, "
                                                                                     "listed by the search kernel itself",
                                                                            "scored": f"their {args.seeds} nearest are the seeds"}[args.entry_mode]
                            if args.entry_groups > 0 else ""))
                        if use_entry else "random ids of the window (reference)"),
            "filter": ("place in timestamp order read per visited neighbour, 4 bytes" if rank_mode else
                       "id interval of the window (timestamps = insertion order)" if id_filter else "timestamp read per visited neighbour"),
        },
        "recall_at_10": rec,
        "recall_at_10_per_batch": recalls,
        "recall_target_met": bool(rec >= 0.95),
        "build_seconds": build_s,
        "build": {"knn_seconds": t_knn, "knn_kernel_ms": knn_ms, "knn_tflops": knn_tflops,
                  "knn_pipe": "bf16" if knn_on_bf16 else "fp32",
                  "knn_matrix_pipe": "bf16 (rows split into two bf16 halves, three instructions a product, fp32 sums)" if knn_on_bf16 else "fp32",
                  "knn_flop_executed": knn_flop_bf16 if knn_on_bf16 else knn_flop, "knn_flop_executed_fp32_instructions": knn_flop,
                  "knn_fp32_equivalent_tflops": ((knn_flop_bf16 / 3.0 if knn_on_bf16 else knn_flop) / (knn_ms * 1e-3) / 1e12) if knn_ms else 0.0,
                  "knn_flop_all_pairs": 2.0 * n * n * dim, "knn_rows_redone": knn_redone, "knn_rows_not_proven_redone_exactly": knn_exact_rows,
                  "optimize_seconds": t_opt,
                  "mfma_peak_tflops": knn_peak, "mfma_frac": knn_tflops / knn_peak},
        "roofline": roofline,
        "roofline_secondary": roofline_secondary,
        "visited_set_overflows": hash_full,
        "pcie_inclusive_qps": pcie_qps,
        "handle": handle,
        "two_batches_in_flight": two_lanes,
        "entry_layer": ({"samples": args.entry_samples, "groups": args.entry_groups, "nprobe": args.entry_nprobe,
                         "min_rows": args.entry_min_rows, "mode": args.entry_mode, "centroid_ranking_ms": entry_ms,
                         "centroid_ranking_arithmetic": "fp32 operands split into bf16 halves (hi*hi + lo*hi + hi*lo), fp32 sums",
                         "group_walk_ms": select_ms}
                        if use_entry else None),
        "reference_seeding": ref_seeding,
        "cpu_baseline": cpu,
        "configs": configs,
        "partitioned_build_seconds": partitioned_build_s,
        "configs_other_benchmarks": side,
    }
    if sweep is not None:
        result["sweep"] = sweep
    # everything measured goes to stderr and to a side file; stdout carries one short line
    detail = json.dumps(result)
    log("[bench] detail " + detail)
    try:
        os.makedirs(os.path.join(ROOT, "gpurun_out"), exist_ok=True)
        with open(os.path.join(ROOT, "gpurun_out", "bench_detail.json"), "w") as f:
            f.write(detail + "\n")
    except OSError as e:
        log(f"[bench] detail file not written: {e}")
    print(compact_line(result), flush=True)


if __name__ == "__main__":
    main()
