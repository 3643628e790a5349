"""bench.py's last stdout line is read back from a tail of a few thousand characters: it must stay short and whole.

The line builder is fed canned values of the size a full run produces (every configuration row, both side
benchmarks, long text fields and per-batch trajectories in the detail) and the result must parse, stay far below
the limit and carry the fields a reader of the line needs.
"""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402


def canned():
    configs = []
    for graph in ("global", "part100x48"):
        for sel in (0.01, 0.1, 0.5):
            for itk in (64, 128, 256):
                configs.append({"cfg": "cfg3", "graph_short": graph, "graph": "time-partitioned, 100 buckets, 48 local slots " * 3,
                                "selectivity": sel, "itopk": itk, "hash_bitlen": 13, "seeding": "entry layer " * 10,
                                "qps": 12345678.123456789, "ms_per_step": 1.2345678901, "recall_at_10": 0.993812345678,
                                "visited_set_overflows": 0, "kernel": "wave"})
    for mi in (10, 10):
        configs.append({"cfg": "cfg3 op", "graph_short": "global", "selectivity": 0.1, "itopk": 64,
                        "max_iterations": mi, "listed_seeds": 32, "hash_bitlen": 10, "qps": 67812345.678, "recall_at_10": 0.97234567,
                        "visited_set_overflows": 0})
    for s in ("reference formula ids", "entry layer 32"):
        configs.append({"cfg": "cfg2 unfiltered", "graph_short": "global", "itopk": 64, "hash_bitlen": 13, "seeding_short": s,
                        "qps": 9687817.820972573, "recall_at_10": 0.9999520000000001, "visited_set_overflows": 0})
    for sel in (0.001, 0.01, 0.1, 0.5):
        configs.append({"cfg": "cfg3 scan", "method": "exact window scan", "selectivity": sel, "qps": 12912345.678, "ms_per_step": 0.7741234,
                        "recall_at_10": 1.0, "ids_equal_exact_filtered_topk": True, "queries_redone_row_by_row": 0,
                        "prepare_base_seconds": 0.0123456})
    batches = [{"batch": b, "rows": 500000 + 10000 * b, "insert_vectors_per_s": 239443.28048912765, "recall_at_10": 0.9567,
                "query_qps_host_buffers": 3518711.409395973, "mapped_bytes": 522190848, "logical_bytes": 519920000} for b in range(1, 51)]
    for b in (24, 49):
        batches[b].update({"from_scratch_build_s": 0.4225287437438965, "from_scratch_recall_at_10": 0.9895,
                           "recall_drift": -0.046700000000000075})
    cfg4 = {"workload": "streaming insert " * 12, "insert_vectors_per_s": 223456.789, "insert_seconds_total": 2.24,
            "initial_build_s": 0.2345678, "recall_before_inserts": 0.960123, "recall_min": 0.92123, "recall_last": 0.922123,
            "mapped_bytes_final": 780100000, "logical_bytes_final": 776000000, "mapped_over_logical": 1.00528,
            "checkpoints": [r for r in batches if "recall_drift" in r], "batches": batches}
    cfg5 = {"workload": "bucket-filtered search " * 10, "build_seconds": 8.812345, "knn_pipe": "bf16", "knn_tflops": 800.123,
            "search": [{"method": m, "itopk": i, "seeds": i, "entry_layer_ms": None, "kernel_ms": 16.612345, "qps": 601234.567,
                        "recall_at_10": 0.378123, "algorithmic_bytes": 100600000000, "achieved_GBps": 6012.345,
                        "frac_of_hbm_peak": 0.7512345, "mfma_frac": 0.3, "mean_iterations": 49.9, "rows_scored_per_query": 3264.5}
                       for m, i in (("graph", 64), ("graph", 128), ("graph", 256), ("exact bucket scan", 0))]}
    return {
        "metric": "filtered QPS @ recall@10>=0.95 (1M x 128)", "value": 56912345.678901, "unit": "queries/s", "n_gpus": 1,
        "steps": 20, "warmup": 5, "settling": {"ms": 40.0, "untimed_steps": 240}, "ms_per_step": 0.17561234567,
        "ms_per_step_spread": {"blocks": 5, "min": 0.17521234, "median": 0.17561234, "max": 0.17591234, "all": [0.1756] * 5},
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload_short": "cfg3: timestamp range-filtered search, 1000000x128 fp32 mixture, 10000 queries/step, 0.1 windows, L2",
                   "seeding_short": "entry layer 65536 samples/768 groups/nprobe 16/list 32", "filter_short": "id interval",
                   "workload": "x" * 300, "batches": "y" * 100, "k": 10, "itopk": 64, "itopk_eff": 64, "search_width": 4,
                   "max_iterations": 50, "hash_bitlen": 10, "graph_degree": 64, "intermediate_degree": 128, "seeds_per_query": 32,
                   "graph": "global", "seeding": "z" * 400, "filter": "w" * 100},
        "recall_at_10": 0.99381234, "recall_at_10_per_batch": [0.9938] * 8, "recall_target_met": True, "build_seconds": 0.5812345,
        "build": {"knn_seconds": 0.5312345, "knn_kernel_ms": 500.12345, "knn_tflops": 793.12345, "knn_pipe": "bf16",
                  "knn_matrix_pipe": "bf16 " * 20, "knn_flop_executed": 3.97e14, "knn_flop_executed_fp32_instructions": 1e12,
                  "knn_fp32_equivalent_tflops": 264.123, "knn_flop_all_pairs": 2.56e14, "knn_rows_redone": 407,
                  "knn_rows_not_proven_redone_exactly": 0, "optimize_seconds": 0.0512345, "mfma_peak_tflops": 2500.0, "mfma_frac": 0.31712345},
        "roofline": {"bound": "hbm", "achieved": 5501.2345, "peak": 8000.0, "unit": "GB/s", "frac": 0.68812345, "traffic": 756700000,
                     "kernel_short": "search_wave_reg_kernel", "kernel": "k" * 80, "kernel_ms": 0.14341234, "algorithmic_bytes": 789372096.0},
        "roofline_secondary": {"bound": "mfma", "achieved": 229.12345, "peak": 2500.0, "unit": "TFLOP/s", "frac": 0.0912345,
                               "traffic": 9365000, "kernel_short": "centroid_probe_kernel", "kernel": "k" * 150, "kernel_ms": 0.02581234,
                               "algorithmic_flops": 1966080000.0, "executed_flops": 5898240000.0, "fp32_equivalent_tflops": 76.2},
        "visited_set_overflows": 0, "pcie_inclusive_qps": 28412345.678,
        "handle": {"qps": 31234567.89, "ms_per_call": 0.32012345, "recall_at_10": 0.99391234, "buffers": "pageable host memory",
                   "one_shot_qps": 15512345.6},
        "two_batches_in_flight": {"qps": 68612345.6, "ms_per_step": 0.14571234, "ms_per_step_min": 0.145, "ms_per_step_max": 0.146,
                                  "blocks": 5, "streams": 2, "results_equal_one_stream": True},
        "entry_layer": {"samples": 65536, "groups": 768, "nprobe": 16, "min_rows": 16, "mode": "list", "centroid_ranking_ms": 0.0258,
                        "centroid_ranking_arithmetic": "a" * 90, "group_walk_ms": 0.0116},
        "reference_seeding": {"itopk": 256, "seeds_per_query": 256, "qps": 9112345.67, "recall_at_10": 0.22712345},
        "cpu_baseline": {"value": 11121.12345, "unit": "queries/s", "cores": 16, "kind": "port",
                         "sample_short": "first 2000 of 10000 queries, oracle search + exact seed selection, OpenMP", "sample": "s" * 400,
                         "recall_at_k": 0.99431234, "gpu_recall_same_queries_same_seeds": 0.9943, "gpu_ids_equal_cpu_same_seeds": True,
                         "gpu_counters_equal_cpu_same_seeds": True, "gpu_recall_same_queries_grouped_seeds": 0.9941,
                         "exact_filtered_bruteforce_qps": 867.12345, "exact_bruteforce_sample": "first 200 queries",
                         "hnsw": {"rows": 1000000, "M": 32, "ef_construction": 200, "ef_search": 128, "threads": 16,
                                  "build_seconds": 24.512345, "insert_vectors_per_s": 41612.345, "filtered_qps": 41012.345,
                                  "recall_at_10": 0.99912345, "queries": 1000, "filter": "f" * 70}},
        "configs": configs, "partitioned_build_seconds": 0.7912345,
        "configs_other_benchmarks": {"cfg4_streaming_insert": cfg4, "cfg5_bucket_filter_1Mx768": cfg5},
    }


def test_line_is_short_whole_and_carries_the_contract():
    full = canned()
    assert len(json.dumps(full)) > 15000   # the detail is long; the line must not be
    line = bench.compact_line(full)
    assert "\n" not in line
    assert len(line) < 4500, len(line)
    assert len(line) < bench.MAX_LINE_CHARS < 8000
    got = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "recall_at_10", "build_seconds", "roofline", "roofline_secondary", "cpu_baseline", "configs",
                "handle_qps"):
        assert key in got, key
    assert got["value"] > 5e7 and got["n_gpus"] == 1 and got["vs_baseline"] is None
    assert "workload" in got["config"] and "model" not in got["config"]
    rl = got["roofline"]
    assert rl["bound"] == "hbm" and rl["unit"] == "GB/s" and abs(rl["frac"] - rl["achieved"] / rl["peak"]) < 1e-3
    assert rl["traffic"] == 756700000
    cpu = got["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] == 16 and cpu["value"] > 0 and cpu["unit"] == "queries/s" and cpu["sample"]
    assert cpu["hnsw"]["filtered_qps"] > 0
    scan = got["configs"]["cfg3_exact_scan"]
    assert scan["columns"][0] == "selectivity" and len(scan["rows"]) == 4 and scan["rows"][1][2] == 1.0 and scan["rows"][1][3] is True
    sweep = got["configs"]["cfg3_sweep"]
    cols, rows = sweep["columns"], sweep["rows"]
    assert len(rows) == 18 and all(len(r) == len(cols) for r in rows)
    qi, ri = cols.index("qps"), cols.index("recall_at_10")
    assert all(r[qi] > 0 and 0 < r[ri] <= 1 for r in rows)
    assert len(got["configs"]["cfg3_other"]) == 2 and len(got["configs"]["cfg2"]) == 2
    assert got["configs"]["cfg2"][0]["qps"] > 0
    assert got["cfg4"]["insert_vectors_per_s"] > 0 and len(got["cfg4"]["checkpoints"]) == 2 and "batches" not in got["cfg4"]
    assert len(got["cfg5"]["search"]) == 4


def test_line_survives_missing_optional_parts():
    full = canned()
    for key in ("roofline_secondary", "cpu_baseline", "configs", "two_batches_in_flight", "reference_seeding", "handle",
                "configs_other_benchmarks"):
        full[key] = None
    got = json.loads(bench.compact_line(full))
    assert got["roofline"]["frac"] > 0 and got["cpu_baseline"] is None and got["configs"] is None
    full["configs_other_benchmarks"] = {"cfg4_streaming_insert": {"error": "TimeoutExpired()"}}
    assert json.loads(bench.compact_line(full))["cfg4"] == {"error": "TimeoutExpired()"}


def test_an_overlong_line_is_refused():
    full = canned()
    full["configs"] = full["configs"] * 6
    try:
        bench.compact_line(full)
    except AssertionError as e:
        assert "characters" in str(e)
    else:
        raise AssertionError("an overlong line went through")


def test_traffic_figures_are_tied_to_kernel_sources_and_configuration(tmp_path, monkeypatch):
    monkeypatch.setattr(bench, "TRAFFIC_FILE", str(tmp_path / "traffic.txt"))
    bench.record_traffic(["search=1000", "entry=20"])
    assert bench.load_traffic(bench.PMC_CONFIG) == {"search": 1000, "entry": 20}
    other = list(bench.PMC_CONFIG)
    other[1] = 20_000
    assert bench.load_traffic(other) == {"search": None, "entry": None}
    # a kernel source that changed since the figure was recorded: the figure is dropped
    monkeypatch.setattr(bench, "source_digest", lambda kernel: "0" * 16 if kernel == "search" else "f" * 16)
    assert bench.load_traffic(bench.PMC_CONFIG) == {"search": None, "entry": None}
    monkeypatch.setattr(bench, "TRAFFIC_FILE", str(tmp_path / "absent.txt"))
    assert bench.load_traffic(bench.PMC_CONFIG) == {"search": None, "entry": None}
