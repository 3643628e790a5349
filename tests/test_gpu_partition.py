"""Time-partitioned graph on the GPU against the CPU restatement (bit for bit), and what it buys:
recall of searches confined to a bucket."""
import numpy as np
import pytest

import datasets

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("total,local,buckets", [(32, 28, 7), (16, 8, 12), (24, 0, 5)])
def test_remote_edge_kernels_match_oracle(oracle, grab, total, local, buckets):
    rng = np.random.default_rng(total + local)
    n = 5000
    gk = grab.remote_global_k(total, local)
    assert gk == oracle.remote_global_k(total, local)
    ts = np.sort(rng.integers(0, buckets, n)).astype(np.uint64)
    ts[0], ts[-1] = 0, buckets - 1
    graph = rng.integers(0, n, (n, total)).astype(np.uint32)
    cand = np.stack([rng.choice(n, gk, replace=False) for _ in range(n)]).astype(np.uint32)
    cand[rng.random((n, gk)) < 0.02] = 0xFFFFFFFF
    d_graph, d_ts = grab.DeviceArray.from_numpy(graph), grab.DeviceArray.from_numpy(ts)
    grab.update_remote_edges(d_graph, d_ts, grab.DeviceArray.from_numpy(cand), n, total, local, gk)
    exp = oracle.remote_edges(cand, ts, graph, total, local)
    assert np.array_equal(d_graph.numpy(), exp)
    grab.enhance_global_connectivity(d_graph, n, total, local)
    assert np.array_equal(d_graph.numpy(), oracle.inject_reverse_remote(exp, total, local))


@pytest.mark.parametrize("metric,sizes", [(0, [700, 300, 1100, 40, 860]), (1, [700, 300, 1100, 40, 860]),
                                          (0, [900, 5200, 300, 4500])])
def test_partitioned_build_matches_oracle(oracle, grab, metric, sizes):
    # one bucket smaller than the intermediate degree; in the last case the first bucket is small and later ones are
    # large - they outgrow the block of scratch memory that the first one sized, and are big enough for the symmetric
    # pass on bf16 instructions
    n, dim, total, local = sum(sizes), 64, 32, 24
    data = datasets.unit_rows(n, dim, 5) if metric else datasets.gaussian(n, dim, 5)
    ts = np.repeat(np.arange(len(sizes), dtype=np.uint64), sizes)
    got = grab.build_time_partitioned_graph(grab.DeviceArray.from_numpy(data), n, dim, grab.DeviceArray.from_numpy(ts), sizes, total,
                                            local, metric).numpy()
    exp = oracle.build_time_partitioned(data, ts, sizes, total, local, metric)
    bad = np.nonzero((got != exp).any(axis=1))[0]
    assert bad.size == 0, f"{bad.size} rows differ, first {bad[0]}: {exp[bad[0]]} vs {got[bad[0]]}"


def test_index_partitioned_build_serves_bucket_queries(oracle, grab):
    # 40 buckets of 500 rows, 50 clusters: a bucket holds ~10 rows of a cluster.  In the global graph the 32 edges of
    # a row stay inside its cluster and mostly leave the bucket, so a search confined to one bucket starves; the
    # bucket's own graph connects the bucket.
    nb, per, dim, deg, local, k = 40, 500, 64, 32, 24, 10
    n = nb * per
    data = datasets.mixture(n, dim, 50, 10, 11)
    ts = np.repeat(np.arange(nb, dtype=np.uint64), per)
    q = datasets.mixture(200, dim, 50, 10, 12)
    recalls = {}
    for kind in ("global", "partitioned"):
        idx = grab.CagraIndex(dim, deg, vmm_max_bytes=1 << 28, local_degree=local)
        idx.setQueryParams(64, 4, 0, 50, 13)
        idx.set_seed(3)
        idx.add(data, ts)
        idx.build() if kind == "global" else idx.build_partitioned()
        g = idx.get_graph()
        if kind == "partitioned":
            assert np.array_equal(g, oracle.build_time_partitioned(data, ts, [per] * nb, deg, local))
            assert (ts[g[:, :local]] == ts[:, None]).all()
        hits = tot = 0
        for b in (0, 13, 39):
            ids, dist = idx.query_range(q, k, 0.5, b, b + 1)
            gt, _ = oracle.bruteforce_topk(data, q, k, filter_kind=oracle.FILTER_RANGE, ts=ts, win=(b, b + 1))
            v = ids[ids >= 0]
            assert (ts[v] == b).all()
            hits += datasets.recall(ids, gt)
            tot += 1
            loc, _ = idx.query_local(q, k, b)   # local edges only
            assert (ts[loc[loc >= 0]] == b).all() or kind == "global"
            if kind == "partitioned":
                assert datasets.recall(loc, gt) > 0.9
        recalls[kind] = hits / tot
        idx.close()
    print("recall@10 inside one bucket:", recalls)
    assert recalls["partitioned"] > 0.95 and recalls["partitioned"] > recalls["global"] + 0.1
