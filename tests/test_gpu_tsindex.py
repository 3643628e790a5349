"""k-means and the two-level timestamp index (timestamp::TimeStampIndex)."""
import numpy as np
import pytest

import datasets

pytestmark = pytest.mark.gpu


def test_kmeans_matches_oracle_and_is_lloyd(oracle, grab):
    n, dim, k = 3000, 32, 40
    data = datasets.mixture(n, dim, 25, 3, 4, sigma=6.0)
    cent, assign = grab.kmeans(data, k, 12, 99)
    ecent, eassign = oracle.kmeans(data, k, 12, 99)
    assert np.array_equal(cent.view(np.uint32), ecent.view(np.uint32)) and np.array_equal(assign, eassign)
    # every row sits with its nearest centroid; the objective does not increase with more iterations
    d = ((data[:, None, :] - cent[None, :, :]) ** 2).sum(axis=2)
    assert np.array_equal(d.argmin(axis=1), assign)
    obj = lambda c, a: float(((data - c[a]) ** 2).sum())
    c3, a3 = grab.kmeans(data, k, 3, 99)
    assert obj(cent, assign) <= obj(c3, a3) + 1e-3
    # a fixed point of Lloyd: every centroid with rows is the mean of its rows (one more assignment round ran after
    # the last update, so compare with the means under the assignment that produced the centroids: 0 iterations more)
    c_more, a_more = grab.kmeans(data, k, 40, 99)
    for c in range(k):
        rows = data[a_more == c]
        if len(rows) and np.array_equal(a_more, grab.kmeans(data, k, 41, 99)[1]):
            assert np.allclose(c_more[c], rows.mean(axis=0), rtol=1e-5, atol=1e-4)


def test_timestamp_index_routes_queries_to_the_right_buckets(oracle, grab):
    # 6 timestamps; every timestamp's rows come from its own part of space (own centroids), so a query near a
    # bucket's rows must be routed there by the virtual layer
    dim, per, nb, k = 64, 1500, 6, 10
    rng = np.random.default_rng(11)
    parts, ts = [], []
    for b in range(nb):
        parts.append(datasets.mixture(per, dim, 20, 100 + b, 200 + b, sigma=8.0))
        ts.append(np.full(per, 1000 + 10 * b, np.uint64))
    data, ts = np.concatenate(parts), np.concatenate(ts)
    order = rng.permutation(len(data))         # arrival order mixes the timestamps
    data, ts = data[order], ts[order]
    idx = grab.TimeStampIndex(dim, 32)
    first = idx.insert(data[:5000], ts[:5000])
    second = idx.insert(data[5000:], ts[5000:])
    assert (first, second) == (0, 5000) and idx.size() == len(data) and idx.num_buckets() == nb
    t0, l0 = idx.locate(7)
    assert t0 == ts[7] and l0 == int((ts[:7] == ts[7]).sum())
    ids, dist = idx.query(data[0], k)           # no virtual index yet
    assert (ids == -1).all() and (dist == -1.0).all()
    idx.build_virtual_index()
    assert idx.num_virtual_points() == nb * 16 * int(np.sqrt(per))
    q = data[rng.choice(len(data), 60, replace=False)] + rng.normal(0, 0.5, (60, dim)).astype(np.float32)
    gt, gd = oracle.bruteforce_topk(data, q, k)
    hit = 0
    for i in range(60):
        ids, dist = idx.query(q[i], k, probe_buckets=2)
        assert (np.diff(dist[ids >= 0]) >= 0).all()
        v = ids[ids >= 0]
        assert np.allclose(dist[ids >= 0], ((data[v] - q[i]) ** 2).sum(axis=1), rtol=1e-4)  # global ids are arrival order
        hit += len(set(v.tolist()) & set(gt[i].tolist()))
    assert hit / (60 * k) > 0.9
    idx.close()


def _expected_query(oracle, levels, q, topk, probe, order="votes, then first vote", entry_points=True):
    """TimeStampIndex::query (src/timeStampIndex.cu:240-419) put together outside the library: the CPU search of
    the virtual layer, votes per bucket, most votes first (earlier first vote on ties), the CPU search of each
    probed bucket from the voters' entry points, merge by (distance, global id).  `levels` holds what the index
    exposes read-only: rows and graph of the virtual layer and of every bucket, the virtual points' buckets and
    entry points, the global id of every bucket row.  The rand_xor_mask of a search is the low half of the next
    splitmix64 output of its handle, read from the handle before the library's own query advances it.
    `order` and `entry_points` switch single steps of the rule off, to show that the comparison notices."""
    def search(view, data, graph, k, seeds):
        itopk, width, _, max_iter, bitlen = view.query_params()
        mask = oracle.splitmix64(view.rng_state())[0] & 0xFFFFFFFF
        # clamps of cagra::search: src/index/cagra.cu:862-864 (itopk), :887 (itopk / 4 seeds, from the parameter)
        ids, dist, _ = oracle.search(data, graph, q[None, :], k, max(k, itopk, 64), width, max_iter, bitlen, itopk // 4, mask,
                                     seeds=None if seeds is None else np.asarray(seeds, np.uint32)[None, :])
        return ids[0], dist[0]
    vview, vdata, vgraph, meta = levels["virtual"]
    vk = min(probe * 10, len(meta))
    vids, _ = search(vview, vdata, vgraph, vk, None)
    votes = {}
    for rank, v in enumerate(vids):
        if v < 0 or v >= len(meta):
            continue
        ts, eps = meta[v]
        c = votes.setdefault(ts, {"count": 0, "first": rank, "seeds": []})
        c["count"] += 1
        c["seeds"].extend(eps.tolist())
    key = {"votes, then first vote": lambda kv: (-kv[1]["count"], kv[1]["first"]),
           "first vote only": lambda kv: kv[1]["first"],
           "votes, then timestamp": lambda kv: (-kv[1]["count"], kv[0])}[order]
    ranked = sorted(votes.items(), key=key)[:probe]
    found = []
    for ts, c in ranked:
        view, data, graph, to_global = levels["buckets"][ts]
        k = min(topk, len(data))
        ids, dist = search(view, data, graph, k, (c["seeds"] or None) if entry_points else None)
        found += [(dist[r], int(to_global[ids[r]])) for r in range(k) if 0 <= ids[r] < len(to_global)]
    found.sort()
    eids = np.full(topk, -1, np.int64)
    edist = np.full(topk, -1.0, np.float32)
    for r, (d, g) in enumerate(found[:topk]):
        eids[r], edist[r] = g, d
    return eids, edist, [ts for ts, _ in ranked]


def test_timestamp_index_query_equals_the_routing_rule_on_cpu_searches(oracle, grab):
    # Six timestamps whose rows all come from the same 40 far-apart clusters, so the virtual points nearest to a query
    # belong to every bucket (votes tie, and which buckets are probed decides the answer) and a bucket's graph falls
    # into components (a bucket search from other seeds than the voters' entry points misses the query's cluster);
    # a seventh bucket holds fewer rows than topk.
    dim, per, nb, k = 32, 2500, 6, 10
    rng = np.random.default_rng(5)
    parts, ts = [], []
    for b in range(nb):
        parts.append(datasets.mixture(per, dim, 40, 300, 400 + b, sigma=8.0))
        ts.append(np.full(per, 50 + 7 * b, np.uint64))
    parts.append(datasets.mixture(6, dim, 1, 390, 490, sigma=8.0))
    ts.append(np.full(6, 999, np.uint64))
    data, ts = np.concatenate(parts), np.concatenate(ts)
    order = rng.permutation(len(data))
    data, ts = data[order], ts[order]
    idx = grab.TimeStampIndex(dim, 32)
    idx.set_seed(77)
    idx.insert(data[:8000], ts[:8000])
    idx.insert(data[8000:], ts[8000:])
    idx.build_virtual_index()
    assert idx.num_buckets() == nb + 1
    # what the index exposes, read once: nothing below changes rows or graphs
    vview = idx.virtual_index()
    meta = [idx.virtual_point(i) for i in range(idx.num_virtual_points())]
    where = np.array([idx.locate(g) for g in range(len(data))], dtype=np.uint64)
    buckets = {}
    for t in idx.bucket_timestamps().tolist():
        view = idx.bucket_index(t)
        to_global = np.flatnonzero(where[:, 0] == t)
        assert np.array_equal(where[to_global, 1], np.arange(len(to_global)))   # local ids follow arrival order
        bdata = view.get_data()
        assert np.array_equal(bdata, data[to_global])
        buckets[t] = (view, bdata, view.get_graph(), to_global)
    assert sorted(buckets) == sorted(set(ts.tolist())) and len(buckets[999][1]) == 6
    assert all(t in buckets and (eps < len(buckets[t][1])).all() for t, eps in meta)
    levels = {"virtual": (vview, vview.get_data(), vview.get_graph(), meta), "buckets": buckets}
    nq = 40
    pick = rng.choice(len(data), nq, replace=False)
    q = data[pick] + rng.normal(0, 0.5, (nq, dim)).astype(np.float32)
    q[:6] = data[ts == 999] + np.float32(0.25)          # queries that the small bucket must answer
    probed_small, short, noticed = 0, 0, {"first vote only": 0, "votes, then timestamp": 0, "no entry points": 0}
    for probe in (1, 2, 3, nb + 3):
        for i in range(nq if probe <= 2 else 12):
            eids, edist, routed = _expected_query(oracle, levels, q[i], k, probe)
            others = {"first vote only": _expected_query(oracle, levels, q[i], k, probe, order="first vote only")[0],
                      "votes, then timestamp": _expected_query(oracle, levels, q[i], k, probe, order="votes, then timestamp")[0],
                      "no entry points": _expected_query(oracle, levels, q[i], k, probe, entry_points=False)[0]}
            ids, dist = idx.query(q[i], k, probe_buckets=probe)
            assert np.array_equal(ids, eids), f"probe {probe}, query {i}: ids differ (buckets {routed})"
            assert np.array_equal(dist.view(np.uint32), edist.view(np.uint32)), f"probe {probe}, query {i}: distances differ"
            assert len(routed) <= probe
            probed_small += 999 in routed
            short += int((ids == -1).any())
            for name, other in others.items():
                noticed[name] += not np.array_equal(other, eids)
    assert probed_small >= 6 and short >= 1    # the small bucket was probed, and alone it leaves slots unfilled
    # each step of the rule decides answers here: with it changed the expectation is another one for some queries
    assert all(v >= 3 for v in noticed.values()), noticed
    idx.close()


def test_kmeans_random_configurations(oracle, grab):
    # sizes on both sides of the threshold above which the nearest-centroid contraction has enough rows for whole
    # tiles, k from 1 to 768, duplicated rows (ties between centroids)
    rng = np.random.default_rng(1)
    for case in range(10):
        n = int(rng.integers(50, 70000))
        dim = int(rng.choice([4, 32, 64, 128]))
        k = min(int(rng.choice([1, 3, 40, 300, 768])), n)
        niter, seed, kind = int(rng.integers(0, 8)), int(rng.integers(1 << 30)), rng.choice(["mix", "gauss", "dup"])
        if kind == "mix":
            data = datasets.mixture(n, dim, 25, 3, seed, sigma=6.0)
        elif kind == "gauss":
            data = datasets.gaussian(n, dim, seed)
        else:
            data = datasets.mixture(n, dim, 5, 3, seed)
            data[n // 2:] = data[:n - n // 2]
        cent, assign = grab.kmeans(data, k, niter, seed)
        ecent, eassign = oracle.kmeans(data, k, niter, seed)
        assert np.array_equal(cent.view(np.uint32), ecent.view(np.uint32)) and np.array_equal(assign, eassign), \
            f"case {case}: n {n} dim {dim} k {k} iterations {niter} {kind}"
