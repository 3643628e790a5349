"""Coarse level of the entry-point layer: the centroid ranking kernel against a float64 ranking, the listing walk
against a numpy restatement of its rule, and the search that lists its own seeds against listing + search."""
import numpy as np
import pytest

import datasets

pytestmark = pytest.mark.gpu

INVALID = 0xFFFFFFFF


def _rank_check(got, cent, q, nprobe, metric_ip, what):
    """Every row: distinct valid groups, ascending in value, and no group left out that is clearly nearer than the
    last one kept (fp32 sums in another order may swap near-ties, nothing more)."""
    G = cent.shape[0]
    c64, q64 = cent.astype(np.float64), q.astype(np.float64)
    val = -(q64 @ c64.T) if metric_ip else (c64 * c64).sum(1)[None, :] - 2.0 * (q64 @ c64.T)
    keep = min(nprobe, G)
    assert (got[:, keep:] == INVALID).all(), what
    g = got[:, :keep].astype(np.int64)
    assert (g >= 0).all() and (g < G).all(), what
    assert all(len(set(r.tolist())) == keep for r in g), what
    picked = np.take_along_axis(val, g, axis=1)
    scale = np.abs(val).max(axis=1, keepdims=True) + 1.0
    tol = 4e-6 * scale
    assert (np.diff(picked, axis=1) >= -tol).all(), what
    kth = np.sort(val, axis=1)[:, keep - 1:keep]
    assert (picked <= kth + tol).all(), what
    exact = np.argsort(val, axis=1, kind="stable")[:, :keep]
    return float((g == exact).all(axis=1).mean())


@pytest.mark.parametrize("G,nprobe,dim,nq,metric_ip", [
    (768, 16, 128, 5000, False),   # the benchmark's shape, 48 queries a workgroup
    (700, 16, 128, 300, False),    # 16 queries a workgroup, a last subtile that is not full
    (1000, 64, 64, 200, False),    # 1024-column instance, the longest list
    (300, 8, 256, 130, False),     # two chunks of 128 dimensions
    (40, 16, 100, 77, False),      # rows that end inside a chunk; fewer positions with a column than a list is long
    (5, 16, 32, 33, False),        # fewer groups than nprobe: padding
    (1, 1, 128, 3, False),
    (768, 1, 128, 500, False),     # the bound comes from the smallest of each set of sixteen minima
    (768, 3, 128, 500, False),
    (1000, 61, 128, 500, False),   # ... and from the largest
    (512, 32, 128, 4500, True),    # inner product
    (200, 12, 36, 4200, True),
])
def test_probe_ranks_the_centroids(grab, G, nprobe, dim, nq, metric_ip):
    n, S = 30000, max(G, 6000)
    data = datasets.gaussian(n, dim, 3) * 3.0 + 1.0
    q = datasets.gaussian(nq, dim, 4) * 3.0 + 1.0
    if metric_ip:
        data /= np.linalg.norm(data, axis=1, keepdims=True)
        q /= np.linalg.norm(q, axis=1, keepdims=True)
    d_data, d_q = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(q)
    layer = grab.EntryLayer(d_data, n, dim, S, d_ts=grab.DeviceArray.from_numpy(np.arange(n, dtype=np.uint64)))
    with pytest.raises(grab.GrabError):
        layer.probe(d_q, nq, nprobe)  # no groups yet
    layer.build_groups(G, niter=3, seed=5)
    cent = layer.centroids()
    assert cent.shape == (G, dim)
    got = layer.probe(d_q, nq, nprobe, metric=grab.METRIC_IP if metric_ip else grab.METRIC_L2).numpy()
    same = _rank_check(got, cent, q, nprobe, metric_ip, f"G {G} nprobe {nprobe} dim {dim} nq {nq}")
    assert same > 0.97
    with pytest.raises(grab.GrabError):
        layer.probe(d_q, nq, 65)
    layer.close()


def test_probe_when_every_value_ties(grab):
    # identical rows: all centroids coincide, every list overflows and the exact path takes the keys out one by one,
    # lowest group first
    n, dim, nq, G = 4000, 128, 70, 300
    data = np.full((n, dim), 2.0, np.float32)
    d_data = grab.DeviceArray.from_numpy(data)
    layer = grab.EntryLayer(d_data, n, dim, 2000, d_ts=grab.DeviceArray.from_numpy(np.arange(n, dtype=np.uint64)))
    layer.build_groups(G, niter=2, seed=1)
    cent = layer.centroids()
    q = np.full((nq, dim), 1.0, np.float32)
    got = layer.probe(grab.DeviceArray.from_numpy(q), nq, 16).numpy()
    val = (cent.astype(np.float64) ** 2).sum(1)[None, :] - 2.0 * (q.astype(np.float64) @ cent.T.astype(np.float64))
    if np.ptp(val) == 0.0:
        assert np.array_equal(got, np.tile(np.arange(16, dtype=np.uint32), (nq, 1)))
    else:  # k-means left empty groups at other places: still the smallest keys in (value, group) order
        _rank_check(got, cent, q, 16, False, "ties")
    layer.close()


def _list_model(ts, off, members, groups, ws, we, min_rows, max_ids):
    """The listing rule restated: window -> id interval; groups nearest first; a group is taken (whole) while fewer
    than min_rows rows were listed before it; ids in group order, cut at max_ids."""
    nq = groups.shape[0]
    out = np.full((nq, max_ids), INVALID, np.uint32)
    lo = np.searchsorted(ts, ws, side="left")
    hi = np.maximum(np.searchsorted(ts, we, side="left"), lo)
    for i in range(nq):
        row = []
        for g in groups[i]:
            if g == INVALID or len(row) >= min_rows:
                continue
            m = members[off[g]:off[g + 1]]
            row.extend(m[(m >= lo[i]) & (m < hi[i])].tolist())
        row = row[:max_ids]
        out[i, :len(row)] = row
    return out, lo, hi


@pytest.mark.parametrize("n,S,G,nprobe,min_rows,max_ids,rep,frac", [
    (50000, 8000, 100, 16, 32, 40, 1, 0.1),     # sixteen lanes a query
    (50000, 8000, 100, 16, 16, 32, 5, 0.3),     # repeated timestamps
    (33000, 33000, 60, 8, 0xFFFFFFFF, 64, 1, 0.02),  # every row a sample row; no early stop
    (20000, 3000, 40, 3, 8, 5, 1, 0.5),         # a short list that is cut
    (70, 40, 4, 4, 10, 16, 1, 0.5),             # a base without pivot levels above the first
    (50000, 8000, 100, 24, 32, 40, 1, 0.1),     # more than 16 groups: the wave-per-query walk
    (9000, 2000, 2000, 16, 32, 40, 1, 0.2),     # one member a group; more groups than the ranking kernel takes
])
def test_list_grouped_follows_its_rule(grab, n, S, G, nprobe, min_rows, max_ids, rep, frac):
    dim, nq = 64, 333
    data = datasets.mixture(n, dim, 20, 3, 4)
    q = datasets.mixture(nq, dim, 20, 3, 5)
    ts = np.arange(n, dtype=np.uint64) // rep * 3
    ws, we = datasets.windows(int(ts[-1]) + 3, nq, frac, 6)
    ws[0], we[0] = 7, 7                       # empty window
    ws[1], we[1] = 0, int(ts[-1]) + 100       # everything
    ws[2], we[2] = int(ts[-1]) + 1, int(ts[-1]) + 50   # behind the last row
    d_data, d_ts, d_q = (grab.DeviceArray.from_numpy(x) for x in (data, ts, q))
    d_ws, d_we = grab.DeviceArray.from_numpy(ws), grab.DeviceArray.from_numpy(we)
    layer = grab.EntryLayer(d_data, n, dim, S, d_ts=d_ts)
    layer.build_groups(G, niter=3, seed=2)
    off, members = layer.groups()
    assert off[0] == 0 and off[-1] == layer.size and (np.diff(off.astype(np.int64)) >= 0).all()
    assert np.array_equal(np.sort(members), (np.arange(layer.size, dtype=np.int64) * n // layer.size).astype(np.uint32))
    d_lo, d_hi = grab.DeviceArray((nq,), np.uint64), grab.DeviceArray((nq,), np.uint64)
    got = layer.list_grouped(d_q, nq, max_ids, nprobe, min_rows, d_win_start=d_ws, d_win_end=d_we, d_base_ts=d_ts, num_base=n,
                             d_id_lo=d_lo, d_id_hi=d_hi).numpy()
    if G <= 1024:
        groups = layer.probe(d_q, nq, nprobe).numpy()
        exp, lo, hi = _list_model(ts, off, members, groups, ws, we, min_rows, max_ids)
        assert np.array_equal(got, exp)
    else:
        lo = np.searchsorted(ts, ws, side="left")
        hi = np.maximum(np.searchsorted(ts, we, side="left"), lo)
        for i in range(nq):
            f = got[i][got[i] != INVALID]
            assert ((f >= lo[i]) & (f < hi[i])).all() and len(set(f.tolist())) == len(f)
    assert np.array_equal(d_lo.numpy(), lo) and np.array_equal(d_hi.numpy(), hi)
    assert (got[0] == INVALID).all() and (got[2] == INVALID).all()
    # without the base's timestamps the wave-per-query walk over the sample's own timestamps lists the same rows
    again = layer.list_grouped(d_q, nq, max_ids, nprobe, min_rows, d_win_start=d_ws, d_win_end=d_we).numpy()
    assert np.array_equal(again, got)
    # the scored selection keeps the nearest of exactly these rows (integer data: distances are exact)
    if max_ids == 64 or min_rows <= 32:
        full = layer.list_grouped(d_q, nq, 64, nprobe, min_rows, d_win_start=d_ws, d_win_end=d_we).numpy()
        ns = 8
        sel = layer.select_grouped(d_q, nq, ns, nprobe, min_rows, d_win_start=d_ws, d_win_end=d_we).numpy()
        for i in range(0, nq, 5):
            f = full[i][full[i] != INVALID]
            if len(f) == 64:
                continue  # the list was cut: the scored walk saw more rows
            d = ((data[f].astype(np.float64) - q[i]) ** 2).sum(1)
            order = np.lexsort((f, d))[:ns]  # ties go by the row's place in the sample, i.e. by its id here
            exp_sel = np.full(ns, INVALID, np.uint32)
            exp_sel[:len(order)] = f[order]
            assert np.array_equal(sel[i], exp_sel), i
    layer.close()


@pytest.mark.parametrize("itopk,degree,nprobe,min_rows,n_seeds", [
    (64, 64, 16, 16, 32),    # the benchmark's instance (rows of 64 slots, filter first)
    (64, 32, 12, 32, 40),    # the general register-queue kernel
    (128, 64, 16, 24, 64),   # two queue entries a lane
    (256, 32, 20, 64, 64),   # four
])
def test_search_that_lists_its_own_seeds(oracle, grab, itopk, degree, nprobe, min_rows, n_seeds):
    # grab_search_desc.entry_layer: same seeds, hence same results and counters, as grab_entry_layer_list_grouped
    # followed by the search with that list and the id intervals; and that pair equals the CPU restatement
    n, dim, nq, k, S, G = 40000, 128, 1500, 10, 6000, 90
    data = datasets.mixture(n, dim, 30, 10, 11)
    q = datasets.mixture(nq, dim, 30, 10, 12)
    ts = np.arange(n, dtype=np.uint64) // 2
    ws, we = datasets.windows(int(ts[-1]) + 1, nq, 0.1, 13)
    ws[5], we[5] = 9, 9
    d_data, d_ts, d_q = (grab.DeviceArray.from_numpy(x) for x in (data, ts, q))
    d_ws, d_we = grab.DeviceArray.from_numpy(ws), grab.DeviceArray.from_numpy(we)
    d_knn, _ = grab.generate_knn_graph(d_data, n, dim, 2 * degree)
    d_graph = grab.build_graph(d_data, n, d_knn, 2 * degree, degree)
    layer = grab.EntryLayer(d_data, n, dim, S, d_ts=d_ts)
    layer.build_groups(G, niter=4, seed=3)
    d_groups = layer.probe(d_q, nq, nprobe)
    flags = grab.FLAG_FILTER_FIRST | grab.FLAG_WAVE_PER_QUERY
    bitlen = 11
    ids, dist, ctr, _ = grab.search_ex(d_data, d_graph, n, dim, degree, d_q, nq, k, itopk, 4, 50, bitlen, n_seeds, 0x5EED,
                                       filter_kind=grab.FILTER_ID_RANGE, d_ts=d_ts, d_win_start=d_ws, d_win_end=d_we, flags=flags,
                                       want_counters=True, entry=(layer, d_groups, nprobe, min_rows))
    d_lo, d_hi = grab.DeviceArray((nq,), np.uint64), grab.DeviceArray((nq,), np.uint64)
    d_list = layer.list_grouped(d_q, nq, n_seeds, nprobe, min_rows, d_win_start=d_ws, d_win_end=d_we, d_base_ts=d_ts, num_base=n,
                                d_id_lo=d_lo, d_id_hi=d_hi)
    ids2, dist2, ctr2, _ = grab.search_ex(d_data, d_graph, n, dim, degree, d_q, nq, k, itopk, 4, 50, bitlen, n_seeds, 0x5EED,
                                          d_seeds=d_list, n_provided=n_seeds, filter_kind=grab.FILTER_ID_RANGE, d_win_start=d_lo,
                                          d_win_end=d_hi, flags=flags, want_counters=True)
    assert np.array_equal(ids, ids2) and np.array_equal(dist.view(np.uint32), dist2.view(np.uint32))
    assert np.array_equal(ctr, ctr2)
    assert ctr[:, 5].sum() == 0
    eids, edist, ectr = oracle.search(data, d_graph.numpy(), q, k, itopk, 4, 50, bitlen, n_seeds, 0x5EED, seeds=d_list.numpy(),
                                      filter_kind=oracle.FILTER_ID_RANGE, win_start=d_lo.numpy(), win_end=d_hi.numpy(),
                                      flags=oracle.FLAG_FILTER_FIRST)
    assert np.array_equal(ids, eids) and np.array_equal(dist.view(np.uint32), edist.view(np.uint32))
    assert np.array_equal(ctr[:, [0, 1, 2, 4]], ectr[:, [0, 1, 2, 4]])
    assert (ids[5] == -1).all()
    gt, _, _ = grab.bruteforce_topk(d_data, n, dim, d_q, nq, k, filter_kind=grab.FILTER_RANGE, d_ts=d_ts, d_win_start=d_ws, d_win_end=d_we)
    assert datasets.recall(ids, gt) > 0.9
    layer.close()


def test_search_entry_layer_argument_checks(grab):
    n, dim, nq, degree = 6000, 64, 1100, 32
    data = datasets.mixture(n, dim, 10, 3, 4)
    q = datasets.mixture(nq, dim, 10, 3, 5)
    ts = np.arange(n, dtype=np.uint64)
    ws, we = datasets.windows(n, nq, 0.2, 6)
    d_data, d_ts, d_q = (grab.DeviceArray.from_numpy(x) for x in (data, ts, q))
    d_ws, d_we = grab.DeviceArray.from_numpy(ws), grab.DeviceArray.from_numpy(we)
    d_knn, _ = grab.generate_knn_graph(d_data, n, dim, 64)
    d_graph = grab.build_graph(d_data, n, d_knn, 64, degree)
    layer = grab.EntryLayer(d_data, n, dim, 1500, d_ts=d_ts)
    d_groups = grab.DeviceArray((nq, 8), np.uint32)

    def run(lay=layer, filter_kind=grab.FILTER_ID_RANGE, flags=grab.FLAG_FILTER_FIRST, n_seeds=32, itopk=64, bitlen=10, ts_arg=d_ts,
            nprobe=8):
        return grab.search_ex(d_data, d_graph, n, dim, degree, d_q, nq, 10, itopk, 4, 50, bitlen, n_seeds, 1, filter_kind=filter_kind,
                              d_ts=ts_arg, d_win_start=d_ws, d_win_end=d_we, flags=flags, entry=(lay, d_groups, nprobe, 16))
    with pytest.raises(grab.GrabError):
        run()                                   # no groups
    layer.build_groups(20, niter=2, seed=1)
    layer.probe(d_q, nq, 8, d_out=d_groups)
    run()
    for bad in (dict(filter_kind=grab.FILTER_RANGE), dict(ts_arg=None), dict(n_seeds=0), dict(nprobe=65),
                dict(flags=grab.FLAG_FILTER_FIRST | grab.FLAG_BLOCK_PER_QUERY), dict(flags=grab.FLAG_STRICT_REFERENCE),
                dict(itopk=512, n_seeds=64)):
        with pytest.raises(grab.GrabError):
            run(**bad)
    # a layer over timestamps that do not ascend with the row id offers no id intervals
    shuffled = np.random.default_rng(1).permutation(n).astype(np.uint64)
    order = np.argsort(shuffled, kind="stable").astype(np.uint32)
    other = grab.EntryLayer(d_data, n, dim, 1500, d_ids_by_ts=grab.DeviceArray.from_numpy(order), d_ts=grab.DeviceArray.from_numpy(shuffled))
    other.build_groups(20, niter=2, seed=1)
    with pytest.raises(grab.GrabError):
        run(lay=other)
    unordered = grab.EntryLayer(d_data, n, dim, 1500, d_ts=grab.DeviceArray.from_numpy(shuffled))
    unordered.build_groups(20, niter=2, seed=1)
    with pytest.raises(grab.GrabError):
        run(lay=unordered)
    for lay in (layer, other, unordered):
        lay.close()
