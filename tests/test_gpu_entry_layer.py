"""Entry-point layer (sample of the base + MFMA seed selection) against exact brute force over the sample."""
import numpy as np
import pytest

import datasets

pytestmark = pytest.mark.gpu


def _expected(oracle, data, ts, sid, q, n_seeds, **flt):
    sub_ts = ts[sid] if ts is not None else None
    ids, _ = oracle.bruteforce_topk(data[sid], q, n_seeds, ts=sub_ts, **flt)
    return np.where(ids >= 0, sid[np.clip(ids, 0, len(sid) - 1)], 0xFFFFFFFF).astype(np.uint32)


@pytest.mark.parametrize("n,S,nq,n_seeds", [(20000, 4096, 700, 16), (9000, 1000, 130, 32), (5000, 5000, 64, 64)])
def test_select_range_per_query_matches_bruteforce(oracle, grab, n, S, nq, n_seeds):
    data = datasets.mixture(n, 128, 12, 10, 11)  # integer data: the GEMM-form distance is exact
    q = datasets.mixture(nq, 128, 12, 10, 12)
    ts = (np.arange(n, dtype=np.uint64) // 7)     # repeated timestamps
    ws, we = datasets.windows(int(ts[-1]) + 1, nq, 0.1, 3)
    ws[0], we[0] = 5, 5                            # an empty window
    ws[1], we[1] = 0, 1                            # fewer rows than n_seeds
    d_data = grab.DeviceArray.from_numpy(data)
    layer = grab.EntryLayer(d_data, n, 128, S, d_ts=grab.DeviceArray.from_numpy(ts))
    assert layer.size == S
    sid = (np.arange(S, dtype=np.int64) * n // S).astype(np.uint32)
    got = layer.select(grab.DeviceArray.from_numpy(q), nq, n_seeds, filter_kind=grab.FILTER_RANGE,
                       d_win_start=grab.DeviceArray.from_numpy(ws), d_win_end=grab.DeviceArray.from_numpy(we)).numpy()
    exp = _expected(oracle, data, ts, sid, q, n_seeds, filter_kind=oracle.FILTER_RANGE, win_start=ws, win_end=we)
    assert np.array_equal(got, exp)
    assert (got[0] == 0xFFFFFFFF).all()
    layer.close()


def test_select_single_window_unfiltered_and_mask(oracle, grab):
    n, S, nq = 12000, 3000, 200
    data = datasets.mixture(n, 128, 12, 10, 11)
    q = datasets.mixture(nq, 128, 12, 10, 12)
    ts = np.arange(n, dtype=np.uint64)
    labels = datasets.zipf_labels(n, 64, 1.1, 21)
    masks = datasets.label_masks(nq, 64, 23)
    d_data, d_q = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(q)
    layer = grab.EntryLayer(d_data, n, 128, S, d_ts=grab.DeviceArray.from_numpy(ts), d_labels=grab.DeviceArray.from_numpy(labels))
    sid = (np.arange(S, dtype=np.int64) * n // S).astype(np.uint32)
    got = layer.select(d_q, nq, 16, filter_kind=grab.FILTER_RANGE, win=(2000, 9000)).numpy()
    assert np.array_equal(got, _expected(oracle, data, ts, sid, q, 16, filter_kind=oracle.FILTER_RANGE, win=(2000, 9000)))
    got = layer.select(d_q, nq, 16).numpy()
    assert np.array_equal(got, _expected(oracle, data, None, sid, q, 16))
    got = layer.select(d_q, nq, 16, filter_kind=grab.FILTER_MASK, d_masks=grab.DeviceArray.from_numpy(masks)).numpy()
    ids, _ = oracle.bruteforce_topk(data[sid], q, 16, filter_kind=oracle.FILTER_MASK, labels=labels[sid], masks=masks)
    exp = np.where(ids >= 0, sid[np.clip(ids, 0, S - 1)], 0xFFFFFFFF).astype(np.uint32)
    assert np.array_equal(got, exp)
    layer.close()


def test_select_unsorted_timestamps_and_float_data(oracle, grab):
    # timestamps not monotone in the row id: the layer samples in timestamp order through ids_by_ts
    n, S, nq = 8000, 2000, 100
    rng = np.random.default_rng(4)
    data = datasets.gaussian(n, 96, 5)
    q = datasets.gaussian(nq, 96, 6)
    ts = rng.integers(0, 1000, n).astype(np.uint64)
    order = np.argsort(ts, kind="stable").astype(np.uint32)
    ws, we = datasets.windows(1000, nq, 0.2, 7)
    layer = grab.EntryLayer(grab.DeviceArray.from_numpy(data), n, 96, S, d_ids_by_ts=grab.DeviceArray.from_numpy(order),
                            d_ts=grab.DeviceArray.from_numpy(ts))
    got = layer.select(grab.DeviceArray.from_numpy(q), nq, 16, filter_kind=grab.FILTER_RANGE,
                       d_win_start=grab.DeviceArray.from_numpy(ws), d_win_end=grab.DeviceArray.from_numpy(we)).numpy()
    sid = order[(np.arange(S, dtype=np.int64) * n // S)]
    exp = _expected(oracle, data, ts, sid, q, 16, filter_kind=oracle.FILTER_RANGE, win_start=ws, win_end=we)
    for i in range(nq):
        v = got[i][got[i] != 0xFFFFFFFF]
        assert ((ts[v] >= ws[i]) & (ts[v] < we[i])).all()
        # float data: the GEMM-form distance may order near-ties differently; the sets agree almost everywhere
        assert len(set(v.tolist()) & set(exp[i].tolist())) >= len(v) - 1
    layer.close()


def test_seeds_from_the_layer_lift_recall_on_disconnected_clusters(oracle, grab):
    # 200 well separated clusters: the kNN graph falls apart into components, random in-window seeds miss most of them
    n, nq, deg = 40000, 300, 32
    data = datasets.mixture(n, 128, 200, 10, 11)
    q = datasets.mixture(nq, 128, 200, 10, 12)
    ts = np.arange(n, dtype=np.uint64)
    ws, we = datasets.windows(n, nq, 0.25, 13)
    d_data, d_q = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(q)
    d_ts = grab.DeviceArray.from_numpy(ts)
    d_ws, d_we = grab.DeviceArray.from_numpy(ws), grab.DeviceArray.from_numpy(we)
    d_knn, _ = grab.generate_knn_graph(d_data, n, 128, 64)
    d_graph = grab.build_graph(d_data, n, d_knn, 64, deg)
    gt, _, _ = grab.bruteforce_topk(d_data, n, 128, d_q, nq, 10, filter_kind=grab.FILTER_RANGE, d_ts=d_ts, d_win_start=d_ws, d_win_end=d_we)
    rnd = grab.sample_window_seeds(d_ts, grab.DeviceArray.from_numpy(np.arange(n, dtype=np.uint32)), n, nq, 32, 1, d_win_start=d_ws, d_win_end=d_we)
    layer = grab.EntryLayer(d_data, n, 128, 8192, d_ts=d_ts)
    ent = layer.select(d_q, nq, 32, filter_kind=grab.FILTER_RANGE, d_win_start=d_ws, d_win_end=d_we)
    rec = {}
    for name, seeds in (("random", rnd), ("entry", ent)):
        ids, _, _, _ = grab.search_ex(d_data, d_graph, n, 128, deg, d_q, nq, 10, 64, 4, 50, 13, 32, 3, d_seeds=seeds, n_provided=32,
                                      filter_kind=grab.FILTER_RANGE, d_ts=d_ts, d_win_start=d_ws, d_win_end=d_we)
        rec[name] = datasets.recall(ids, gt)
    assert rec["random"] < 0.5 and rec["entry"] > 0.95, rec


@pytest.mark.parametrize("near_lanes", [3, 15])
def test_select_when_few_lanes_hold_all_the_near_columns(oracle, grab, near_lanes):
    # near rows confined to a few lanes of the selection pass (lane of column c = (c % 256) / 4): every insertion
    # comes from the same lanes, many per step
    n, nq, n_seeds = 8192, 70, 16
    rng = np.random.default_rng(7)
    col = np.arange(n)
    near = ((col % 256) // 4) < near_lanes
    data = np.where(near[:, None], rng.integers(0, 12, (n, 128)), rng.integers(100, 140, (n, 128))).astype(np.float32)
    q = rng.integers(0, 12, (nq, 128)).astype(np.float32)
    ts = np.arange(n, dtype=np.uint64)
    layer = grab.EntryLayer(grab.DeviceArray.from_numpy(data), n, 128, n, d_ts=grab.DeviceArray.from_numpy(ts))
    sid = np.arange(n, dtype=np.uint32)
    ws = rng.integers(0, 500, nq).astype(np.uint64)
    we = ws + rng.integers(6000, 7600, nq).astype(np.uint64)
    got = layer.select(grab.DeviceArray.from_numpy(q), nq, n_seeds, filter_kind=grab.FILTER_RANGE,
                       d_win_start=grab.DeviceArray.from_numpy(ws), d_win_end=grab.DeviceArray.from_numpy(we)).numpy()
    exp = _expected(oracle, data, ts, sid, q, n_seeds, filter_kind=oracle.FILTER_RANGE, win_start=ws, win_end=we)
    assert np.array_equal(got, exp)
    layer.close()


def test_grouped_select_with_every_group_probed_equals_exact_select(oracle, grab):
    # 40 groups, all of them probed and no early stop: the walk over the groups must find exactly the nearest
    # in-window sample rows, whatever the grouping
    n, dim, S, nq, ns = 20000, 64, 4096, 300, 16
    data = datasets.gaussian(n, dim, 3)
    q = datasets.gaussian(nq, dim, 4)
    ts = np.arange(n, dtype=np.uint64) * 3
    rng = np.random.default_rng(8)
    ws = rng.integers(0, 3 * n - 9000, nq).astype(np.uint64)
    we = ws + rng.integers(0, 9000, nq).astype(np.uint64)   # some windows hold no sample row at all
    d_data, d_ts, d_q = (grab.DeviceArray.from_numpy(x) for x in (data, ts, q))
    d_ws, d_we = grab.DeviceArray.from_numpy(ws), grab.DeviceArray.from_numpy(we)
    layer = grab.EntryLayer(d_data, n, dim, S, d_ts=d_ts)
    exact = layer.select(d_q, nq, ns, filter_kind=grab.FILTER_RANGE, d_win_start=d_ws, d_win_end=d_we).numpy()
    assert layer.num_groups == 0
    with pytest.raises(grab.GrabError):
        layer.select_grouped(d_q, nq, ns, 8, 32, d_win_start=d_ws, d_win_end=d_we)   # no groups yet
    layer.build_groups(40, niter=5, seed=2)
    assert layer.num_groups == 40
    d_lo, d_hi = grab.DeviceArray((nq,), np.uint64), grab.DeviceArray((nq,), np.uint64)
    got = layer.select_grouped(d_q, nq, ns, 40, 0xFFFFFFFF, d_win_start=d_ws, d_win_end=d_we, d_base_ts=d_ts, num_base=n,
                               d_id_lo=d_lo, d_id_hi=d_hi).numpy()
    assert np.array_equal(got, exact)
    # the id intervals written on the side are those of grab_windows_to_id_ranges
    assert np.array_equal(d_lo.numpy(), np.searchsorted(ts, ws, side="left"))
    assert np.array_equal(d_hi.numpy(), np.maximum(np.searchsorted(ts, we, side="left"), np.searchsorted(ts, ws, side="left")))
    v = got[got != 0xFFFFFFFF]
    assert v.size > 0 and (got == 0xFFFFFFFF).any()
    # a bounded walk returns rows of the window, nearest first, and never more rows than the window holds
    few = layer.select_grouped(d_q, nq, ns, 4, 24, d_win_start=d_ws, d_win_end=d_we).numpy()
    for i in range(nq):
        f = few[i][few[i] != 0xFFFFFFFF]
        assert ((ts[f] >= ws[i]) & (ts[f] < we[i])).all()
        d = ((data[f] - q[i]) ** 2).sum(1)
        assert (np.diff(d) >= -1e-3).all()
        assert len(f) <= (exact[i] != 0xFFFFFFFF).sum()
    layer.close()


@pytest.mark.parametrize("case", ["nprobe64", "two_passes", "inner_product", "many_groups"])
def test_grouped_select_other_paths(oracle, grab, case):
    # the paths that do not pick the centroids inside the walk kernel (more than 48 centroids kept, more than 16384
    # queries, more than 1024 groups), and the inner product
    dim, ns = 128, 16
    metric = grab.METRIC_IP if case == "inner_product" else grab.METRIC_L2
    n, S, nq, groups, nprobe = 30000, 6000, 400, 40, 40
    if case == "nprobe64":
        groups, nprobe = 60, 64
    if case == "two_passes":
        nq = 17000
    if case == "many_groups":
        S, groups, nprobe = 6000, 1100, 32
    data = datasets.mixture(n, dim, 60, 3, 4)
    q = datasets.mixture(nq, dim, 60, 3, 5)
    if metric == grab.METRIC_IP:
        data /= np.linalg.norm(data, axis=1, keepdims=True)
        q /= np.linalg.norm(q, axis=1, keepdims=True)
    ts = np.arange(n, dtype=np.uint64)
    ws, we = datasets.windows(n, nq, 0.2, 6)
    d_data, d_ts, d_q = (grab.DeviceArray.from_numpy(x) for x in (data, ts, q))
    d_ws, d_we = grab.DeviceArray.from_numpy(ws), grab.DeviceArray.from_numpy(we)
    layer = grab.EntryLayer(d_data, n, dim, S, d_ts=d_ts)
    exact = layer.select(d_q, nq, ns, metric=metric, filter_kind=grab.FILTER_RANGE, d_win_start=d_ws, d_win_end=d_we).numpy()
    layer.build_groups(groups, niter=6, seed=2)
    if case == "many_groups":
        # not every group can be probed: the nearest sample row of the window is still found nearly always on
        # clustered data, and everything returned lies inside the window, nearest first
        got = layer.select_grouped(d_q, nq, ns, nprobe, 64, metric=metric, d_win_start=d_ws, d_win_end=d_we).numpy()
        assert (got[:, 0] == exact[:, 0]).mean() > 0.95
        for i in range(0, nq, 7):
            f = got[i][got[i] != 0xFFFFFFFF]
            assert ((ts[f] >= ws[i]) & (ts[f] < we[i])).all()
            assert (np.diff(((data[f] - q[i]) ** 2).sum(1)) >= 0).all()
    else:
        got = layer.select_grouped(d_q, nq, ns, nprobe, 0xFFFFFFFF, metric=metric, d_win_start=d_ws, d_win_end=d_we).numpy()
        if metric == grab.METRIC_IP:  # float data: near-ties may be ordered differently by the two distance forms
            same = np.mean([len(set(a.tolist()) & set(b.tolist())) / ns for a, b in zip(got, exact)])
            assert same > 0.99
        else:
            assert np.array_equal(got, exact)
    layer.close()


def test_grouped_select_degenerate_inputs(grab):
    # every row identical: all centroid distances tie (the listing overflows and falls back to insertion), all row
    # distances tie; and a sample smaller than a wave.  Seeds must still be distinct rows of the window.
    n, dim, nq, ns = 3000, 128, 130, 16
    data = np.ones((n, dim), np.float32)
    q = np.ones((nq, dim), np.float32)
    ts = np.arange(n, dtype=np.uint64)
    rng = np.random.default_rng(3)
    ws = rng.integers(0, n - 600, nq).astype(np.uint64)
    we = ws + np.uint64(500)
    d_data, d_ts, d_q = (grab.DeviceArray.from_numpy(x) for x in (data, ts, q))
    d_ws, d_we = grab.DeviceArray.from_numpy(ws), grab.DeviceArray.from_numpy(we)
    for S, groups, nprobe in ((1500, 300, 16), (40, 5, 8), (1, 1, 1)):
        layer = grab.EntryLayer(d_data, n, dim, S, d_ts=d_ts)
        layer.build_groups(groups, niter=3, seed=1)
        got = layer.select_grouped(d_q, nq, ns, nprobe, 32, d_win_start=d_ws, d_win_end=d_we).numpy()
        for i in range(nq):
            f = got[i][got[i] != 0xFFFFFFFF]
            assert len(set(f.tolist())) == len(f)
            assert ((ts[f] >= ws[i]) & (ts[f] < we[i])).all()
        if S == 1500:
            assert (got != 0xFFFFFFFF).any()
        layer.close()


def test_select_random_configurations(oracle, grab):
    # random sizes, dimensions, sample sizes, seed counts, repeated timestamps and window widths: the exact selection
    # against brute force over the sample, the grouped selection with every group probed against the exact one, and
    # the id intervals written on the side (integer data: both distance forms agree bit for bit)
    rng = np.random.default_rng(5)
    for case in range(12):
        n = int(rng.integers(3000, 40000))
        dim = int(rng.choice([32, 64, 128, 128, 256]))
        S = min(int(rng.choice([64, 500, 1000, 4096, 7000])), n)
        nq, ns = int(rng.choice([1, 60, 700, 1500])), int(rng.choice([1, 8, 16, 32, 64]))
        groups = min(int(rng.choice([1, 7, 40, 200])), S)
        rep, frac = int(rng.choice([1, 1, 7])), float(rng.choice([0.02, 0.1, 0.5, 1.0]))
        data = datasets.mixture(n, dim, 12, 10, int(rng.integers(1 << 30)))
        q = datasets.mixture(nq, dim, 12, 10, int(rng.integers(1 << 30)))
        ts = np.arange(n, dtype=np.uint64) // rep
        ws, we = datasets.windows(int(ts[-1]) + 1, nq, frac, int(rng.integers(1 << 30)))
        what = f"case {case}: n {n} dim {dim} S {S} nq {nq} seeds {ns} groups {groups} rep {rep} window {frac}"
        d_data, d_ts, d_q = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(ts), grab.DeviceArray.from_numpy(q)
        d_ws, d_we = grab.DeviceArray.from_numpy(ws), grab.DeviceArray.from_numpy(we)
        layer = grab.EntryLayer(d_data, n, dim, S, d_ts=d_ts)
        sid = (np.arange(S, dtype=np.int64) * n // S).astype(np.uint32)
        got = layer.select(d_q, nq, ns, filter_kind=grab.FILTER_RANGE, d_win_start=d_ws, d_win_end=d_we).numpy()
        exp = _expected(oracle, data, ts, sid, q, ns, filter_kind=oracle.FILTER_RANGE, win_start=ws, win_end=we)
        assert np.array_equal(got, exp), what
        layer.build_groups(groups, niter=4, seed=3)
        d_lo, d_hi = grab.DeviceArray((nq,), np.uint64), grab.DeviceArray((nq,), np.uint64)
        g = layer.select_grouped(d_q, nq, ns, min(groups, 64), 0xFFFFFFFF, d_win_start=d_ws, d_win_end=d_we, d_base_ts=d_ts,
                                 num_base=n, d_id_lo=d_lo, d_id_hi=d_hi).numpy()
        if groups <= 64:
            assert np.array_equal(g, exp), what
        lo = np.searchsorted(ts, ws, side="left")
        assert np.array_equal(d_lo.numpy(), lo) and np.array_equal(d_hi.numpy(), np.maximum(np.searchsorted(ts, we, side="left"), lo)), what
        layer.close()
