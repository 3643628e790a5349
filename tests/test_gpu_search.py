"""Beam search on the GPU against the CPU restatement, on the same seeded inputs.

Graphs come from the oracle so that this file tests the search path alone.  The bar is
bit-exact: ids, distance bits and the per-query work counters.
"""
import numpy as np
import pytest

import datasets

pytestmark = pytest.mark.gpu


class Case:
    def __init__(self, oracle, grab, data, degree, knn_k):
        self.data = data
        self.n, self.dim = data.shape
        self.graph = oracle.optimize(oracle.knn_graph(data, knn_k), degree)
        self.degree = degree
        self.d_data = grab.DeviceArray.from_numpy(data)
        self.d_graph = grab.DeviceArray.from_numpy(self.graph)


@pytest.fixture(scope="module")
def gauss(oracle, grab):
    return Case(oracle, grab, datasets.gaussian(3000, 128, 1), 32, 64)


@pytest.fixture(scope="module")
def mix(oracle, grab):
    # integer-valued rows: many exactly equal distances, so the (dist,id) rule is exercised
    return Case(oracle, grab, datasets.mixture(4000, 128, 10, 10, 11), 32, 64)


def run_both(oracle, grab, case, queries, k, itopk, sw, max_iter, bitlen, n_seeds, mask, **kw):
    seeds = kw.pop("seeds", None)
    ts = kw.get("ts")
    labels = kw.get("labels")
    masks = kw.get("masks")
    ws, we = kw.get("win_start"), kw.get("win_end")
    exp = oracle.search(case.data, case.graph, queries, k, itopk, sw, max_iter, bitlen, n_seeds, mask, seeds=seeds, **kw)
    dev = {}
    if ts is not None:
        dev["d_ts"] = grab.DeviceArray.from_numpy(np.asarray(ts, np.uint64))
    if labels is not None:
        dev["d_labels"] = grab.DeviceArray.from_numpy(np.asarray(labels, np.uint8))
        dev["d_masks"] = grab.DeviceArray.from_numpy(np.asarray(masks, np.uint64))
    if ws is not None:
        dev["d_win_start"] = grab.DeviceArray.from_numpy(np.asarray(ws, np.uint64))
        dev["d_win_end"] = grab.DeviceArray.from_numpy(np.asarray(we, np.uint64))
    d_seeds = grab.DeviceArray.from_numpy(np.asarray(seeds, np.uint32)) if seeds is not None else None
    d_q = grab.DeviceArray.from_numpy(queries)
    def gpu(decomposition, **more):
        return grab.search_ex(case.d_data, case.d_graph, case.n, case.dim, case.degree, d_q, queries.shape[0], k, itopk,
                              sw, max_iter, bitlen, n_seeds, mask, active_degree=kw.get("active_degree"),
                              metric=kw.get("metric", 0), d_seeds=d_seeds,
                              n_provided=0 if seeds is None else np.asarray(seeds).shape[1],
                              filter_kind=kw.get("filter_kind", 0), win=kw.get("win"),
                              flags=kw.get("flags", 0) | decomposition, want_counters=True, **dev, **more)

    # both decompositions of the search (workgroup per query, wave per query) must agree bit for bit
    got = gpu(grab.FLAG_BLOCK_PER_QUERY)
    if bitlen <= 15:
        wave = gpu(grab.FLAG_WAVE_PER_QUERY)
        for x, y, what in zip(got[:3], wave[:3], ("ids", "distances", "counters")):
            assert np.array_equal(x.view(np.uint32) if x.dtype == np.float32 else x,
                                  y.view(np.uint32) if y.dtype == np.float32 else y), f"wave-per-query {what} differ"
        if kw.get("filter_kind", 0) == 1:
            # the neighbours' timestamps read from rows laid out like the graph: nothing may change
            d_gts = grab.neighbor_timestamps(case.d_graph, dev["d_ts"], case.n, case.degree)
            exp_gts = np.where(case.graph < case.n, np.asarray(ts, np.uint64)[np.minimum(case.graph, case.n - 1)], np.uint64(2**64 - 1))
            assert np.array_equal(d_gts.numpy(), exp_gts)
            rows = gpu(grab.FLAG_WAVE_PER_QUERY, d_graph_ts=d_gts)
            for x, y, what in zip(wave[:3], rows[:3], ("ids", "distances", "counters")):
                assert np.array_equal(x.view(np.uint32) if x.dtype == np.float32 else x,
                                      y.view(np.uint32) if y.dtype == np.float32 else y), f"neighbour-timestamp rows: {what} differ"
            # the same filter as an interval of places in timestamp order (filter kind 3 with d_rank): the window
            # becomes [lower_bound(start), lower_bound(end)) over the sorted timestamps, a row passes when its place
            # lies inside.  Same answers, same counters (a 4-byte place is read wherever a timestamp was).
            tsa = np.asarray(ts, np.uint64)
            order = np.argsort(tsa, kind="stable")
            rank = np.empty(case.n, np.uint32)
            rank[order] = np.arange(case.n, dtype=np.uint32)
            sorted_ts = tsa[order]
            d_rank = grab.DeviceArray.from_numpy(rank)
            d_grank = grab.neighbor_ranks(case.d_graph, d_rank, case.n, case.degree)
            assert np.array_equal(d_grank.numpy(), np.where(case.graph < case.n, rank[np.minimum(case.graph, case.n - 1)], 0xFFFFFFFF))
            nq = queries.shape[0]
            if ws is not None:
                lo = np.searchsorted(sorted_ts, np.asarray(ws, np.uint64), side="left").astype(np.uint64)
                hi = np.maximum(np.searchsorted(sorted_ts, np.asarray(we, np.uint64), side="left").astype(np.uint64), lo)
                win_args = dict(d_win_start=grab.DeviceArray.from_numpy(lo), d_win_end=grab.DeviceArray.from_numpy(hi))
            else:
                w0, w1 = kw["win"]
                lo = int(np.searchsorted(sorted_ts, np.uint64(w0), side="left"))
                win_args = dict(win=(lo, max(int(np.searchsorted(sorted_ts, np.uint64(w1), side="left")), lo)))
            def by_place(decomposition, **more):
                return grab.search_ex(case.d_data, case.d_graph, case.n, case.dim, case.degree, d_q, nq, k, itopk, sw, max_iter,
                                      bitlen, n_seeds, mask, active_degree=kw.get("active_degree"), metric=kw.get("metric", 0),
                                      d_seeds=d_seeds, n_provided=0 if seeds is None else np.asarray(seeds).shape[1],
                                      filter_kind=grab.FILTER_ID_RANGE, flags=kw.get("flags", 0) | decomposition, want_counters=True,
                                      d_rank=d_rank, **win_args, **more)
            for what, res in (("block", by_place(grab.FLAG_BLOCK_PER_QUERY)), ("wave", by_place(grab.FLAG_WAVE_PER_QUERY)),
                              ("wave, rows of places", by_place(grab.FLAG_WAVE_PER_QUERY, d_graph_rank=d_grank))):
                for x, y, part in zip(wave[:3], res[:3], ("ids", "distances", "counters")):
                    assert np.array_equal(x.view(np.uint32) if x.dtype == np.float32 else x,
                                          y.view(np.uint32) if y.dtype == np.float32 else y), f"filter by place ({what}): {part} differ"
    return exp, got


def assert_same(exp, got):
    eid, edist, ectr = exp
    gid, gdist, gctr, _ = got
    bad = np.nonzero((eid != gid).any(axis=1))[0]
    assert bad.size == 0, f"ids differ for queries {bad[:5]}: {eid[bad[0]]} vs {gid[bad[0]]}"
    assert np.array_equal(edist.view(np.uint32), gdist.view(np.uint32))
    assert np.array_equal(ectr[:, :5], gctr[:, :5]), "work counters differ"
    assert int(gctr[:, 5].sum()) == 0 and int(ectr[:, 5].sum()) == 0, "visited set overflowed"


@pytest.mark.parametrize("itopk,sw,max_iter,bitlen", [(64, 4, 50, 13), (64, 1, 20, 11), (128, 6, 40, 13), (256, 6, 50, 14), (96, 3, 35, 12)])
def test_unfiltered_matches_oracle(oracle, grab, gauss, itopk, sw, max_iter, bitlen):
    q = datasets.gaussian(200, 128, 2)
    it, ns, _ = grab.search_plan(grab.WRAP_SEARCH, 10, itopk, sw, gauss.degree)
    assert (it, ns) == oracle.search_plan(oracle.WRAP_SEARCH, 10, itopk, sw, gauss.degree)[:2]
    exp, got = run_both(oracle, grab, gauss, q, 10, it, sw, max_iter, bitlen, ns, 0x9E3779B9)
    assert_same(exp, got)
    assert (np.diff(got[1], axis=1) >= 0).all()


def test_integer_data_ties_match_oracle(oracle, grab, mix):
    q = datasets.mixture(300, 128, 10, 10, 12)
    exp, got = run_both(oracle, grab, mix, q, 10, 64, 4, 50, 13, 16, 12345)
    assert_same(exp, got)
    # on this data the search is close to exact: compare with the brute-force ground truth
    gt, _ = oracle.bruteforce_topk(mix.data, q, 10)
    assert datasets.recall(got[0], gt) > 0.8  # 16 random seeds over 10 disconnected clusters


@pytest.mark.parametrize("flags", [0, 1])
def test_range_single_window(oracle, grab, gauss, flags):
    q = datasets.gaussian(150, 128, 3)
    ts = np.arange(gauss.n, dtype=np.uint64)
    win = (900, 1500)
    seeds = np.tile(np.random.default_rng(5).choice(np.arange(900, 1500), 64, replace=False).astype(np.uint32), (150, 1))
    it, ns, _ = grab.search_plan(grab.WRAP_RANGE, 10, 64, 4, gauss.degree, 64)
    exp, got = run_both(oracle, grab, gauss, q, 10, it, 4, 50, 13, ns, 777, seeds=seeds, filter_kind=1, ts=ts,
                        win=win, flags=flags)
    assert_same(exp, got)
    ids = got[0]
    valid = ids[(ids >= 0) & (ids != 0x7FFFFFFF)]
    assert ((valid >= win[0]) & (valid < win[1])).all()  # bound errors == 0


def test_range_per_query_windows(oracle, grab, mix):
    q = datasets.mixture(200, 128, 10, 10, 13)
    ts = np.arange(mix.n, dtype=np.uint64)
    ws, we = datasets.windows(mix.n, 200, 0.1, 3)
    order = np.arange(mix.n, dtype=np.uint32)
    seeds = oracle.sample_window_seeds(ts, order, 64, 99, win_start=ws, win_end=we)
    exp, got = run_both(oracle, grab, mix, q, 10, 64, 4, 50, 13, 64, 1, seeds=seeds, filter_kind=1, ts=ts,
                        win_start=ws, win_end=we)
    assert_same(exp, got)
    ids = got[0]
    for i in range(200):
        v = ids[i][ids[i] >= 0]
        assert ((v >= ws[i]) & (v < we[i])).all()
    gt, _ = oracle.bruteforce_topk(mix.data, q, 10, filter_kind=1, ts=ts, win_start=ws, win_end=we)
    assert datasets.recall(ids, gt) > 0.5


def test_seed_quirks_strict_vs_fixed(oracle, grab, gauss):
    # duplicated seeds, an out-of-window seed and an out-of-range id (replaced by a random one)
    q = datasets.gaussian(50, 128, 4)
    ts = np.arange(gauss.n, dtype=np.uint64)
    base = np.array([1000, 1000, 1001, 5, 0xFFFFFFFF, 1002, 1002, 1003] * 4, np.uint32)
    seeds = np.tile(base, (50, 1))
    for flags in (0, 1):
        exp, got = run_both(oracle, grab, gauss, q, 10, 64, 4, 30, 13, 32, 4242, seeds=seeds, filter_kind=1, ts=ts,
                            win=(990, 1400), flags=flags)
        assert_same(exp, got)
    # fixed mode: no id outside the window, no duplicate ids
    ids = got[0] if flags == 0 else run_both(oracle, grab, gauss, q, 10, 64, 4, 30, 13, 32, 4242, seeds=seeds,
                                             filter_kind=1, ts=ts, win=(990, 1400), flags=0)[1][0]
    for row in ids:
        v = row[row >= 0]
        assert len(set(v.tolist())) == v.size
        assert ((v >= 990) & (v < 1400)).all()


def test_bucket_active_degree(oracle, grab, gauss):
    q = datasets.gaussian(100, 128, 5)
    seeds = np.tile(np.arange(0, 128, dtype=np.uint32), (100, 1))
    it, ns, _ = grab.search_plan(grab.WRAP_BUCKET, 10, 64, 4, gauss.degree, 128)
    assert it == 128 and ns == 128  # clamp of search_bucket_opt
    exp, got = run_both(oracle, grab, gauss, q, 10, it, 4, 50, 13, ns, 31337, seeds=seeds, active_degree=20)
    assert_same(exp, got)


def test_mask_filter_inner_product(oracle, grab):
    data = datasets.unit_rows(2500, 96, 20)
    case = Case(oracle, grab, data, 32, 64)
    labels = datasets.zipf_labels(2500, 64, 1.1, 21)
    q = datasets.unit_rows(120, 96, 22)
    masks = datasets.label_masks(120, 64, 23)
    exp, got = run_both(oracle, grab, case, q, 10, 128, 4, 50, 13, 64, 2024, metric=1, filter_kind=2, labels=labels,
                        masks=masks)
    assert_same(exp, got)
    ids = got[0]
    for i in range(120):
        v = ids[i][ids[i] >= 0]
        assert all((int(masks[i]) >> int(labels[x])) & 1 for x in v)


@pytest.mark.parametrize("dim", [96, 256, 768])
def test_other_dims(oracle, grab, dim):
    case = Case(oracle, grab, datasets.gaussian(1500, dim, 30 + dim), 32, 48)
    q = datasets.gaussian(40, dim, 31)
    exp, got = run_both(oracle, grab, case, q, 10, 64, 4, 40, 13, 16, 555)
    assert_same(exp, got)


def test_visited_set_in_device_memory(oracle, grab, gauss):
    q = datasets.gaussian(20, 128, 6)
    exp, got = run_both(oracle, grab, gauss, q, 10, 64, 4, 45, 16, 16, 999)
    assert_same(exp, got)


@pytest.mark.parametrize("itopk,sw,bitlen,flags", [(1024, 64, 13, 0), (1024, 64, 13, 2), (4096, 16, 13, 0), (64, 128, 13, 0),
                                                   (1024, 64, 16, 0), (256, 8, 13, 0)])
def test_small_batches_with_long_queues_and_wide_iterations(oracle, grab, itopk, sw, bitlen, flags):
    # Batches of up to 256 queries run 1024 threads a query and split their merges over the waves, with partial counts
    # in LDS.  Shapes whose counts would not fit beside the queue and the visited set (the first five) must still run,
    # on the plain merge, with the visited set where it was; the last shape takes the split merge.  flags 2 = the
    # reference's literal behaviour, where a list may hold an id twice (ties in the merge).
    case = Case(oracle, grab, datasets.mixture(3000, 128, 10, 10, 11), 64, 128)
    q = datasets.mixture(40, 128, 10, 10, 12)
    n_seeds = min(itopk // 4, 64)
    exp, got = run_both(oracle, grab, case, q, 10, itopk, sw, 12, bitlen, n_seeds, 0xABCDEF, flags=flags)
    assert_same(exp, got)


def test_exhaustive_search_equals_exact_topk(oracle, grab):
    # itopk >= window size and enough iterations on a connected window: result == exact filtered top-k
    data = datasets.gaussian(400, 128, 40)
    case = Case(oracle, grab, data, 32, 64)
    q = datasets.gaussian(30, 128, 41)
    ids, dists, _, _ = grab.search_ex(case.d_data, case.d_graph, 400, 128, 32, grab.DeviceArray.from_numpy(q), 30, 10,
                                      512, 8, 200, 13, 128, 7)
    gt, gd = oracle.bruteforce_topk(data, q, 10)
    assert np.array_equal(ids, gt)
    assert np.array_equal(dists.view(np.uint32), gd.view(np.uint32))


def test_wrappers_and_errors(oracle, grab, gauss):
    import ctypes as C
    q = datasets.gaussian(16, 128, 7)
    d_q = grab.DeviceArray.from_numpy(q)
    out_i = grab.DeviceArray((16, 10), np.int64)
    out_d = grab.DeviceArray((16, 10), np.float32)
    p = grab.SearchParams(64, 4, 0, 50, 13)
    grab.check(grab.lib.grab_search(C.c_void_p(gauss.d_data.ptr), C.c_size_t(gauss.n), C.c_uint32(128),
                                    C.c_void_p(gauss.d_graph.ptr), C.c_uint32(32), C.c_void_p(d_q.ptr), C.c_int64(16),
                                    C.c_int64(10), p, C.c_void_p(out_i.ptr), C.c_void_p(out_d.ptr), None, C.c_uint32(0),
                                    C.c_uint64(42), C.c_uint32(0), None))
    exp = oracle.search(gauss.data, gauss.graph, q, 10, 64, 4, 50, 13, 16, 42)
    assert np.array_equal(out_i.numpy(), exp[0])
    # null graph -> error, as the reference throws (src/index/cagra.cu:858-860)
    rc = grab.lib.grab_search(C.c_void_p(gauss.d_data.ptr), C.c_size_t(gauss.n), C.c_uint32(128), None, C.c_uint32(32),
                              C.c_void_p(d_q.ptr), C.c_int64(16), C.c_int64(10), p, C.c_void_p(out_i.ptr),
                              C.c_void_p(out_d.ptr), None, C.c_uint32(0), C.c_uint64(42), C.c_uint32(0), None)
    assert rc == 1 and b"Graph is null" in grab.lib.grab_last_error()
    # range wrapper
    ts = grab.DeviceArray.from_numpy(np.arange(gauss.n, dtype=np.uint64))
    seeds = np.tile(np.arange(500, 564, dtype=np.uint32), (16, 1))
    d_s = grab.DeviceArray.from_numpy(seeds)
    grab.check(grab.lib.grab_search_range(C.c_void_p(gauss.d_data.ptr), C.c_uint32(128), C.c_size_t(gauss.n),
                                          C.c_void_p(gauss.d_graph.ptr), C.c_void_p(ts.ptr), C.c_uint32(32), C.c_uint32(32),
                                          C.c_void_p(d_q.ptr), C.c_int64(16), C.c_int64(10), C.c_uint64(400), C.c_uint64(900),
                                          p, C.c_void_p(out_i.ptr), C.c_void_p(out_d.ptr), C.c_void_p(d_s.ptr), C.c_uint32(64),
                                          C.c_uint64(42), C.c_uint32(0), None))
    exp = oracle.search(gauss.data, gauss.graph, q, 10, 64, 4, 50, 13, 64, 42, seeds=seeds, filter_kind=1,
                        ts=np.arange(gauss.n), win=(400, 900))
    assert np.array_equal(out_i.numpy(), exp[0])


def test_id_range_filter_equals_timestamp_filter_on_monotone_timestamps(oracle, grab, mix):
    # timestamps that never decrease with the row id: a window is an id interval, no timestamp is read
    q = datasets.mixture(150, 128, 10, 10, 14)
    ts = (np.arange(mix.n, dtype=np.uint64) // 3) * 5  # repeated, with gaps
    ws = np.random.default_rng(8).integers(0, int(ts[-1]), 150).astype(np.uint64)
    we = ws + np.uint64(900)
    d_ts, d_ws, d_we = (grab.DeviceArray.from_numpy(x) for x in (ts, ws, we))
    lo, hi = grab.windows_to_id_ranges(d_ts, mix.n, d_ws, d_we, 150)
    lo, hi = lo.numpy(), hi.numpy()
    assert np.array_equal(lo, np.searchsorted(ts, ws, side="left")) and np.array_equal(hi, np.searchsorted(ts, we, side="left"))
    seeds = oracle.sample_window_seeds(ts, np.arange(mix.n, dtype=np.uint32), 64, 3, win_start=ws, win_end=we)
    exp_t, got_t = run_both(oracle, grab, mix, q, 10, 64, 4, 50, 13, 64, 1, seeds=seeds, filter_kind=1, ts=ts,
                            win_start=ws, win_end=we)
    exp_i, got_i = run_both(oracle, grab, mix, q, 10, 64, 4, 50, 13, 64, 1, seeds=seeds, filter_kind=3,
                            win_start=lo, win_end=hi)
    assert_same(exp_t, got_t)
    assert_same(exp_i, got_i)
    assert np.array_equal(got_t[0], got_i[0]) and np.array_equal(got_t[1], got_i[1])
    assert int(got_i[2][:, 3].sum()) == 0 and int(got_t[2][:, 3].sum()) > 0  # no filter words read
    assert np.array_equal(got_t[2][:, [0, 1, 2, 4]], got_i[2][:, [0, 1, 2, 4]])


@pytest.mark.parametrize("kind", [1, 2, 3])
def test_filter_before_visited_set(oracle, grab, mix, kind):
    # filter-first keeps rejected rows out of the visited set: same answers from a table 16x smaller
    nq = 160
    q = datasets.mixture(nq, 128, 10, 10, 15)
    ts = np.arange(mix.n, dtype=np.uint64)
    ws, we = datasets.windows(mix.n, nq, 0.1, 5)
    seeds = oracle.sample_window_seeds(ts, np.arange(mix.n, dtype=np.uint32), 32, 17, win_start=ws, win_end=we)
    kw = {}
    if kind == 1:
        kw = dict(ts=ts, win_start=ws, win_end=we)
    elif kind == 3:
        kw = dict(win_start=ws, win_end=we)
    else:
        labels = (np.arange(mix.n) * 64 // mix.n).astype(np.uint8)  # label = position decile-ish
        masks = (np.uint64(1) << (ws * np.uint64(64) // np.uint64(mix.n))) | \
                (np.uint64(1) << (np.minimum(we, mix.n - 1) * np.uint64(64) // np.uint64(mix.n)))
        kw = dict(labels=labels, masks=masks)
    plain = run_both(oracle, grab, mix, q, 10, 64, 4, 50, 13, 32, 3, seeds=seeds, filter_kind=kind, **kw)
    first = run_both(oracle, grab, mix, q, 10, 64, 4, 50, 9, 32, 3, seeds=seeds, filter_kind=kind,
                     flags=grab.FLAG_FILTER_FIRST, **kw)
    assert_same(*plain)
    assert_same(*first)
    assert np.array_equal(plain[1][0], first[1][0]) and np.array_equal(plain[1][1], first[1][1])


def test_large_batch_takes_wave_path_by_default(oracle, grab, gauss):
    q = datasets.gaussian(1500, 128, 9)
    d_q = grab.DeviceArray.from_numpy(q)
    ids, dists, ctr, _ = grab.search_ex(gauss.d_data, gauss.d_graph, gauss.n, 128, gauss.degree, d_q, 1500, 10, 64, 4,
                                        30, 12, 16, 5, want_counters=True)
    exp = oracle.search(gauss.data, gauss.graph, q, 10, 64, 4, 30, 12, 16, 5)
    assert_same(exp, (ids, dists, ctr, None))


def test_wave_lists_shorter_than_an_iteration(oracle, grab, gauss):
    # a small visited set makes the wave-per-query kernel keep short survivor/candidate lists (128 entries here):
    # 256 seeds and 8 x 32 neighbours per iteration, most of them admissible, force it to score and merge early
    nq = 120
    q = datasets.gaussian(nq, 128, 16)
    lo = np.full(nq, 300, np.uint64)
    hi = np.full(nq, 2400, np.uint64)
    rng = np.random.default_rng(3)
    seeds = np.stack([rng.choice(np.arange(300, 2400), 256, replace=False) for _ in range(nq)]).astype(np.uint32)
    exp, got = run_both(oracle, grab, gauss, q, 10, 256, 8, 3, 10, 256, 9, seeds=seeds, filter_kind=3, win_start=lo, win_end=hi,
                        flags=grab.FLAG_FILTER_FIRST)
    assert_same(exp, got)
    assert int(got[2][:, 4].max()) > 128  # more survivors in the run than a list holds


@pytest.mark.parametrize("seed", [1, 2])
def test_random_configurations_match_oracle(oracle, grab, seed):
    """Random draws over sizes, dimensions, degrees, metrics, filters, flags, queue and table sizes: ids, distance bits
    and work counters of both decompositions (and of the automatic choice) against the oracle."""
    rng = np.random.default_rng(seed)
    eq = lambda x, y: np.array_equal(x.view(np.uint32) if x.dtype == np.float32 else x,
                                     y.view(np.uint32) if y.dtype == np.float32 else y)
    compared = 0
    for case in range(6):
        n = int(rng.integers(1500, 4000))
        dim = int(rng.choice([32, 64, 96, 128, 128, 132, 256, 384, 768]))
        degree = int(rng.choice([16, 32, 64]))
        metric = int(rng.integers(0, 2))
        data = datasets.gaussian(n, dim, int(rng.integers(1 << 30))) if rng.random() < 0.6 else \
            datasets.mixture(n, dim, 10, 10, int(rng.integers(1 << 30)))
        graph = oracle.optimize(oracle.knn_graph(data, 2 * degree, metric), degree)
        d_data, d_graph = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(graph)
        for sub in range(4):
            nq = int(rng.choice([3, 70, 260, 1100]))
            k = int(rng.choice([1, 10, 32]))
            itopk = max(int(rng.choice([32, 64, 96, 128, 192, 256, 320])), k)
            sw, max_iter, bitlen = int(rng.integers(1, 9)), int(rng.integers(5, 51)), int(rng.integers(11, 15))
            fk = int(rng.integers(0, 4))
            flags = int(rng.choice([0, grab.FLAG_FILTER_FIRST, grab.FLAG_STRICT_REFERENCE,
                                    grab.FLAG_STRICT_REFERENCE | grab.FLAG_FILTER_FIRST]))
            q = datasets.gaussian(nq, dim, int(rng.integers(1 << 30)))
            kw, dev = {"metric": metric, "filter_kind": fk, "flags": flags}, {}
            ts = rng.permutation(n).astype(np.uint64) if rng.random() < 0.5 else np.arange(n, dtype=np.uint64)
            if fk in (1, 3):
                lo = rng.integers(0, n // 2, nq).astype(np.uint64)
                hi = lo + rng.integers(n // 20, n // 2, nq).astype(np.uint64)
                if fk == 1:
                    kw["ts"], dev["d_ts"] = ts, grab.DeviceArray.from_numpy(ts)
                kw["win_start"], kw["win_end"] = lo, hi
                dev["d_win_start"], dev["d_win_end"] = grab.DeviceArray.from_numpy(lo), grab.DeviceArray.from_numpy(hi)
            if fk == 2:
                labels = rng.integers(0, 64, n).astype(np.uint8)
                masks = rng.integers(1, 1 << 63, nq).astype(np.uint64)
                kw["labels"], kw["masks"] = labels, masks
                dev["d_labels"], dev["d_masks"] = grab.DeviceArray.from_numpy(labels), grab.DeviceArray.from_numpy(masks)
            n_seeds, mask = int(rng.integers(1, itopk + 1)), int(rng.integers(1, 1 << 31))
            exp = oracle.search(data, graph, q, k, itopk, sw, max_iter, bitlen, n_seeds, mask, **kw)
            if int(exp[2][:, 5].sum()) != 0:
                continue  # the visited set overflowed: the outcome depends on the order of the inserts
            d_q = grab.DeviceArray.from_numpy(q)
            what = (f"n {n} dim {dim} degree {degree} metric {metric} nq {nq} k {k} itopk {itopk} width {sw} "
                    f"iterations {max_iter} bitlen {bitlen} filter {fk} flags {flags} seeds {n_seeds}")
            for dec in (grab.FLAG_BLOCK_PER_QUERY, grab.FLAG_WAVE_PER_QUERY, 0):
                got = grab.search_ex(d_data, d_graph, n, dim, degree, d_q, nq, k, itopk, sw, max_iter, bitlen, n_seeds, mask,
                                     metric=metric, filter_kind=fk, flags=flags | dec, want_counters=True, **dev)
                assert eq(exp[0], got[0]), f"ids differ ({what}, decomposition flag {dec})"
                assert eq(exp[1], got[1]), f"distances differ ({what}, decomposition flag {dec})"
                assert np.array_equal(exp[2][:, :5], got[2][:, :5]), f"counters differ ({what}, decomposition flag {dec})"
            compared += 1
    assert compared >= 12


def test_two_batches_in_flight_on_two_streams_match_the_plain_calls(oracle, grab):
    # seed selection and search of two batches queued on two streams, several rounds, nothing awaited in between:
    # every result must equal that of the synchronous calls
    n, dim, deg, k, itopk, nq, ns = 20000, 128, 32, 10, 64, 1500, 16
    data = datasets.mixture(n, dim, 50, 10, 41)
    ts = np.arange(n, dtype=np.uint64)
    d_data, d_ts = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(ts)
    d_knn, _ = grab.generate_knn_graph(d_data, n, dim, 64)
    d_graph = grab.build_graph(d_data, n, d_knn, 64, deg)
    lanes = []
    for b in range(2):
        q = datasets.mixture(nq, dim, 50, 10, 42 + b)
        ws, we = datasets.windows(n, nq, 0.1, 44 + b)
        layer = grab.EntryLayer(d_data, n, dim, 4000, d_ts=d_ts)
        layer.build_groups(40, niter=5, seed=1)
        lane = dict(q=grab.DeviceArray.from_numpy(q), ws=grab.DeviceArray.from_numpy(ws), we=grab.DeviceArray.from_numpy(we),
                    layer=layer, seeds=grab.DeviceArray((nq, ns), np.uint32), lo=grab.DeviceArray((nq,), np.uint64),
                    hi=grab.DeviceArray((nq,), np.uint64), out=(grab.DeviceArray((nq, k), np.int64), grab.DeviceArray((nq, k), np.float32)),
                    stream=grab.Stream())
        lanes.append(lane)

    def step(ln, stream, d_out):
        ln["layer"].select_grouped(ln["q"], nq, ns, 8, 32, d_win_start=ln["ws"], d_win_end=ln["we"], d_out=ln["seeds"], sync=False,
                                   d_base_ts=d_ts, num_base=n, d_id_lo=ln["lo"], d_id_hi=ln["hi"], stream=stream)
        return grab.search_ex(d_data, d_graph, n, dim, deg, ln["q"], nq, k, itopk, 4, 50, 10, ns, 1, d_seeds=ln["seeds"], n_provided=ns,
                              filter_kind=grab.FILTER_ID_RANGE, d_win_start=ln["lo"], d_win_end=ln["hi"],
                              flags=grab.FLAG_FILTER_FIRST, stream=stream, d_out=d_out)

    expected = []
    for ln in lanes:
        grab.synchronize()
        ids, dist, _, _ = step(ln, None, None)
        expected.append((ids, dist))
        assert (ids >= 0).any()
    for rnd in range(6):
        for ln in lanes:
            step(ln, ln["stream"], ln["out"])
    lanes[0]["stream"].wait(lanes[1]["stream"])   # the first stream now ends after both
    lanes[0]["stream"].synchronize()
    for ln, (ids, dist) in zip(lanes, expected):
        assert np.array_equal(ln["out"][0].numpy(), ids)
        assert np.array_equal(ln["out"][1].numpy().view(np.uint32), dist.view(np.uint32))
        ln["stream"].close()
        ln["layer"].close()


def test_long_walks_match_the_literal_model(oracle, grab):
    """Walks of more than 90 iterations (the visited set is rebuilt at 30, 60 and 90) compared directly with the
    literal Python model of the reference's kernels (flat queue, whole-queue sort, table rebuilt before the sort):
    strict mode is the reference as written, the default mode is the reference plus the three documented fixes.
    Integer-valued rows and tie-free queries, so every summation order gives the same distance bits."""
    import ref_literal as lit
    rng = np.random.default_rng(77)
    n, dim, deg = 420, 32, 16
    data = rng.integers(0, 256, (n, dim)).astype(np.float32)
    graph = oracle.optimize(oracle.knn_graph(data, 32), deg)
    graph[::41, 12:] = 0xFFFFFFFF
    q = []
    for cand in rng.integers(0, 256, (200, dim)).astype(np.float32):
        d = ((data.astype(np.float64) - cand.astype(np.float64)) ** 2).sum(axis=1)
        if np.unique(d).size == n:
            q.append(cand)
        if len(q) == 5:
            break
    q = np.stack(q)
    nq = q.shape[0]
    ts = rng.permutation(n).astype(np.uint64)
    window = (60, 330)
    inside = np.nonzero((ts >= window[0]) & (ts < window[1]))[0]
    seeds = rng.choice(inside, (nq, 16)).astype(np.uint32)
    seeds[:, 3] = seeds[:, 2]
    seeds[:, 5] = np.nonzero(ts < 50)[0][:nq]
    d_data, d_graph, d_q = (grab.DeviceArray.from_numpy(x) for x in (data, graph, q))
    d_ts, d_seeds = grab.DeviceArray.from_numpy(ts), grab.DeviceArray.from_numpy(seeds)
    fixes_default = lit.FIX_SEEDS | lit.FIX_RESTORE_ORDER | lit.FIX_EMPTY_SLOTS
    cases = [("plain", 96, 1, 120, 12, 24, None, None), ("plain", 64, 2, 100, 9, 16, None, None),
             ("range", 128, 1, 140, 12, 16, seeds, None), ("strided", 128, 1, 140, 12, 16, seeds, 9)]
    longest = 0
    for variant, itopk, sw, iters, bitlen, n_seeds, sd, active in cases:
        for fixes, flags in ((0, grab.FLAG_STRICT_REFERENCE), (fixes_default, 0)):
            exp = [lit.search_one(data, graph, q[i], 10, itopk, sw, iters, bitlen, n_seeds, None if sd is None else sd[i],
                                  0x9E3779B9, variant=variant, active_degree=active, ts=ts, window=window, fixes=fixes)
                   for i in range(nq)]
            for dec in (grab.FLAG_BLOCK_PER_QUERY, grab.FLAG_WAVE_PER_QUERY):
                ids, dist, ctr, _ = grab.search_ex(
                    d_data, d_graph, n, dim, deg, d_q, nq, 10, itopk, sw, iters, bitlen, n_seeds, 0x9E3779B9,
                    active_degree=active, d_seeds=None if sd is None else d_seeds, n_provided=0 if sd is None else sd.shape[1],
                    filter_kind=1 if variant == "range" else 0, d_ts=d_ts if variant == "range" else None,
                    win=window if variant == "range" else None, flags=flags | dec, want_counters=True)
                for i in range(nq):
                    eids, edist, c = exp[i]
                    what = (variant, itopk, sw, flags, dec, i)
                    assert ids[i].tolist() == eids, what
                    assert np.array_equal(dist[i].view(np.uint32), edist.view(np.uint32)), what
                    assert ctr[i].tolist()[:5] == [c["iterations"], c["S"], c["P"], c["F_fresh"], c["D"]], what
                    assert c["full"] == 0 and int(ctr[i][5]) == 0
                    longest = max(longest, c["iterations"])
    assert longest >= 91


def test_search_opt_and_bucket_wrappers_called_directly(oracle, grab, gauss):
    """grab_search_opt (seeds = max(32, given) capped at the list length) and grab_search_bucket (list of at least 128,
    local slots only) through the C ABI, against the oracle run with the plan of the same wrapper."""
    import ctypes as C
    nq = 24
    q = datasets.gaussian(nq, 128, 17)
    d_q = grab.DeviceArray.from_numpy(q)
    out_i, out_d = grab.DeviceArray((nq, 10), np.int64), grab.DeviceArray((nq, 10), np.float32)
    p = grab.SearchParams(64, 4, 0, 50, 13)
    seeds = np.random.default_rng(18).integers(0, gauss.n, (nq, 20)).astype(np.uint32)
    d_s = grab.DeviceArray.from_numpy(seeds)
    fn = grab.lib.grab_search_opt
    grab.check(fn(C.c_void_p(gauss.d_data.ptr), C.c_uint32(128), C.c_size_t(gauss.n), C.c_void_p(gauss.d_graph.ptr),
                  C.c_uint32(32), C.c_void_p(d_q.ptr), C.c_int64(nq), C.c_int64(10), p, C.c_void_p(out_i.ptr),
                  C.c_void_p(out_d.ptr), C.c_void_p(d_s.ptr), C.c_uint32(20), C.c_uint64(4242), C.c_uint32(0), None))
    it, ns, _ = oracle.search_plan(oracle.WRAP_SEARCH_OPT, 10, 64, 4, 32, 20)
    assert (it, ns) == (64, 32)
    exp = oracle.search(gauss.data, gauss.graph, q, 10, it, 4, 50, 13, ns, 4242, seeds=seeds)
    assert np.array_equal(out_i.numpy(), exp[0]) and np.array_equal(out_d.numpy().view(np.uint32), exp[1].view(np.uint32))
    # without seeds: 32 formula ids
    grab.check(fn(C.c_void_p(gauss.d_data.ptr), C.c_uint32(128), C.c_size_t(gauss.n), C.c_void_p(gauss.d_graph.ptr),
                  C.c_uint32(32), C.c_void_p(d_q.ptr), C.c_int64(nq), C.c_int64(10), p, C.c_void_p(out_i.ptr),
                  C.c_void_p(out_d.ptr), None, C.c_uint32(0), C.c_uint64(99), C.c_uint32(0), None))
    exp = oracle.search(gauss.data, gauss.graph, q, 10, 64, 4, 50, 13, 32, 99)
    assert np.array_equal(out_i.numpy(), exp[0])
    # bucket wrapper: list raised to 128, only the first 20 slots of a row are followed
    seeds = np.tile(np.arange(700, 828, dtype=np.uint32), (nq, 1))
    d_s = grab.DeviceArray.from_numpy(seeds)
    fn = grab.lib.grab_search_bucket
    grab.check(fn(C.c_void_p(gauss.d_data.ptr), C.c_uint32(128), C.c_size_t(gauss.n), C.c_void_p(gauss.d_graph.ptr),
                  C.c_uint32(32), C.c_uint32(20), C.c_void_p(d_q.ptr), C.c_int64(nq), C.c_int64(10), p, C.c_void_p(out_i.ptr),
                  C.c_void_p(out_d.ptr), C.c_void_p(d_s.ptr), C.c_uint32(128), C.c_uint64(7), C.c_uint32(0), None))
    it, ns, _ = oracle.search_plan(oracle.WRAP_BUCKET, 10, 64, 4, 32, 128)
    assert (it, ns) == (128, 128)
    exp = oracle.search(gauss.data, gauss.graph, q, 10, it, 4, 50, 13, ns, 7, seeds=seeds, active_degree=20)
    assert np.array_equal(out_i.numpy(), exp[0]) and np.array_equal(out_d.numpy().view(np.uint32), exp[1].view(np.uint32))


@pytest.mark.parametrize("kind,width,frac", [(3, 4, 0.1), (3, 4, 0.7), (1, 4, 0.3), (2, 3, 0.5), (3, 1, 0.2), (3, 2, 1.0)])
def test_fixed_shape_instance_of_the_register_queue_kernel(oracle, grab, kind, width, frac):
    """Rows of 64 slots, at most four parents, at most 64 seeds, the filter tested first and a list of 64: the wave-per-query
    kernel then runs the instance with that shape compiled in.  Windows from narrow to everything (an iteration can leave
    up to 256 survivors), all three filters, against the oracle: ids, distance bits, counters."""
    n, dim, deg, nq = 5000, 128, 64, 1100
    data = datasets.mixture(n, dim, 10, 10, 51)
    case = Case(oracle, grab, data, deg, 128)
    q = datasets.mixture(nq, dim, 10, 10, 52)
    ts = np.arange(n, dtype=np.uint64)
    ws, we = datasets.windows(n, nq, frac, 53)
    seeds = oracle.sample_window_seeds(ts, np.arange(n, dtype=np.uint32), 48, 7, win_start=ws, win_end=we)
    kw = dict(seeds=seeds, filter_kind=kind, flags=grab.FLAG_FILTER_FIRST)
    if kind == 1:
        kw.update(ts=ts, win_start=ws, win_end=we)
    elif kind == 3:
        kw.update(win_start=ws, win_end=we)
    else:
        labels = (np.arange(n) * 64 // n).astype(np.uint8)
        masks = np.zeros(nq, np.uint64)
        for i in range(nq):
            for b in range(int(ws[i]) * 64 // n, min(63, int(we[i] - 1) * 64 // n) + 1):
                masks[i] |= np.uint64(1) << np.uint64(b)
        kw.update(labels=labels, masks=masks)
    exp, got = run_both(oracle, grab, case, q, 10, 64, width, 40, 13, 48, 99, **kw)
    assert_same(exp, got)
