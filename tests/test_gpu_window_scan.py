"""Exact top-k inside intervals of row ids (grab_window_scan_topk) against the CPU's exact range-filtered scan."""
import numpy as np
import pytest

import datasets

pytestmark = pytest.mark.gpu


def _intervals(n, nq, width_lo, width_hi, seed):
    rng = np.random.default_rng(seed)
    w = rng.integers(width_lo, width_hi + 1, nq)
    lo = rng.integers(0, np.maximum(n - w, 1))
    return lo.astype(np.uint64), np.minimum(lo + w, n).astype(np.uint64)


@pytest.mark.parametrize("n,dim,nq,k,metric,kind,widths", [
    (6000, 128, 300, 10, 0, "mix", (40, 900)),       # integer rows: ties between equal distances go to the lower id
    (40000, 64, 1500, 10, 1, "unit", (300, 500)),    # inner product, more than 1024 queries: rows as bf16 halves
    (70000, 32, 1100, 33, 0, "unit", (5, 30000)),    # intervals from shorter than k to long ones, k above 32
    (9000, 768, 130, 10, 1, "unit", (100, 2000)),    # long rows
    (30000, 132, 1200, 10, 0, "gauss", (200, 4000)), # a row length that is no whole number of 32-dimension chunks: fp32 instructions
])
def test_window_scan_equals_the_cpu_range_scan(oracle, grab, n, dim, nq, k, metric, kind, widths):
    data = {"mix": lambda: datasets.mixture(n, dim, 12, 3, 4), "unit": lambda: datasets.unit_rows(n, dim, 5),
            "gauss": lambda: datasets.gaussian(n, dim, 6)}[kind]()
    q = {"mix": lambda: datasets.mixture(nq, dim, 12, 3, 7), "unit": lambda: datasets.unit_rows(nq, dim, 8),
         "gauss": lambda: datasets.gaussian(nq, dim, 9)}[kind]()
    lo, hi = _intervals(n, nq, widths[0], widths[1], n + dim)
    d_data, d_q = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(q)
    ids, dist, _ = grab.window_scan_topk(d_data, n, dim, d_q, nq, k, lo, hi, metric=metric)
    ts = np.arange(n, dtype=np.uint64)
    eids, edist = oracle.bruteforce_topk(data, q, k, metric=metric, filter_kind=oracle.FILTER_RANGE, ts=ts, win_start=lo, win_end=hi)
    bad = np.flatnonzero((ids != eids).any(axis=1))
    assert bad.size == 0, f"queries {bad[:5]}: {ids[bad[0]]} vs {eids[bad[0]]} in [{lo[bad[0]]}, {hi[bad[0]]})"
    valid = ids >= 0
    assert np.array_equal(dist.view(np.uint32)[valid], edist.view(np.uint32)[valid])
    assert ((ids >= lo[:, None].astype(np.int64)) & (ids < hi[:, None].astype(np.int64)))[valid].all()
    on_bf16 = dim % 32 == 0 and nq >= 1024 - 127 and n >= 4096
    assert (grab.last_knn_bf16_flop() > 0) == on_bf16
    # and the GPU's own scan of every row with the window test
    gids, gdist, _ = grab.bruteforce_topk(d_data, n, dim, d_q, nq, k, metric=metric, filter_kind=grab.FILTER_RANGE,
                                          d_ts=grab.DeviceArray.from_numpy(ts), d_win_start=grab.DeviceArray.from_numpy(lo),
                                          d_win_end=grab.DeviceArray.from_numpy(hi))
    assert np.array_equal(ids, gids) and np.array_equal(dist.view(np.uint32)[valid], gdist.view(np.uint32)[valid])


def test_window_scan_empty_short_and_overlong_intervals(oracle, grab):
    n, dim, nq, k = 3000, 32, 140, 12
    data, q = datasets.mixture(n, dim, 6, 1, 2), datasets.mixture(nq, dim, 6, 1, 3)
    lo, hi = _intervals(n, nq, 1, 400, 11)
    lo[:6], hi[:6] = [5, 700, 2999, 3000, 4000, 10], [5, 600, 3000, 3000, 5000, 9]      # empty, reversed, last row, beyond the end
    lo[6], hi[6] = 2990, 1 << 40                                                       # an end far beyond the rows is cut
    lo[7], hi[7] = 0, n                                                                # every row
    d_data, d_q = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(q)
    ids, dist, _ = grab.window_scan_topk(d_data, n, dim, d_q, nq, k, lo, hi)
    eids, edist = oracle.bruteforce_topk(data, q, k, filter_kind=oracle.FILTER_RANGE, ts=np.arange(n, dtype=np.uint64), win_start=lo,
                                         win_end=np.minimum(hi, np.uint64(n)))
    assert np.array_equal(ids, eids)
    assert (ids[[0, 1, 3, 4, 5]] == -1).all() and ids[2, 0] == 2999 and (ids[2, 1:] == -1).all()
    assert (ids[6] >= 0).sum() == 10 and (ids[7] >= 0).all()
    valid = ids >= 0
    assert np.array_equal(dist.view(np.uint32)[valid], edist.view(np.uint32)[valid])
    # no query admits a row
    ids0, _, _ = grab.window_scan_topk(d_data, n, dim, d_q, 3, k, np.array([4, 9, 3000], np.uint64), np.array([4, 2, 3000], np.uint64))
    assert (ids0 == -1).all()
    with pytest.raises(grab.GrabError):
        grab.window_scan_topk(d_data, n, dim, d_q, nq, 200, lo, hi)


def test_window_scan_queries_that_the_candidates_cannot_prove(oracle, grab):
    # rows within 0.01 of each other far from the origin: a candidate list of GEMM-form keys proves nothing there, and
    # the queries take the plain way (a problem per query row, whose own check goes on to the scan of the interval)
    n, dim, nq, k = 5000, 64, 150, 10
    rng = np.random.default_rng(4)
    data = (np.float32(1000.0) + np.float32(0.01) * rng.standard_normal((n, dim))).astype(np.float32)
    q = (np.float32(1000.0) + np.float32(0.01) * rng.standard_normal((nq, dim))).astype(np.float32)
    lo, hi = _intervals(n, nq, 100, 1500, 12)
    ids, dist, _ = grab.window_scan_topk(grab.DeviceArray.from_numpy(data), n, dim, grab.DeviceArray.from_numpy(q), nq, k, lo, hi)
    sent_on = grab.last_knn_exact_rows()
    eids, edist = oracle.bruteforce_topk(data, q, k, filter_kind=oracle.FILTER_RANGE, ts=np.arange(n, dtype=np.uint64), win_start=lo, win_end=hi)
    assert np.array_equal(ids, eids) and np.array_equal(dist.view(np.uint32), edist.view(np.uint32))
    assert sent_on > nq // 2, sent_on


def test_prepared_base_gives_the_same_answers_call_after_call(oracle, grab):
    # the base's rows are split once and the calls' scratch is kept: a large call, a small one, another metric's base,
    # the bucket scan on the same base - every answer equal to the one-shot entry points'
    n, dim, k = 30000, 64, 10
    data = datasets.unit_rows(n, dim, 31)
    d_data = grab.DeviceArray.from_numpy(data)
    free0 = grab.device_memory()[0]
    for metric in (0, 1):
        base = grab.ScanBase(d_data, n, dim, metric)
        for nq, widths, seed in ((1500, (200, 3000), 1), (70, (10, 400), 2), (1500, (50, 9000), 3)):
            q = datasets.unit_rows(nq, dim, 40 + seed)
            d_q = grab.DeviceArray.from_numpy(q)
            lo, hi = _intervals(n, nq, widths[0], widths[1], seed)
            ids, dist, _ = base.window_topk(d_q, nq, k, lo, hi)
            assert grab.last_knn_bf16_flop() > 0      # the base holds split rows, so small calls use them too
            eids, edist, _ = grab.window_scan_topk(d_data, n, dim, d_q, nq, k, lo, hi, metric=metric)
            assert np.array_equal(ids, eids) and np.array_equal(dist.view(np.uint32), edist.view(np.uint32))
            oids, _ = oracle.bruteforce_topk(data, q[:40], k, metric=metric, filter_kind=oracle.FILTER_RANGE, ts=np.arange(n, dtype=np.uint64),
                                             win_start=lo[:40], win_end=hi[:40])
            assert np.array_equal(ids[:40], oids)
        labels = np.sort(datasets.zipf_labels(n, 16, 1.1, 5))
        offsets = np.searchsorted(labels, np.arange(17)).astype(np.uint64)
        masks = datasets.label_masks(300, 16, 6)
        d_q = grab.DeviceArray.from_numpy(datasets.unit_rows(300, dim, 50))
        ids, dist, _ = base.bucket_topk(offsets, d_q, 300, k, masks)
        eids, edist, _ = grab.bucket_scan_topk(d_data, n, dim, offsets, d_q, 300, k, masks, metric=metric)
        assert np.array_equal(ids, eids) and np.array_equal(dist.view(np.uint32), edist.view(np.uint32))
        base.close()
    assert grab.device_memory()[0] >= free0 - (8 << 20)   # a closed base gives its memory back


def test_index_handle_scans_windows_exactly(oracle, grab):
    # the handle's exact range search: rows in timestamp order (several rows per timestamp) go through the prepared
    # base, which is remade after an insert; rows in any other order are scanned with the window test
    n0, n1, dim, k, nq = 6000, 1500, 64, 10, 300
    data = datasets.mixture(n0 + n1, dim, 20, 3, 4)
    ts = (np.arange(n0 + n1, dtype=np.uint64) // 7) * 3
    q = datasets.mixture(nq, dim, 20, 3, 5)
    rng = np.random.default_rng(6)
    ws = rng.integers(0, int(ts[n0 - 1]), nq).astype(np.uint64)
    we = ws + rng.integers(1, 600, nq).astype(np.uint64)
    ws[:3], we[:3] = [10**9, 50, 0], [10**9 + 5, 50, 1]     # beyond every row, empty, the first timestamp only
    idx = grab.CagraIndex(dim, 32, vmm_max_bytes=1 << 30)
    idx.add(data[:n0], ts[:n0])
    idx.build()
    for n in (n0, n0 + n1):
        if n > n0:
            idx.insert(data[n0:n], ts[n0:n])
        ids, dist = idx.scan_range_batch(q, k, ws, we)
        eids, edist = oracle.bruteforce_topk(data[:n], q, k, filter_kind=oracle.FILTER_RANGE, ts=ts[:n], win_start=ws, win_end=we)
        assert np.array_equal(ids, eids)
        valid = ids >= 0
        assert np.array_equal(dist.view(np.uint32)[valid], edist.view(np.uint32)[valid]) and (dist[~valid] == -1.0).all()
        assert (ids[:2] == -1).all() and (ids[2] >= 0).sum() == 7
    idx.close()
    # timestamps in no order
    ts2 = rng.permutation(ts[:n0])
    idx = grab.CagraIndex(dim, 32, vmm_max_bytes=1 << 30)
    idx.add(data[:n0], ts2)
    idx.build()
    ids, dist = idx.scan_range_batch(q, k, ws, we)
    eids, edist = oracle.bruteforce_topk(data[:n0], q, k, filter_kind=oracle.FILTER_RANGE, ts=ts2, win_start=ws, win_end=we)
    assert np.array_equal(ids, eids)
    idx.close()


def test_range_batches_scan_their_narrow_windows(oracle, grab):
    # set_scan_below: one call, the narrow windows scanned exactly, the wide ones searched on the graph as ever
    n, dim, k, nq = 8000, 64, 10, 400
    data = datasets.mixture(n, dim, 20, 3, 4)
    ts = np.arange(n, dtype=np.uint64) * 2
    q = datasets.mixture(nq, dim, 20, 3, 5)
    rng = np.random.default_rng(9)
    width = np.where(rng.random(nq) < 0.5, rng.integers(20, 300, nq), rng.integers(2000, 6000, nq)).astype(np.uint64)
    ws = rng.integers(0, 2 * n - 2 * int(width.max()), nq).astype(np.uint64)
    we = ws + 2 * width
    idx = grab.CagraIndex(dim, 32, vmm_max_bytes=1 << 30)
    idx.set_seed(5)
    idx.setQueryParams(64, 4, 0, 50, 12)
    idx.add(data, ts)
    idx.build()
    plain_ids, plain_dist = idx.query_range_batch(q, k, ws, we)
    idx.set_seed(5)
    idx.set_scan_below(0.05)                      # 400 rows
    ids, dist = idx.query_range_batch(q, k, ws, we)
    narrow = width <= 400
    assert narrow.any() and (~narrow).any()
    eids, edist = oracle.bruteforce_topk(data, q, k, filter_kind=oracle.FILTER_RANGE, ts=ts, win_start=ws, win_end=we)
    assert np.array_equal(ids[narrow], eids[narrow])
    assert np.array_equal(dist[narrow].view(np.uint32), edist[narrow].view(np.uint32))
    # the wide ones: a graph search of that half alone with the same generator state
    idx.set_scan_below(0.0)
    idx.set_seed(5)
    wide_ids, wide_dist = idx.query_range_batch(q[~narrow], k, ws[~narrow], we[~narrow])
    assert np.array_equal(ids[~narrow], wide_ids) and np.array_equal(dist[~narrow].view(np.uint32), wide_dist.view(np.uint32))
    assert datasets.recall(ids, eids) >= datasets.recall(plain_ids, eids)
    # all narrow / none narrow
    idx.set_scan_below(1.0)
    a, _ = idx.query_range_batch(q, k, ws, we)
    assert np.array_equal(a, eids)
    idx.close()


def test_window_scan_in_several_passes(oracle, grab):
    # the dense block is made in passes of at most 128 row tiles (16,384 queries) and at most 4 GiB: more queries than a
    # pass takes, and intervals so long that 16 row tiles already pass the 4 GiB
    n, dim, k = 60000, 32, 10
    data = datasets.unit_rows(n, dim, 61)
    d_data = grab.DeviceArray.from_numpy(data)
    ts = grab.DeviceArray.from_numpy(np.arange(n, dtype=np.uint64))
    nq = 20000
    q = datasets.unit_rows(nq, dim, 62)
    d_q = grab.DeviceArray.from_numpy(q)
    lo, hi = _intervals(n, nq, 50, 700, 63)
    ids, dist, _ = grab.window_scan_topk(d_data, n, dim, d_q, nq, k, lo, hi)
    gids, gdist, _ = grab.bruteforce_topk(d_data, n, dim, d_q, nq, k, filter_kind=grab.FILTER_RANGE, d_ts=ts,
                                          d_win_start=grab.DeviceArray.from_numpy(lo), d_win_end=grab.DeviceArray.from_numpy(hi))
    assert np.array_equal(ids, gids) and np.array_equal(dist.view(np.uint32), gdist.view(np.uint32))
    pick = np.arange(0, nq, 997)
    eids, _ = oracle.bruteforce_topk(data, q[pick], k, filter_kind=oracle.FILTER_RANGE, ts=np.arange(n, dtype=np.uint64),
                                     win_start=lo[pick], win_end=hi[pick])
    assert np.array_equal(ids[pick], eids)
    del d_data, d_q, ts

    n, nq = 1_000_000, 2100                      # 17 row tiles x 128 rows x ~600,000 columns x 4 bytes: 5 GB
    data = datasets.unit_rows(n, dim, 64)
    q = datasets.unit_rows(nq, dim, 65)
    d_data, d_q = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(q)
    ts = grab.DeviceArray.from_numpy(np.arange(n, dtype=np.uint64))
    lo, hi = _intervals(n, nq, 500000, 520000, 66)
    ids, dist, _ = grab.window_scan_topk(d_data, n, dim, d_q, nq, k, lo, hi)
    gids, gdist, _ = grab.bruteforce_topk(d_data, n, dim, d_q, nq, k, filter_kind=grab.FILTER_RANGE, d_ts=ts,
                                          d_win_start=grab.DeviceArray.from_numpy(lo), d_win_end=grab.DeviceArray.from_numpy(hi))
    assert np.array_equal(ids, gids) and np.array_equal(dist.view(np.uint32), gdist.view(np.uint32))
