"""Exact top-k over sets of buckets (grab_bucket_scan_topk) against the CPU's exact label-set scan."""
import numpy as np
import pytest

import datasets

pytestmark = pytest.mark.gpu


def _case(grab, n, dim, n_buckets, nq, seed, unit, empty=()):
    """Rows stored bucket by bucket with Zipf-sized buckets (the listed ones empty), queries with 1-4 buckets each."""
    rng = np.random.default_rng(seed)
    labels = np.sort(datasets.zipf_labels(n, n_buckets, 1.1, seed + 1))
    for b in empty:
        labels[labels == b] = (b + 1) % n_buckets
    labels = np.sort(labels)
    data = datasets.unit_rows(n, dim, seed + 2) if unit else datasets.mixture(n, dim, 12, seed + 2, seed + 3)
    q = datasets.unit_rows(nq, dim, seed + 4) if unit else datasets.mixture(nq, dim, 12, seed + 2, seed + 5)
    masks = datasets.label_masks(nq, n_buckets, seed + 6)
    offsets = np.searchsorted(labels, np.arange(n_buckets + 1)).astype(np.uint64)
    return data, labels, q, masks, offsets, rng


@pytest.mark.parametrize("n,dim,n_buckets,nq,k,metric,unit", [
    (6000, 128, 8, 300, 10, 0, False),      # integer rows: ties between equal distances go to the lower id
    (20000, 64, 64, 700, 10, 1, True),      # inner product on unit rows, 64 buckets
    (50000, 32, 5, 129, 33, 0, True),       # buckets longer than one piece of 16384 columns, k above 32
    (3000, 768, 64, 64, 10, 1, True),       # the row length of the high-dimensional configuration
])
def test_bucket_scan_equals_the_cpu_label_scan(oracle, grab, n, dim, n_buckets, nq, k, metric, unit):
    data, labels, q, masks, offsets, _ = _case(grab, n, dim, n_buckets, nq, 7 * n_buckets + dim, unit)
    d_data, d_q = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(q)
    ids, dist, _ = grab.bucket_scan_topk(d_data, n, dim, offsets, d_q, nq, k, masks, metric=metric)
    eids, edist = oracle.bruteforce_topk(data, q, k, metric=metric, filter_kind=oracle.FILTER_MASK, labels=labels, masks=masks)
    bad = np.flatnonzero((ids != eids).any(axis=1))
    assert bad.size == 0, f"queries {bad[:5]}: {ids[bad[0]]} vs {eids[bad[0]]}"
    assert np.array_equal(dist.view(np.uint32), edist.view(np.uint32))
    # and the GPU's own scan of every row with the label test
    gids, gdist, _ = grab.bruteforce_topk(d_data, n, dim, d_q, nq, k, metric=metric, filter_kind=grab.FILTER_MASK,
                                          d_labels=grab.DeviceArray.from_numpy(labels), d_masks=grab.DeviceArray.from_numpy(masks))
    assert np.array_equal(ids, gids) and np.array_equal(dist.view(np.uint32), gdist.view(np.uint32))


def test_bucket_scan_queries_that_the_candidates_cannot_prove(oracle, grab):
    # rows that all sit within 0.01 of each other far from the origin: the distances between them are far below the
    # rounding error of |a|^2 + |b|^2 - 2ab, a merged candidate list proves nothing, and every query takes the plain way
    # (a problem per tile-grid row, whose own check sends it on to the scan of every admissible column)
    n, dim, nb, nq, k = 5000, 64, 6, 150, 10
    rng = np.random.default_rng(4)
    data = (np.float32(1000.0) + np.float32(0.01) * rng.standard_normal((n, dim))).astype(np.float32)
    q = (np.float32(1000.0) + np.float32(0.01) * rng.standard_normal((nq, dim))).astype(np.float32)
    labels = np.sort(rng.integers(0, nb, n)).astype(np.uint8)
    masks = datasets.label_masks(nq, nb, 8)
    offsets = np.searchsorted(labels, np.arange(nb + 1)).astype(np.uint64)
    ids, dist, _ = grab.bucket_scan_topk(grab.DeviceArray.from_numpy(data), n, dim, offsets, grab.DeviceArray.from_numpy(q), nq, k, masks)
    sent_on = grab.last_knn_exact_rows()
    eids, edist = oracle.bruteforce_topk(data, q, k, filter_kind=oracle.FILTER_MASK, labels=labels, masks=masks)
    assert np.array_equal(ids, eids) and np.array_equal(dist.view(np.uint32), edist.view(np.uint32))
    assert sent_on > nq // 2, sent_on


def test_bucket_scan_short_and_empty_buckets(oracle, grab):
    # buckets with fewer rows than k, empty buckets, queries whose buckets are all empty, a mask bit beyond the buckets
    n, dim, nb, nq, k = 900, 32, 16, 200, 20
    data, labels, q, masks, offsets, rng = _case(grab, n, dim, nb, nq, 3, False, empty=(2, 9, 15))
    masks[:5] = np.uint64(1 << 2)                       # only an empty bucket
    masks[5:9] = np.uint64((1 << 9) | (1 << 15))
    masks[9] = np.uint64((1 << 40) | (1 << 3))          # a bucket that does not exist is ignored
    sizes = np.diff(offsets.astype(np.int64))
    assert (sizes == 0).sum() >= 3 and ((sizes > 0) & (sizes < k)).any()
    d_data, d_q = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(q)
    ids, dist, _ = grab.bucket_scan_topk(d_data, n, dim, offsets, d_q, nq, k, masks)
    eids, edist = oracle.bruteforce_topk(data, q, k, filter_kind=oracle.FILTER_MASK, labels=labels,
                                         masks=masks & np.uint64((1 << nb) - 1))
    assert np.array_equal(ids, eids)
    assert (ids[:9] == -1).all() and (ids[9] >= 0).any()
    valid = ids >= 0
    assert np.array_equal(dist.view(np.uint32)[valid], edist.view(np.uint32)[valid])
    # all queries empty
    ids0, _, _ = grab.bucket_scan_topk(d_data, n, dim, offsets, d_q, 4, k, masks[:4])
    assert (ids0 == -1).all()
    # argument errors
    import ctypes as C
    bad = offsets.copy()
    bad[3] = bad[4] + 1
    assert grab.lib.grab_bucket_scan_topk(C.c_void_p(d_data.ptr), C.c_size_t(n), C.c_uint32(dim), bad.ctypes.data_as(C.c_void_p),
                                          C.c_uint32(nb), C.c_void_p(d_q.ptr), C.c_size_t(4), C.c_uint32(k), C.c_int(0),
                                          masks.ctypes.data_as(C.c_void_p), C.c_void_p(d_data.ptr), C.c_void_p(d_data.ptr), None, None) == 1
    assert b"offsets" in grab.lib.grab_last_error()
