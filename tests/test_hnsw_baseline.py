"""The CPU HNSW baseline must be a sound index before its timing means anything."""
import numpy as np

import datasets
import hnsw_binding
import oracle_binding as oracle


def test_hnsw_recall_incremental_and_filtered():
    # cfg1 in small: N(0,1) rows added in 10 batches, ids = insertion order, 10 % windows
    n, nq, dim, k = 4000, 200, 64, 10
    data = datasets.gaussian(n, dim, 1)
    q = datasets.gaussian(nq, dim, 2)
    ts = np.arange(n, dtype=np.uint64)
    h = hnsw_binding.Hnsw(dim)
    for b in range(10):
        h.add(data[b * 400:(b + 1) * 400], threads=4)
    assert h.size() == n
    gt, gd = oracle.bruteforce_topk(data, q, k)
    ids, dist = h.search(q, k, ef=128, threads=4)
    assert datasets.recall(ids, gt) > 0.95
    assert (np.diff(dist, axis=1) >= 0).all()
    # distances are those of the ids returned
    i = 7
    assert np.allclose(dist[i], ((data[ids[i]] - q[i]) ** 2).sum(axis=1), rtol=1e-4)
    ws, we = datasets.windows(n, nq, 0.1, 3)
    fgt, _ = oracle.bruteforce_topk(data, q, k, filter_kind=oracle.FILTER_RANGE, ts=ts, win_start=ws, win_end=we)
    fids, _ = h.search_range(q, k, ts, ws, we, ef=128, threads=4)
    for r in range(nq):
        v = fids[r][fids[r] >= 0]
        assert ((v >= ws[r]) & (v < we[r])).all()
    assert datasets.recall(fids, fgt) > 0.9
    h.close()
