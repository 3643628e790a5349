"""Insert into the time-partitioned graph on the GPU against the CPU restatement (bit for bit), and
through the index handle: what the inserted rows do to searches inside their bucket."""
import numpy as np
import pytest

import datasets

pytestmark = pytest.mark.gpu

SIZES = [700, 300, 1100, 40, 860]


def _partitioned(oracle, n_new, dim, total, local, metric, bucket, seed=5):
    n_old = sum(SIZES)
    data = datasets.unit_rows(n_old + n_new, dim, seed) if metric else datasets.gaussian(n_old + n_new, dim, seed)
    ts = np.concatenate([np.repeat(np.arange(len(SIZES), dtype=np.uint64), SIZES), np.full(n_new, bucket, np.uint64)])
    g0 = oracle.build_time_partitioned(data[:n_old], ts[:n_old], SIZES, total, local, metric)
    graph = np.concatenate([g0, np.full((n_new, total), 0xFFFFFFFF, np.uint32)])
    return n_old, data, ts, graph


@pytest.mark.parametrize("metric,n_new,itopk,bucket,n_seeds,flags", [
    (0, 32, 128, 2, 128, 0),   # the shape CagraIndexOpt::insert uses
    (0, 32, 128, 2, 128, 1),   # strict reference traversal
    (1, 17, 64, 0, 32, 0),     # inner product, a ragged step, a list shorter than the bucket wrapper's floor
    (0, 150, 96, 4, 40, 0),    # more rows than half the list: the batch supplies itopk/2 candidates
    (0, 8, 128, 3, 64, 0),     # a bucket with fewer rows than seeds asked for
    (0, 5, 32, 7, 32, 0),      # a bucket that does not exist yet: no seeds, local slots come from the batch alone
])
def test_insert_partitioned_step_matches_oracle(oracle, grab, metric, n_new, itopk, bucket, n_seeds, flags):
    dim, total, local = 64, 32, 24
    n_old, data, ts, graph = _partitioned(oracle, n_new, dim, total, local, metric, bucket)
    rng = np.random.default_rng(n_new)
    members = np.flatnonzero(ts[:n_old] == bucket).astype(np.uint32)
    row = np.full(n_seeds, 0xFFFFFFFF, np.uint32)
    pick = members if len(members) <= n_seeds else np.sort(rng.choice(members, n_seeds, replace=False))
    row[:len(pick)] = pick
    seeds = np.tile(row, (n_new, 1))
    exp, state = oracle.insert_partitioned_batch(data, ts, n_old, n_new, bucket, graph, local, seeds, itopk, 4, 100, 14, 4242,
                                                 metric=metric, flags=flags)
    d_data, d_graph, d_ts = (grab.DeviceArray.from_numpy(x) for x in (data, graph, ts))
    new_state = grab.insert_partitioned(d_data, d_graph, d_ts, grab.DeviceArray.from_numpy(seeds), n_old, n_new, bucket, dim,
                                        total, local, grab.SearchParams(itopk, 4, 0, 100, 14), n_seeds, 4242, metric=metric,
                                        flags=flags)
    got = d_graph.numpy()
    assert new_state == state
    bad = np.nonzero((exp != got).any(axis=1))[0]
    assert bad.size == 0, f"{bad.size} rows differ, first {bad[0]}: {exp[bad[0]]} vs {got[bad[0]]}"
    new = got[n_old:]
    loc = new[:, :local]
    filled = loc != 0xFFFFFFFF
    assert (ts[loc[filled]] == bucket).all()                       # local slots stay inside the bucket
    if len(members) >= n_seeds:  # seeds that are missing are drawn from all rows, and the search then leaves the bucket
        assert filled.sum(1).min() >= local // 2
    assert not (new == np.arange(n_old, n_old + n_new, dtype=np.uint32)[:, None]).any()
    changed = got[:n_old] != graph[:n_old]
    assert (got[:n_old][changed] >= n_old).all()                    # old rows only gain new rows
    if len(members):
        assert changed.any()
    assert (ts[:n_old][changed[:, local:].any(1)] != bucket).all()  # remote requests never go to the bucket itself


def test_insert_partitioned_rejects_bad_arguments(grab):
    d = grab.DeviceArray.from_numpy(np.zeros((64, 16), np.float32))
    g = grab.DeviceArray.from_numpy(np.zeros((64, 8), np.uint32))
    t = grab.DeviceArray.from_numpy(np.zeros(64, np.uint64))
    s = grab.DeviceArray.from_numpy(np.zeros((4, 32), np.uint32))
    p = grab.SearchParams(64, 4, 0, 10, 12)
    with pytest.raises(grab.GrabError):
        grab.insert_partitioned(d, g, t, s, 60, 4, 0, 16, 8, 8, p, 32, 1)       # no remote slots
    with pytest.raises(grab.GrabError):
        grab.insert_partitioned(d, g, t, s, 0, 4, 0, 16, 8, 6, p, 32, 1)        # nothing to search
    with pytest.raises(grab.GrabError):
        grab.insert_partitioned(d, g, t, s, 60, 4, 0, 16, 8, 6, grab.SearchParams(1024, 4, 0, 10, 12), 32, 1)  # merged list too long
    with pytest.raises(grab.GrabError):
        grab.insert_partitioned(d, g, t, s, 10, 2000, 0, 16, 8, 6, p, 32, 1)    # too many rows in one call


def test_index_insert_partitioned_keeps_bucket_searches_good(oracle, grab):
    # 20 buckets of 600 rows are built; then every bucket receives 100 more rows, bucket by bucket.
    nb, per, extra, dim, deg, local, k = 20, 600, 100, 64, 32, 24, 10
    n0 = nb * per
    base = datasets.mixture(n0 + nb * extra, dim, 40, 10, 21)
    data, later = base[:n0], base[n0:]
    ts = np.repeat(np.arange(nb, dtype=np.uint64), per)
    idx = grab.CagraIndex(dim, deg, vmm_max_bytes=1 << 28, local_degree=local)
    idx.setQueryParams(64, 4, 0, 50, 13)
    idx.set_seed(9)
    idx.add(data, ts)
    idx.build_partitioned()
    with pytest.raises(grab.GrabError):
        grab.CagraIndex(dim, deg, vmm_max_bytes=1 << 24).insert_partitioned(later[:4], np.zeros(4, np.uint64))  # no split, empty
    for b in range(nb):
        idx.insert_partitioned(later[b * extra:(b + 1) * extra], np.full(extra, b, np.uint64))
    assert idx.size() == n0 + nb * extra
    all_data = np.concatenate([data, later])
    all_ts = np.concatenate([ts, np.repeat(np.arange(nb, dtype=np.uint64), extra)])
    g = idx.get_graph()
    assert g.shape == (len(all_data), deg)
    new = g[n0:]
    assert (new != 0xFFFFFFFF).all()
    assert (all_ts[new[:, :local]] == all_ts[n0:, None]).all()         # local slots inside the bucket
    assert (new[:, :local] >= n0).any() and (g[:n0] >= n0).any()        # batch neighbours and reverse edges exist
    q = datasets.mixture(200, dim, 40, 10, 22)
    rec_all, rec_new = [], []
    for b in (0, 7, 19):
        ids, _ = idx.query_range(q, k, 0.5, b, b + 1)
        gt, _ = oracle.bruteforce_topk(all_data, q, k, filter_kind=oracle.FILTER_RANGE, ts=all_ts, win=(b, b + 1))
        assert (all_ts[ids[ids >= 0]] == b).all()
        rec_all.append(datasets.recall(ids, gt))
        want = gt >= n0  # how many of the true neighbours that were inserted later are found
        rec_new.append(sum(len(set(gt[i][want[i]].tolist()) & set(ids[i].tolist())) for i in range(len(q))) / max(1, want.sum()))
    print("recall@10 inside a bucket after inserts:", rec_all, "of the inserted rows:", rec_new)
    assert min(rec_all) > 0.9 and min(rec_new) > 0.8
    idx.close()


def test_index_insert_partitioned_is_reproducible(grab):
    # the two searches of a step run on two streams and the steps follow each other without a host round trip:
    # the same seed must give the same graph, run after run, and the bucket's old rows must be the only seeds' source
    nb, per, extra, dim, deg, local = 6, 500, 200, 32, 32, 24
    n0 = nb * per
    base = datasets.mixture(n0 + 2 * extra, dim, 12, 10, 31)
    ts = np.repeat(np.arange(nb, dtype=np.uint64), per)
    graphs = []
    for run in range(3):
        idx = grab.CagraIndex(dim, deg, vmm_max_bytes=1 << 28, local_degree=local)
        idx.set_seed(77)
        idx.add(base[:n0], ts)
        idx.build_partitioned()
        idx.insert_partitioned(base[n0:n0 + extra], np.full(extra, 2, np.uint64))
        idx.insert_partitioned(base[n0 + extra:], np.full(extra, 5, np.uint64))
        graphs.append(idx.get_graph())
        idx.close()
    assert np.array_equal(graphs[0], graphs[1]) and np.array_equal(graphs[0], graphs[2])
    g = graphs[0]
    assert g.shape == (n0 + 2 * extra, deg) and (g[n0:] != 0xFFFFFFFF).all()


def test_partitioned_build_and_insert_random_configurations(oracle, grab):
    # random bucket sizes, degrees, metrics, list lengths and flags: the build and one insert step against the oracle.
    # The draw with the strict traversal, inner product and 6 local slots leaves an id twice in a bucket list, which
    # the merge with the batch neighbours must keep twice.
    rng = np.random.default_rng(7)
    for case in range(10):
        nb = int(rng.integers(2, 8))
        sizes = [int(x) for x in rng.integers(30, 900, nb)]
        n_old = sum(sizes)
        dim, total = int(rng.choice([32, 64, 128])), int(rng.choice([16, 32, 64]))
        local = int(rng.integers(total // 4, total - 1))
        metric, n_new, itopk = int(rng.integers(0, 2)), int(rng.choice([1, 5, 17, 32, 64, 150])), int(rng.choice([32, 64, 96, 128]))
        bucket, n_seeds, flags = int(rng.integers(0, nb + 1)), int(rng.choice([16, 32, 64, 128])), int(rng.choice([0, 0, 1]))
        seed = int(rng.integers(1 << 30))
        data = datasets.unit_rows(n_old + n_new, dim, seed) if metric else datasets.gaussian(n_old + n_new, dim, seed)
        ts = np.concatenate([np.repeat(np.arange(nb, dtype=np.uint64), sizes), np.full(n_new, bucket, np.uint64)])
        what = f"case {case}: sizes {sizes} dim {dim} total {total} local {local} metric {metric} new {n_new} itopk {itopk} " \
               f"bucket {bucket} seeds {n_seeds} flags {flags}"
        g0 = oracle.build_time_partitioned(data[:n_old], ts[:n_old], sizes, total, local, metric)
        gg = grab.build_time_partitioned_graph(grab.DeviceArray.from_numpy(data[:n_old]), n_old, dim,
                                               grab.DeviceArray.from_numpy(ts[:n_old]), sizes, total, local, metric).numpy()
        assert np.array_equal(g0, gg), what
        graph = np.concatenate([g0, np.full((n_new, total), 0xFFFFFFFF, np.uint32)])
        members = np.flatnonzero(ts[:n_old] == bucket).astype(np.uint32)
        row = np.full(n_seeds, 0xFFFFFFFF, np.uint32)
        pick = members if len(members) <= n_seeds else np.sort(rng.choice(members, n_seeds, replace=False))
        row[:len(pick)] = pick
        seeds = np.tile(row, (n_new, 1))
        state = int(rng.integers(1, 1 << 40))
        exp, st = oracle.insert_partitioned_batch(data, ts, n_old, n_new, bucket, graph, local, seeds, itopk, 4, 100, 14, state,
                                                  metric=metric, flags=flags)
        d_data, d_graph, d_ts = (grab.DeviceArray.from_numpy(x) for x in (data, graph, ts))
        ns = grab.insert_partitioned(d_data, d_graph, d_ts, grab.DeviceArray.from_numpy(seeds), n_old, n_new, bucket, dim, total, local,
                                     grab.SearchParams(itopk, 4, 0, 100, 14), n_seeds, state, metric=metric, flags=flags)
        got = d_graph.numpy()
        bad = np.nonzero((exp != got).any(axis=1))[0]
        assert ns == st and bad.size == 0, f"{what}: {bad.size} rows differ, first {bad[:5]}"
