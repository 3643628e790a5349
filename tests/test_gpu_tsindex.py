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
