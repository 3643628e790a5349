"""grab_search_ex_static - the search entry point that allocates nothing - against grab_search_ex on the same
inputs: ids, distance bits and work counters, on two calls in a row, the second with a smaller input (the array
that holds the visited sets keeps the first call's contents), then the size limit and the LDS-only case."""
import numpy as np
import pytest

import datasets

pytestmark = pytest.mark.gpu


def _both(grab, d_data, d_graph, n, dim, deg, q, k, itopk, sw, iters, bitlen, n_seeds, mask, **kw):
    nq = q.shape[0]
    d_q = grab.DeviceArray.from_numpy(q)
    exp = grab.search_ex(d_data, d_graph, n, dim, deg, d_q, nq, k, itopk, sw, iters, bitlen, n_seeds, mask,
                         want_counters=True, **kw)
    out = (grab.DeviceArray((nq, k), np.int64), grab.DeviceArray((nq, k), np.float32))
    ctr = grab.DeviceArray((nq, 6), np.uint64)
    grab.search_ex(d_data, d_graph, n, dim, deg, d_q, nq, k, itopk, sw, iters, bitlen, n_seeds, mask, d_out=out,
                   static_tables=True, d_counters=ctr, **kw)
    grab.synchronize()
    assert np.array_equal(out[0].numpy(), exp[0]), "ids differ"
    assert np.array_equal(out[1].numpy().view(np.uint32), exp[1].view(np.uint32)), "distances differ"
    assert np.array_equal(ctr.numpy(), exp[2]), "work counters differ"
    return exp


def test_static_visited_sets_match_allocated_ones(oracle, grab):
    n, dim, deg = 3000, 128, 32
    data = datasets.gaussian(n, dim, 1)
    graph = oracle.optimize(oracle.knn_graph(data, 64), deg)
    d_data, d_graph = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(graph)
    ts = np.arange(n, dtype=np.uint64)
    d_ts = grab.DeviceArray.from_numpy(ts)
    # 1st call: 60 queries x 2^16 slots = 15 MiB of tables in the static array (unfiltered)
    q1 = datasets.gaussian(60, dim, 2)
    e1 = _both(grab, d_data, d_graph, n, dim, deg, q1, 10, 64, 4, 45, 16, 16, 999)
    o1 = oracle.search(data, graph, q1, 10, 64, 4, 45, 16, 16, 999)
    assert np.array_equal(e1[0], o1[0]) and np.array_equal(e1[2][:, :5], o1[2][:, :5])
    # 2nd call, smaller input, other parameters: 7 queries x 2^17 slots, range filter, wider
    q2 = datasets.gaussian(7, dim, 3)
    seeds = np.tile(np.arange(800, 832, dtype=np.uint32), (7, 1))
    e2 = _both(grab, d_data, d_graph, n, dim, deg, q2, 5, 96, 6, 40, 17, 32, 5, d_seeds=grab.DeviceArray.from_numpy(seeds),
               n_provided=32, filter_kind=1, d_ts=d_ts, win=(700, 1900))
    o2 = oracle.search(data, graph, q2, 5, 96, 6, 40, 17, 32, 5, seeds=seeds, filter_kind=1, ts=ts, win=(700, 1900))
    assert np.array_equal(e2[0], o2[0]) and np.array_equal(e2[1].view(np.uint32), o2[1].view(np.uint32))
    # 3rd: the first again - nothing of the second call's tables may show
    _both(grab, d_data, d_graph, n, dim, deg, q1, 10, 64, 4, 45, 16, 16, 999)
    # a search whose visited set fits LDS needs no table from the array and still allocates nothing
    _both(grab, d_data, d_graph, n, dim, deg, q1, 10, 64, 4, 30, 12, 16, 7)
    q3 = datasets.gaussian(1200, dim, 4)
    _both(grab, d_data, d_graph, n, dim, deg, q3, 10, 64, 4, 30, 11, 16, 7)   # wave per query


def test_static_entry_point_rejects_what_it_cannot_hold(oracle, grab):
    n, dim, deg = 600, 32, 16
    data = datasets.gaussian(n, dim, 5)
    graph = oracle.optimize(oracle.knn_graph(data, 32), deg)
    d_data, d_graph = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(graph)
    nq = 129   # 129 << 16 slots > 8 Mi slots
    q = datasets.gaussian(nq, dim, 6)
    out = (grab.DeviceArray((nq, 10), np.int64), grab.DeviceArray((nq, 10), np.float32))
    with pytest.raises(RuntimeError, match="static array"):
        grab.search_ex(d_data, d_graph, n, dim, deg, grab.DeviceArray.from_numpy(q), nq, 10, 64, 4, 20, 16, 16, 1, d_out=out,
                       static_tables=True)
    with pytest.raises(RuntimeError, match="kernel_ms"):
        grab.search_ex(d_data, d_graph, n, dim, deg, grab.DeviceArray.from_numpy(q), 8, 10, 64, 4, 20, 16, 16, 1, d_out=out,
                       static_tables=True, want_ms=True)
    # exactly at the limit: 128 queries x 2^16
    exp = grab.search_ex(d_data, d_graph, n, dim, deg, grab.DeviceArray.from_numpy(q), 128, 10, 64, 4, 20, 16, 16, 1)
    grab.search_ex(d_data, d_graph, n, dim, deg, grab.DeviceArray.from_numpy(q), 128, 10, 64, 4, 20, 16, 16, 1, d_out=out,
                   static_tables=True)
    grab.synchronize()
    assert np.array_equal(out[0].numpy()[:128], exp[0])


def test_static_entry_point_leaves_device_memory_as_it_is(oracle, grab):
    # what the entry point is for: after the first call on a device (which looks the array's address up) a run of calls
    # - tables in the static array, tables in LDS, a wave per query - changes nothing about the device's free memory,
    # while the allocating entry point takes and returns its tables call by call
    n, dim, deg = 3000, 128, 32
    data = datasets.gaussian(n, dim, 1)
    graph = oracle.optimize(oracle.knn_graph(data, 64), deg)
    d_data, d_graph = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(graph)
    shapes = [(60, 16, 45), (7, 17, 40), (60, 12, 30), (1200, 11, 30)]   # (queries, hash_bitlen, iterations)
    bufs = []
    for nq, bitlen, iters in shapes:
        q = grab.DeviceArray.from_numpy(datasets.gaussian(nq, dim, 2 + nq))
        bufs.append((q, (grab.DeviceArray((nq, 10), np.int64), grab.DeviceArray((nq, 10), np.float32)), grab.DeviceArray((nq, 6), np.uint64)))

    def run(static):
        for (nq, bitlen, iters), (q, out, ctr) in zip(shapes, bufs):
            grab.search_ex(d_data, d_graph, n, dim, deg, q, nq, 10, 64, 4, iters, bitlen, 16, 999, d_out=out, static_tables=static,
                           d_counters=ctr)
    run(True)   # untimed first round: symbol address, kernel images
    grab.synchronize()
    free0, total = grab.device_memory()
    lowest = free0
    for _ in range(3):
        run(True)
        lowest = min(lowest, grab.device_memory()[0])   # the kernels may still be running: an allocation would show here
    grab.synchronize()
    assert lowest == free0 and grab.device_memory()[0] == free0, (free0, lowest)
    assert 0 < free0 <= total
