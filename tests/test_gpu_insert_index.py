"""Insert, the index handle and the growable buffer on the GPU against the CPU restatement."""
import ctypes as C
import os

import numpy as np
import pytest

import datasets

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("flags,striped", [(0, 0), (1, 1), (0, 1)])
def test_insert_step_matches_oracle(oracle, grab, flags, striped):
    n0, n_new, deg = 2000, 150, 32
    data = datasets.gaussian(n0 + n_new, 128, 50)
    g0 = oracle.optimize(oracle.knn_graph(data[:n0], 64), deg)
    graph = np.full((n0 + n_new, deg), 0xFFFFFFFF, np.uint32)
    graph[:n0] = g0
    params = grab.SearchParams(128, 6, 0, 50, 12)
    exp, state = oracle.insert_batch(data, n0, n_new, graph, 128, 6, 50, 12, 777, flags=flags, striped_sort=striped)
    d_data = grab.DeviceArray.from_numpy(data)
    d_graph = grab.DeviceArray.from_numpy(graph)
    new_state = grab.insert(d_data, 128, n0, n_new, d_data.ptr + n0 * 128 * 4, d_graph, deg, params, 777, flags=flags,
                            striped_sort=striped)
    got = d_graph.numpy()
    assert new_state == state
    bad = np.nonzero((exp != got).any(axis=1))[0]
    assert bad.size == 0, f"{bad.size} rows differ, first {bad[0]}"
    # invariants: new rows hold old ids only, old rows stay full, new ids appear in old rows
    new_rows = got[n0:]
    assert ((new_rows < n0) | (new_rows == 0xFFFFFFFF)).all()
    assert (got[:n0] != 0xFFFFFFFF).all()
    assert (got[:n0] >= n0).any()


def test_insert_large_call_uses_global_sort(oracle, grab):
    # 150 rows * 64 results > 8192 requests: the multi-launch sort path
    n0, n_new, deg = 1500, 300, 32
    data = datasets.gaussian(n0 + n_new, 96, 51)
    graph = np.full((n0 + n_new, deg), 0xFFFFFFFF, np.uint32)
    graph[:n0] = oracle.optimize(oracle.knn_graph(data[:n0], 64), deg)
    exp, _ = oracle.insert_batch(data, n0, n_new, graph, 128, 6, 50, 12, 5)
    d_data, d_graph = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(graph)
    grab.insert(d_data, 96, n0, n_new, d_data.ptr + n0 * 96 * 4, d_graph, deg, grab.SearchParams(128, 6, 0, 50, 12), 5)
    assert np.array_equal(d_graph.numpy(), exp)


def _oracle_index_insert(oracle, data, n0, graph0, deg, seed_state, batches, flags=0):
    """CagraIndex::insert on the CPU: 64 rows per inner step (src/cagraIndex.cu:165-179)."""
    n = n0
    graph = graph0.copy()
    state = seed_state
    for b in batches:
        graph = np.vstack([graph, np.full((b, deg), 0xFFFFFFFF, np.uint32)])
        for off in range(0, b, 64):
            cur = min(64, b - off)
            sub, state = oracle.insert_batch(data[:n + off + cur], n + off, cur, graph[:n + off + cur], 128, 6, 50, 12,
                                             state, flags=flags, striped_sort=flags & 1)
            graph[:n + off + cur] = sub
        n += b
    return graph, state


def test_index_build_query_insert_matches_oracle(oracle, grab, tmp_path):
    n0, deg = 3000, 32
    data = datasets.mixture(n0 + 500, 128, 8, 10, 11)
    ts = np.arange(n0 + 500, dtype=np.uint64) // 100  # 100 rows per timestamp
    idx = grab.CagraIndex(128, deg, vmm_max_bytes=1 << 30)
    idx.set_seed(1234)
    idx.setQueryParams(64, 4, 0, 50, 13)
    idx.add(data[:n0], ts[:n0])
    assert idx.size() == n0
    idx.build()
    egraph = oracle.optimize(oracle.knn_graph(data[:n0], 128), deg)  # intermediate = max(128, 2*deg)
    assert np.array_equal(idx.get_graph(), egraph)
    assert np.array_equal(idx.get_data(), data[:n0])
    assert np.array_equal(idx.ids_by_timestamp(3), np.arange(300, 400, dtype=np.uint32))

    # query: the handle draws rand_xor_mask from splitmix64(seed), 32 bits
    q = datasets.mixture(100, 128, 8, 10, 12)
    state = 1234
    v, state = oracle.splitmix64(state)
    ids, dist = idx.query(q, 10)
    eids, edist, _ = oracle.search(data[:n0], egraph, q, 10, 64, 4, 50, 13, 16, v & 0xFFFFFFFF)
    assert np.array_equal(ids, eids) and np.array_equal(dist.view(np.uint32), edist.view(np.uint32))
    assert idx.last_kernel_ms() > 0

    # insert two user batches (one ragged), graph compared after each
    graph = egraph
    n = n0
    for b in (200, 300):
        idx.insert(data[n:n + b], ts[n:n + b])
        graph, state = _oracle_index_insert(oracle, data, n, graph, deg, state, [b])
        n += b
        assert idx.size() == n
        assert np.array_equal(idx.get_graph(), graph)
    # timestamps of inserted rows are recorded (the reference drops them)
    assert np.array_equal(idx.ids_by_timestamp(34), np.arange(3400, 3500, dtype=np.uint32))

    # recall gate of the reference's insert test (tests/test_cagra_insert.cu:284): > 90 %
    idx.setQueryParams(128, 6, 0, 50, 13)
    ids, _ = idx.query(q, 10)
    gt, _ = oracle.bruteforce_topk(data[:n], q, 10)
    assert datasets.recall(ids, gt) > 0.90

    # range query over bucket timestamps, bound errors == 0
    ids, dist = idx.query_range(q, 10, 0.1, 5, 12)
    valid = ids[ids >= 0]
    assert valid.size > 0 and ((ts[valid] >= 5) & (ts[valid] < 12)).all()
    gt, _ = oracle.bruteforce_topk(data[:n], q, 10, filter_kind=1, ts=ts[:n], win=(5, 12))
    assert datasets.recall(ids, gt) > 0.8
    # range_radius >= 0.99 means unfiltered (src/cagraIndex.cu:305,323)
    ids_u, _ = idx.query_range(q, 10, 1.0, 5, 12)
    assert (ts[ids_u[ids_u >= 0]] >= 12).any()
    # empty window
    ids_e, dist_e = idx.query_range(q, 10, 0.1, 1000, 2000)
    assert (ids_e == -1).all() and (dist_e == -1.0).all()

    # single bucket
    ids_b, _ = idx.query_local(q, 10, 7)
    vb = ids_b[ids_b >= 0]
    assert vb.size > 0

    # per-query windows (extension)
    ws = np.random.default_rng(1).integers(0, 25, 100).astype(np.uint64)
    we = ws + np.uint64(6)
    ids_w, _ = idx.query_range_batch(q, 10, ws, we)
    for i in range(100):
        v = ids_w[i][ids_w[i] >= 0]
        assert ((ts[v] >= ws[i]) & (ts[v] < we[i])).all()
    gt, _ = oracle.bruteforce_topk(data[:n], q, 10, filter_kind=1, ts=ts[:n], win_start=ws, win_end=we)
    assert datasets.recall(ids_w, gt) > 0.8

    # save / load round trip, byte layout of the reference (src/cagraIndex.cu:352-395)
    path = str(tmp_path / "index.bin")
    idx.save(path)
    raw = open(path, "rb").read()
    assert np.frombuffer(raw[:8], np.uint32).tolist() == [128, deg]
    assert int(np.frombuffer(raw[8:16], np.uint64)[0]) == n
    assert len(raw) == 16 + n * 128 * 4 + n * deg * 4
    assert np.array_equal(np.frombuffer(raw[16 + n * 512:], np.uint32).reshape(n, deg), graph)
    idx2 = grab.CagraIndex(128, deg, vmm_max_bytes=1 << 30)
    idx2.set_seed(99)
    idx2.setQueryParams(128, 6, 0, 50, 13)
    idx2.load(path)
    idx.set_seed(99)
    a = idx.query(q, 10)
    b = idx2.query(q, 10)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    with pytest.raises(grab.GrabError):
        idx2.load(str(tmp_path / "missing.bin"))
    idx.close()
    idx2.close()


def test_index_empty_and_errors(grab):
    idx = grab.CagraIndex(128, 32, vmm_max_bytes=1 << 28)
    q = np.zeros((3, 128), np.float32)
    ids, dist = idx.query(q, 5)  # empty index: silent return, outputs untouched (src/cagraIndex.cu:196)
    assert (ids == -7).all()
    idx.add(datasets.gaussian(100, 128, 1))
    with pytest.raises(grab.GrabError):  # rows added but no graph yet
        idx.query(q, 5)
    idx.close()
    with pytest.raises(grab.GrabError):
        grab.CagraIndex(130, 32)  # dim must be a multiple of 4


def test_index_insert_into_empty_builds(oracle, grab):
    data = datasets.gaussian(500, 128, 9)
    idx = grab.CagraIndex(128, 32, vmm_max_bytes=1 << 28)
    idx.insert(data)  # src/cagraIndex.cu:134-138
    assert np.array_equal(idx.get_graph(), oracle.optimize(oracle.knn_graph(data, 128), 32))
    idx.close()


def test_index_mask_filter_ip(oracle, grab):
    data = datasets.unit_rows(4000, 768, 20)
    labels = datasets.zipf_labels(4000, 64, 1.1, 21)
    q = datasets.unit_rows(50, 768, 22)
    masks = datasets.label_masks(50, 64, 23)
    idx = grab.CagraIndex(768, 64, vmm_max_bytes=1 << 30)
    idx.set_metric(grab.METRIC_IP)
    idx.setQueryParams(128, 4, 0, 50, 13)
    idx.add(data)
    idx.set_labels(labels)
    idx.build()
    ids, _ = idx.query_mask(q, 10, masks)
    for i in range(50):
        v = ids[i][ids[i] >= 0]
        assert all((int(masks[i]) >> int(labels[x])) & 1 for x in v)
    gt, _ = oracle.bruteforce_topk(data, q, 10, metric=1, filter_kind=2, labels=labels, masks=masks)
    assert datasets.recall(ids, gt) > 0.8
    idx.close()


def test_vmm_contract(grab):
    # src/vmm_allocator.cuh:23-118: stable pointer, bytes preserved, no shrink, capacity error
    b = grab.Vmm(64 << 20)
    assert b.size == 0 and b.capacity >= 64 << 20
    b.resize(1000)
    p0, s0 = b.ptr, b.size
    assert s0 >= 1000
    src = np.arange(250, dtype=np.uint32)
    grab.check(grab.lib.grab_copy_to_device(C.c_void_p(p0), src.ctypes.data_as(C.c_void_p), C.c_size_t(1000)))
    b.resize(10)  # no-op
    assert b.size == s0
    for grow in (s0 + 1, 3 * s0, 40 << 20):
        b.resize(grow)
        assert b.ptr == p0 and b.size >= grow
    out = np.zeros(250, np.uint32)
    grab.check(grab.lib.grab_copy_to_host(out.ctypes.data_as(C.c_void_p), C.c_void_p(p0), C.c_size_t(1000)))
    assert np.array_equal(out, src)
    # the tail that was mapped later is usable
    tail = np.full(1024, 7, np.uint32)
    grab.check(grab.lib.grab_copy_to_device(C.c_void_p(p0 + (40 << 20) - 4096), tail.ctypes.data_as(C.c_void_p), C.c_size_t(4096)))
    with pytest.raises(grab.GrabError) as e:
        b.resize(b.capacity + 1)
    assert e.value.code == 3 and "VMM OOM" in str(e.value)
    b.close()


def test_index_vmm_capacity_error(grab):
    idx = grab.CagraIndex(128, 32, vmm_max_bytes=1 << 22)  # 2 MiB for data: ~4000 rows
    idx.add(datasets.gaussian(6000, 128, 1))
    with pytest.raises(grab.GrabError) as e:
        idx.build()
    assert e.value.code == 3
    idx.close()


def test_window_seed_sampler_matches_oracle(oracle, grab):
    rng = np.random.default_rng(3)
    ts = np.sort(rng.integers(0, 500, 5000)).astype(np.uint64)
    order = rng.permutation(5000).astype(np.uint32)
    ws = rng.integers(0, 480, 64).astype(np.uint64)
    we = ws + rng.integers(0, 40, 64).astype(np.uint64)
    got = grab.sample_window_seeds(grab.DeviceArray.from_numpy(ts), grab.DeviceArray.from_numpy(order), 5000, 64, 32, 42,
                                   d_win_start=grab.DeviceArray.from_numpy(ws), d_win_end=grab.DeviceArray.from_numpy(we)).numpy()
    assert np.array_equal(got, oracle.sample_window_seeds(ts, order, 32, 42, win_start=ws, win_end=we))
    got1 = grab.sample_window_seeds(grab.DeviceArray.from_numpy(ts), grab.DeviceArray.from_numpy(order), 5000, 1, 16, 7,
                                    win=(100, 300)).numpy()
    assert np.array_equal(got1, oracle.sample_window_seeds(ts, order, 16, 7, win=(100, 300)))


@pytest.mark.parametrize("monotone", [True, False])
def test_index_range_search_with_entry_layer(oracle, grab, monotone):
    # 40 well-separated clusters: the graph is disconnected, random in-window seeds miss most queries' clusters,
    # seeds from the entry-point layer do not.  The handle must give what the stateless pieces give.
    n, nq, deg, S, ns = 6000, 150, 32, 2000, 16
    data = datasets.mixture(n + 400, 128, 40, 10, 11)
    q = datasets.mixture(nq, 128, 40, 10, 12)
    rng = np.random.default_rng(5)
    ts = np.arange(n + 400, dtype=np.uint64) // 4 if monotone else rng.integers(0, 1500, n + 400).astype(np.uint64)
    span = int(ts[:n].max()) + 1
    ws, we = datasets.windows(span, nq, 0.2, 6)
    idx = grab.CagraIndex(128, deg, vmm_max_bytes=1 << 30)
    idx.setQueryParams(64, 4, 0, 50, 12)
    idx.set_flags(grab.FLAG_FILTER_FIRST)
    idx.add(data[:n], ts[:n])
    idx.build()
    graph = idx.get_graph()
    gt, _ = oracle.bruteforce_topk(data[:n], q, 10, filter_kind=oracle.FILTER_RANGE, ts=ts[:n], win_start=ws, win_end=we)
    plain, _ = idx.query_range_batch(q, 10, ws, we)
    idx.set_entry_layer(S, ns)
    ids, dist = idx.query_range_batch(q, 10, ws, we)
    assert datasets.recall(ids, gt) > 0.97 > datasets.recall(plain, gt)
    # the same from the stateless entry points + the oracle's search on those seeds
    order = np.argsort(ts[:n], kind="stable").astype(np.uint32)
    layer = grab.EntryLayer(grab.DeviceArray.from_numpy(data[:n]), n, 128, S,
                            d_ids_by_ts=None if monotone else grab.DeviceArray.from_numpy(order),
                            d_ts=grab.DeviceArray.from_numpy(ts[:n]))
    seeds = layer.select(grab.DeviceArray.from_numpy(q), nq, ns, filter_kind=grab.FILTER_RANGE,
                         d_win_start=grab.DeviceArray.from_numpy(ws), d_win_end=grab.DeviceArray.from_numpy(we)).numpy()
    eids, edist, _ = oracle.search(data[:n], graph, q, 10, 64, 4, 50, 12, ns, 1, seeds=seeds, filter_kind=oracle.FILTER_RANGE,
                                   ts=ts[:n], win_start=ws, win_end=we, flags=oracle.FLAG_FILTER_FIRST)
    full = (seeds != 0xFFFFFFFF).all(axis=1)  # a missing seed is replaced by a random row: mask-dependent
    assert full.sum() > nq // 2
    assert np.array_equal(ids[full], eids[full]) and np.array_equal(dist[full].view(np.uint32), edist[full].view(np.uint32))
    for i in range(nq):
        v = ids[i][ids[i] >= 0]
        assert ((ts[v] >= ws[i]) & (ts[v] < we[i])).all()
    # the coarse level (k-means groups of the sample rows) finds seeds as good, with a fraction of the distances
    idx.set_entry_groups(50, 16, 32)
    gids, _ = idx.query_range_batch(q, 10, ws, we)
    assert datasets.recall(gids, gt) > 0.97
    for i in range(nq):
        v = gids[i][gids[i] >= 0]
        assert ((ts[v] >= ws[i]) & (ts[v] < we[i])).all()
    # single window for the whole batch, then rows are inserted: the layer follows
    one, _ = idx.query_range(q, 10, 0.5, int(ws[0]), int(we[0]))
    v = one[one >= 0]
    assert ((ts[v] >= ws[0]) & (ts[v] < we[0])).all()
    idx.insert(data[n:], ts[n:] if monotone else ts[n:])
    ids2, _ = idx.query_range_batch(q, 10, ws, we)
    gt2, _ = oracle.bruteforce_topk(data, q, 10, filter_kind=oracle.FILTER_RANGE, ts=ts, win_start=ws, win_end=we)
    assert datasets.recall(ids2, gt2) > 0.9
    idx.close()


def test_index_mcag_file_round_trip_and_layout(oracle, grab, tmp_path):
    # CagraIndexOpt's file: header, timestamps, timestamp -> ids map, data, graph (src/cagraIndexOpt.cu:725-789)
    import struct
    n, dim, deg = 1200, 64, 32
    data = datasets.gaussian(n, dim, 3)
    ts = (np.arange(n, dtype=np.uint64) // 50) * 7  # 24 buckets of 50 rows, keys 0,7,14,...
    idx = grab.CagraIndex(dim, deg, vmm_max_bytes=1 << 28, local_degree=16)
    idx.add(data, ts)
    idx.build()
    graph = idx.get_graph().copy()
    path = str(tmp_path / "opt.mcag")
    idx.save_mcag(path)
    raw = open(path, "rb").read()
    assert raw[:4] == b"MCAG" and struct.unpack_from("<IIIQQ", raw, 4) == (1, dim, deg, 16, n)
    off = 4 + 4 + 4 + 4 + 8 + 8
    assert struct.unpack_from("<Q", raw, off)[0] == n
    assert np.array_equal(np.frombuffer(raw, np.uint64, n, off + 8), ts)
    off += 8 + 8 * n
    assert struct.unpack_from("<Q", raw, off)[0] == 24
    off += 8
    for b in range(24):
        key, cnt = struct.unpack_from("<QQ", raw, off)
        assert key == 7 * b and cnt == 50
        assert np.array_equal(np.frombuffer(raw, np.uint32, 50, off + 16), np.arange(50 * b, 50 * b + 50, dtype=np.uint32))
        off += 16 + 200
    assert struct.unpack_from("<Q", raw, off)[0] == n * dim
    assert np.array_equal(np.frombuffer(raw, np.float32, n * dim, off + 8).reshape(n, dim), data)
    off += 8 + 4 * n * dim
    assert struct.unpack_from("<Q", raw, off)[0] == n * deg
    assert np.array_equal(np.frombuffer(raw, np.uint32, n * deg, off + 8).reshape(n, deg), graph)
    assert off + 8 + 4 * n * deg == len(raw)

    other = grab.CagraIndex(dim, deg, vmm_max_bytes=1 << 28)
    other.load_mcag(path)
    assert other.size() == n and np.array_equal(other.get_graph(), graph) and np.array_equal(other.get_data(), data)
    assert np.array_equal(other.ids_by_timestamp(14), np.arange(100, 150, dtype=np.uint32))
    q = datasets.gaussian(40, dim, 4)
    idx.set_seed(5)
    other.set_seed(5)
    a, _ = idx.query_range(q, 10, 0.5, 35, 99)
    b, _ = other.query_range(q, 10, 0.5, 35, 99)
    assert np.array_equal(a, b)
    # seeds by time: inclusive upper bound, ids inside the range, at most `num`
    s = other.sample_seeds_by_time(7, 21, 64)
    assert s.size == 64 and ((s >= 50) & (s < 200)).all() and np.unique(s).size == 64
    assert other.sample_seeds_by_time(1, 6, 8).size == 0
    with open(path, "r+b") as f:
        f.write(b"XCAG")
    with pytest.raises(grab.GrabError, match="Magic"):
        other.load_mcag(path)
    idx.close()
    other.close()


def test_index_timestamp_filter_reads_neighbour_rows_and_follows_graph_changes(oracle, grab):
    # timestamps in no order: the traversal has to read them.  A large batch with a short queue and the filter
    # ahead of the visited set reads them from rows laid out like the graph; those rows must follow every change
    # of the graph (a stale row would let rows outside the window through, or drop rows inside it).
    n, extra, nq, deg, k = 8000, 500, 1500, 32, 10
    data = datasets.mixture(n + extra, 128, 30, 10, 31)
    q = datasets.mixture(nq, 128, 30, 10, 32)
    rng = np.random.default_rng(9)
    ts = rng.integers(0, 4000, n + extra).astype(np.uint64)
    ws, we = datasets.windows(4000, nq, 0.3, 4)
    idx = grab.CagraIndex(128, deg, vmm_max_bytes=1 << 30)
    idx.setQueryParams(64, 4, 0, 50, 12)
    idx.set_flags(grab.FLAG_FILTER_FIRST)
    idx.set_entry_layer(2000, 16)
    idx.add(data[:n], ts[:n])
    idx.build()

    def check(rows, limit):
        ids, dist = idx.query_range_batch(q, k, ws, we)
        gt, _ = oracle.bruteforce_topk(data[:rows], q, k, filter_kind=oracle.FILTER_RANGE, ts=ts[:rows], win_start=ws, win_end=we)
        v = ids >= 0
        assert ((ts[np.where(v, ids, 0)] >= ws[:, None]) & (ts[np.where(v, ids, 0)] < we[:, None]))[v].all()
        rec = datasets.recall(ids, gt)
        assert rec > limit, rec
        return ids, dist

    first, fdist = check(n, 0.97)
    # the same through the stateless search without the rows: identical answers
    idx.set_flags(grab.FLAG_FILTER_FIRST | grab.FLAG_BLOCK_PER_QUERY)
    plain, pdist = idx.query_range_batch(q, k, ws, we)
    idx.set_flags(grab.FLAG_FILTER_FIRST)
    same = (first == plain).all(axis=1)
    assert same.mean() > 0.99  # seeds that a window cannot supply are replaced by random rows, a draw per call
    idx.insert(data[n:], ts[n:])       # new rows, and old rows' slots rewritten
    check(n + extra, 0.9)
    idx.build()                        # a different graph over the same number of rows
    check(n + extra, 0.97)
    idx.close()


def test_chunked_range_batch_equals_the_undivided_call(oracle, grab):
    # A large batch with a window per query is cut into chunks that overlap on streams of the handle, its rows staged
    # through page-locked memory by two threads.  Same rows, same windows, same rand_xor_mask: same answers as the
    # undivided call, for scored and for listed seeds, odd k, chunks that do not divide the batch, and call after call.
    n, dim, deg = 20000, 128, 32
    data = datasets.mixture(n, dim, 40, 10, 11)
    ts = np.arange(n, dtype=np.uint64) // 3          # never decreasing, with repeats
    idx = grab.CagraIndex(dim, deg, vmm_max_bytes=1 << 30)
    idx.setQueryParams(64, 4, 0, 50, 12)   # 4096 slots: more than the 2100 rows a window holds at most, so no visited set fills up
    idx.set_flags(grab.FLAG_FILTER_FIRST)
    idx.set_entry_layer(2000, 16)
    idx.set_entry_groups(64, 8, 16)
    idx.add(data, ts)
    idx.build()
    rng = np.random.default_rng(3)
    # the first range search makes the entry layer, whose grouping draws from the handle's generator: out of the way first
    idx.query_range_batch(data[:4], 1, np.zeros(4, np.uint64), np.full(4, 100, np.uint64))
    for nq, k, chunk, listed in ((3001, 10, 1000, 0), (3001, 7, 700, 32), (2049, 5, 256, 32), (4000, 10, 3999, 0), (2600, 1, 1300, 16)):
        q = datasets.mixture(nq, dim, 40, 10, 100 + nq)
        ws = rng.integers(0, n // 3 - 700, nq).astype(np.uint64)
        we = ws + rng.integers(1, 700, nq).astype(np.uint64)
        idx.set_entry_list(listed)
        idx.set_batch_chunk(0)
        idx.set_seed(9)
        one_i, one_d = idx.query_range_batch(q, k, ws, we)
        idx.set_batch_chunk(chunk)
        for rep in range(2):
            idx.set_seed(9)
            ids, dist = idx.query_range_batch(q, k, ws, we)
            assert np.array_equal(ids, one_i), f"nq {nq} k {k} chunk {chunk} listed {listed} call {rep}: ids differ"
            assert np.array_equal(dist.view(np.uint32), one_d.view(np.uint32))
        v = ids >= 0
        assert v.any() and ((ts[ids[v]] >= np.repeat(ws, k).reshape(nq, k)[v]) & (ts[ids[v]] < np.repeat(we, k).reshape(nq, k)[v])).all()
    idx.close()


def test_failed_inserts_leave_the_index_as_it_was(oracle, grab):
    # An insert that fails on the way (forced from the host before a chosen inner step; every kernel that was queued
    # still runs to its end) must leave what searches see as it was: row count, timestamp map, host rows, the
    # generator that draws rand_xor_mask, the query parameters.  Both kinds of insert; failing before the first inner
    # step (nothing of the graph touched: the same answers as before) and after it (old rows may hold edges to the
    # failed batch's ids, which searches skip).
    n0, dim, deg = 2500, 64, 32
    data = datasets.mixture(n0 + 400, dim, 10, 10, 11)
    ts = np.repeat(np.arange(5, dtype=np.uint64), n0 // 5)
    q = datasets.mixture(60, dim, 10, 10, 12)
    for partitioned in (False, True):
        idx = grab.CagraIndex(dim, deg, vmm_max_bytes=1 << 28, local_degree=24 if partitioned else 0)
        idx.set_seed(3)
        idx.setQueryParams(64, 4, 0, 40, 12)
        idx.add(data[:n0], ts)
        idx.build_partitioned() if partitioned else idx.build()
        new_ts = np.full(200, 3 if partitioned else 9, np.uint64)
        for step in (0, 1):
            graph_before = idx.get_graph()
            state, params = idx.rng_state(), idx.query_params()
            in_bucket = idx.ids_by_timestamp(int(new_ts[0]))
            idx.set_seed(state)
            before = idx.query(q, 10)
            idx.set_seed(state)
            idx.debug_fail_insert(step)
            with pytest.raises(RuntimeError, match="injected"):
                (idx.insert_partitioned if partitioned else idx.insert)(data[n0:n0 + 200], new_ts)
            assert idx.size() == n0 and idx.rng_state() == state and idx.query_params() == params
            assert np.array_equal(idx.ids_by_timestamp(int(new_ts[0])), in_bucket)
            assert np.array_equal(idx.get_data(), data[:n0])
            after = idx.query(q, 10)
            assert after[0].max() < n0 and (np.diff(after[1], axis=1) >= 0).all()
            g = idx.get_graph()
            assert g.shape == graph_before.shape
            if step == 0:
                assert np.array_equal(g, graph_before)
                assert np.array_equal(after[0], before[0]) and np.array_equal(after[1].view(np.uint32), before[1].view(np.uint32))
            else:
                assert (g[g != 0xFFFFFFFF] >= n0).any()      # the step that ran left reverse edges behind
        # the index still takes rows, and finds them
        (idx.insert_partitioned if partitioned else idx.insert)(data[n0:n0 + 200], new_ts)
        assert idx.size() == n0 + 200
        ids, _ = idx.query(data[n0:n0 + 50], 1)
        assert (ids[:, 0] == np.arange(n0, n0 + 50)).mean() > 0.9
        idx.close()
