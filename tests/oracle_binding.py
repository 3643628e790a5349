"""ctypes binding of oracle/liboracle.so (the CPU restatement used as the checker).

Test infrastructure only: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py.
"""
import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(ROOT, "oracle", "liboracle.so")
REF_SMEM_PATH = os.path.join(ROOT, "oracle", "_ref", "libref_smem.so")

INVALID = 0xFFFFFFFF
WRAP_SEARCH, WRAP_SEARCH_OPT, WRAP_BUCKET, WRAP_RANGE = 0, 1, 2, 3
FILTER_NONE, FILTER_RANGE, FILTER_MASK, FILTER_ID_RANGE = 0, 1, 2, 3
METRIC_L2, METRIC_IP = 0, 1
FLAG_STRICT = 1
FLAG_FILTER_FIRST = 2

lib = C.CDLL(LIB_PATH)
lib.orc_next_power_of_2.restype = C.c_uint32
lib.orc_queue_capacity.restype = C.c_uint32
lib.orc_smem_bytes.restype = C.c_size_t
lib.orc_l2_canon.restype = C.c_float
lib.orc_ip_canon.restype = C.c_float
lib.orc_l2_natural.restype = C.c_float
lib.orc_l2_ref_warp.restype = C.c_float
lib.orc_splitmix64.restype = C.c_uint64
lib.orc_hash_insert.restype = C.c_int


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def f32(a):
    return np.ascontiguousarray(a, np.float32)


def u32(a):
    return np.ascontiguousarray(a, np.uint32)


def u64(a):
    return np.ascontiguousarray(a, np.uint64)


def ref_smem():
    """The reference's own smem_cal.cuh compiled in place (oracle/_ref), or None if not built."""
    if not os.path.exists(REF_SMEM_PATH):
        return None
    r = C.CDLL(REF_SMEM_PATH)
    r.ref_next_power_of_2.restype = C.c_uint32
    r.ref_calculate_and_check_smem.restype = C.c_size_t
    return r


def search_plan(wrapper, k, itopk_param, sw, degree, n_provided=0):
    it, ns, cap = C.c_uint32(), C.c_uint32(), C.c_uint32()
    lib.orc_search_plan(C.c_int(wrapper), C.c_uint32(k), C.c_uint32(itopk_param), C.c_uint32(sw),
                        C.c_uint32(degree), C.c_uint32(n_provided), C.byref(it), C.byref(ns), C.byref(cap))
    return it.value, ns.value, cap.value


def bitonic_network(keys, vals, lanes, per_lane, asc=True):
    keys, vals = f32(keys).copy(), u32(vals).copy()
    lib.orc_bitonic_network(_p(keys), _p(vals), C.c_uint32(lanes), C.c_uint32(per_lane), C.c_int(int(asc)))
    return keys, vals


def sort_pairs(keys, vals):
    keys, vals = f32(keys).copy(), u32(vals).copy()
    lib.orc_sort_pairs(_p(keys), _p(vals), C.c_size_t(keys.size))
    return keys, vals


def hash_insert_many(bitlen, keys):
    keys = u32(keys)
    table = np.full(1 << bitlen, INVALID, np.uint32)
    res = np.zeros(keys.size, np.uint32)
    lib.orc_hash_insert_many(_p(table), C.c_uint32(bitlen), _p(keys), C.c_size_t(keys.size), _p(res))
    return res, table


def l2(kind, a, b):
    a, b = f32(a), f32(b)
    fn = {"canon": lib.orc_l2_canon, "ip": lib.orc_ip_canon, "natural": lib.orc_l2_natural,
          "ref_warp": lib.orc_l2_ref_warp}[kind]
    return float(fn(_p(a), _p(b), C.c_uint32(a.size)))


def distance_many(q, data, ids, metric=METRIC_L2):
    q, data, ids = f32(q), f32(data), u32(ids)
    out = np.zeros(ids.size, np.float32)
    lib.orc_l2_canon_many(_p(q), _p(data), _p(ids), C.c_size_t(ids.size), C.c_uint32(data.shape[1]),
                          C.c_int(metric), _p(out))
    return out


def _filter_args(filter_kind, ts, win, win_start, win_end, labels, masks):
    per_query = 0
    ws = we = None
    if filter_kind in (FILTER_RANGE, FILTER_ID_RANGE):
        if win_start is not None:
            ws, we, per_query = u64(win_start), u64(win_end), 1
        else:
            ws, we = u64([win[0]]), u64([win[1]])
    return (None if ts is None else u64(ts)), ws, we, per_query, \
        (None if labels is None else np.ascontiguousarray(labels, np.uint8)), (None if masks is None else u64(masks))


def bruteforce_topk(data, queries, k, metric=METRIC_L2, filter_kind=FILTER_NONE, ts=None, win=None,
                    win_start=None, win_end=None, labels=None, masks=None, threads=0):
    data, queries = f32(data), f32(queries)
    nq = queries.shape[0]
    ts, ws, we, pq, labels, masks = _filter_args(filter_kind, ts, win, win_start, win_end, labels, masks)
    ids = np.zeros((nq, k), np.int64)
    dists = np.zeros((nq, k), np.float32)
    lib.orc_bruteforce_topk(_p(data), C.c_size_t(data.shape[0]), C.c_uint32(data.shape[1]), _p(queries),
                            C.c_size_t(nq), C.c_uint32(k), C.c_int(metric), C.c_int(filter_kind), _p(ts), _p(ws),
                            _p(we), C.c_int(pq), _p(labels), _p(masks), _p(ids), _p(dists), C.c_int(threads))
    return ids, dists


def knn_graph(data, k, metric=METRIC_L2, threads=0):
    data = f32(data)
    out = np.zeros((data.shape[0], k), np.uint32)
    lib.orc_knn_graph(_p(data), C.c_size_t(data.shape[0]), C.c_uint32(data.shape[1]), C.c_uint32(k),
                      C.c_int(metric), _p(out), C.c_int(threads))
    return out


def detour_counts(knn, threads=0):
    knn = u32(knn)
    out = np.zeros(knn.shape, np.uint8)
    lib.orc_detour_counts(_p(knn), C.c_size_t(knn.shape[0]), C.c_uint32(knn.shape[1]), _p(out), C.c_int(threads))
    return out


def prune(knn, out_degree, threads=0):
    knn = u32(knn)
    out = np.zeros((knn.shape[0], out_degree), np.uint32)
    lib.orc_prune(_p(knn), C.c_size_t(knn.shape[0]), C.c_uint32(knn.shape[1]), C.c_uint32(out_degree), _p(out),
                  C.c_int(threads))
    return out


def reverse_graph(graph):
    graph = u32(graph)
    rev = np.zeros(graph.shape, np.uint32)
    cnt = np.zeros(graph.shape[0], np.uint32)
    lib.orc_reverse_graph(_p(graph), C.c_size_t(graph.shape[0]), C.c_uint32(graph.shape[1]), _p(rev), _p(cnt))
    return rev, cnt


def merge_graphs(graph, rev, cnt, threads=0):
    graph = u32(graph).copy()
    rev, cnt = u32(rev), u32(cnt)
    lib.orc_merge_graphs(_p(graph), _p(rev), _p(cnt), C.c_size_t(graph.shape[0]), C.c_uint32(graph.shape[1]),
                         C.c_int(threads))
    return graph


def optimize(knn, out_degree, threads=0):
    knn = u32(knn)
    out = np.zeros((knn.shape[0], out_degree), np.uint32)
    lib.orc_optimize(_p(knn), C.c_size_t(knn.shape[0]), C.c_uint32(knn.shape[1]), C.c_uint32(out_degree), _p(out),
                     C.c_int(threads))
    return out


def search(data, graph, queries, k, itopk, sw, max_iter, bitlen, n_seeds, mask, active_degree=None,
           seeds=None, metric=METRIC_L2, filter_kind=FILTER_NONE, ts=None, win=None, win_start=None,
           win_end=None, labels=None, masks=None, flags=0, threads=0):
    """Returns (ids int64 [nq,k], dists f32 [nq,k], counters uint64 [nq,6])."""
    data, graph, queries = f32(data), u32(graph), f32(queries)
    n, dim = data.shape
    deg = graph.shape[1]
    nq = queries.shape[0]
    n_prov = 0
    if seeds is not None:
        seeds = u32(seeds)
        n_prov = seeds.shape[1]
    ts, ws, we, pq, labels, masks = _filter_args(filter_kind, ts, win, win_start, win_end, labels, masks)
    ids = np.zeros((nq, k), np.int64)
    dists = np.zeros((nq, k), np.float32)
    ctr = np.zeros((nq, 6), np.uint64)
    lib.orc_search(_p(data), C.c_size_t(n), C.c_uint32(dim), _p(graph), C.c_uint32(deg),
                   C.c_uint32(deg if active_degree is None else active_degree), _p(queries), C.c_size_t(nq),
                   C.c_uint32(k), C.c_uint32(itopk), C.c_uint32(sw), C.c_uint32(max_iter), C.c_uint32(bitlen),
                   C.c_uint32(n_seeds), _p(seeds), C.c_uint32(n_prov), C.c_uint64(mask), C.c_int(metric),
                   C.c_int(filter_kind), _p(ts), _p(ws), _p(we), C.c_int(pq), _p(labels), _p(masks),
                   C.c_uint32(flags & 3), _p(ids), _p(dists), _p(ctr), C.c_int(threads))
    return ids, dists, ctr


def sample_window_seeds(sorted_ts, ids_by_ts, n_seeds, seed, win=None, win_start=None, win_end=None):
    sorted_ts, ids_by_ts = u64(sorted_ts), u32(ids_by_ts)
    if win_start is not None:
        ws, we, pq = u64(win_start), u64(win_end), 1
        nq = ws.size
    else:
        ws, we, pq, nq = u64([win[0]]), u64([win[1]]), 0, 1
    out = np.zeros((nq, n_seeds), np.uint32)
    lib.orc_sample_window_seeds(_p(sorted_ts), _p(ids_by_ts), C.c_size_t(sorted_ts.size), _p(ws), _p(we),
                                C.c_size_t(nq), C.c_int(pq), C.c_uint32(n_seeds), C.c_uint64(seed), _p(out))
    return out


def remote_global_k(total_degree, local_degree):
    lib.orc_remote_global_k.restype = C.c_uint32
    return lib.orc_remote_global_k(C.c_uint32(total_degree), C.c_uint32(local_degree))


def remote_edges(cand, ts, graph, total_degree, local_degree):
    cand, ts, graph = u32(cand), u64(ts), u32(graph).copy()
    lib.orc_remote_edges(_p(cand), _p(ts), C.c_size_t(ts.size), C.c_uint32(cand.shape[1]), C.c_uint32(total_degree),
                         C.c_uint32(local_degree), _p(graph))
    return graph


def inject_reverse_remote(graph, total_degree, local_degree):
    graph = u32(graph).copy()
    lib.orc_inject_reverse_remote(_p(graph), C.c_size_t(graph.shape[0]), C.c_uint32(total_degree), C.c_uint32(local_degree))
    return graph


def build_time_partitioned(data, ts, bucket_sizes, total_degree, local_degree, metric=METRIC_L2, threads=0):
    data, ts = f32(data), u64(ts)
    n = data.shape[0]
    graph = np.zeros((n, total_degree), np.uint32)
    bs = (C.c_size_t * len(bucket_sizes))(*[int(b) for b in bucket_sizes])
    lib.orc_build_time_partitioned(_p(data), C.c_size_t(n), C.c_uint32(data.shape[1]), _p(ts), bs, C.c_size_t(len(bucket_sizes)),
                                   C.c_uint32(total_degree), C.c_uint32(local_degree), C.c_int(metric), _p(graph), C.c_int(threads))
    return graph


def kmeans(data, k, niter, seed, threads=0):
    data = f32(data)
    cent = np.zeros((k, data.shape[1]), np.float32)
    assign = np.zeros(data.shape[0], np.int64)
    lib.orc_kmeans(_p(data), C.c_size_t(data.shape[0]), C.c_uint32(data.shape[1]), C.c_uint32(k), C.c_uint32(niter),
                   C.c_uint64(seed), _p(cent), _p(assign), C.c_int(threads))
    return cent, assign


def splitmix64(state):
    s = C.c_uint64(state)
    v = lib.orc_splitmix64(C.byref(s))
    return v, s.value


def insert_batch(data, n_existing, n_new, graph, itopk, sw, max_iter, bitlen, rng_state, metric=METRIC_L2,
                 flags=0, striped_sort=0, threads=0):
    """graph: [n_existing+n_new, deg] (modified copy returned).  Returns (graph, new_rng_state)."""
    data = f32(data)
    graph = u32(graph).copy()
    s = C.c_uint64(rng_state)
    lib.orc_insert_batch(_p(data), C.c_uint32(data.shape[1]), C.c_size_t(n_existing), C.c_size_t(n_new), _p(graph),
                         C.c_uint32(graph.shape[1]), C.c_uint32(itopk), C.c_uint32(sw), C.c_uint32(max_iter),
                         C.c_uint32(bitlen), C.byref(s), C.c_int(metric), C.c_uint32(flags), C.c_int(striped_sort),
                         C.c_int(threads))
    return graph, s.value


def merge_batch_neighbours(new_data, n_existing, search_k, local_ids, local_dists, metric=METRIC_L2):
    """orc_merge_batch_neighbours: returns the merged [n_new, search_k] id lists."""
    new_data = f32(new_data)
    ids = np.ascontiguousarray(local_ids, np.int64).copy()
    d = f32(local_dists)
    lib.orc_merge_batch_neighbours(_p(new_data), C.c_size_t(new_data.shape[0]), C.c_uint32(new_data.shape[1]),
                                   C.c_size_t(n_existing), C.c_uint32(search_k), C.c_int(metric), _p(ids), _p(d))
    return ids


def insert_partitioned_update(graph, ts, local_ids, global_ids, n_existing, n_new, target_ts, local_degree):
    """orc_insert_partitioned_update on copies; returns the new graph."""
    graph = u32(graph).copy()
    ts = np.ascontiguousarray(ts, np.uint64)
    li = np.ascontiguousarray(local_ids, np.int64).copy()
    gi = np.ascontiguousarray(global_ids, np.int64).copy()
    lib.orc_insert_partitioned_update(_p(graph), _p(ts), _p(li), _p(gi), C.c_size_t(n_existing), C.c_size_t(n_new),
                                      C.c_uint64(target_ts), C.c_uint32(graph.shape[1]), C.c_uint32(local_degree),
                                      C.c_uint32(li.shape[1]))
    return graph


def insert_partitioned_batch(data, ts, n_existing, n_new, target_ts, graph, local_degree, seeds, itopk, sw, max_iter,
                             bitlen, rng_state, metric=METRIC_L2, flags=0, threads=0):
    """graph: [n_existing+n_new, total_degree] (modified copy returned).  Returns (graph, new_rng_state)."""
    data = f32(data)
    graph = u32(graph).copy()
    ts = np.ascontiguousarray(ts, np.uint64)
    seeds = u32(seeds)
    s = C.c_uint64(rng_state)
    lib.orc_insert_partitioned_batch(_p(data), C.c_uint32(data.shape[1]), _p(ts), C.c_size_t(n_existing), C.c_size_t(n_new),
                                     C.c_uint64(target_ts), _p(graph), C.c_uint32(graph.shape[1]), C.c_uint32(local_degree),
                                     _p(seeds), C.c_uint32(seeds.shape[1]), C.c_uint32(itopk), C.c_uint32(sw),
                                     C.c_uint32(max_iter), C.c_uint32(bitlen), C.byref(s), C.c_int(metric),
                                     C.c_uint32(flags & 3), C.c_int(threads))
    return graph, s.value
