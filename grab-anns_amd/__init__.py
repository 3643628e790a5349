"""ctypes binding of libgrab_anns.so, the C ABI declared in include/grab_anns.h.

This module only loads what `make -C grab-anns_amd` (or __graft_entry__.build()) has built
and forwards calls; there is no CPU fallback.  If the shared library is missing the import
fails, and compute calls fail on a machine without a GPU.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgrab_anns.so")

OK = 0
INVALID_ID = 0xFFFFFFFF
METRIC_L2, METRIC_IP = 0, 1
FILTER_NONE, FILTER_RANGE, FILTER_MASK, FILTER_ID_RANGE = 0, 1, 2, 3
WRAP_SEARCH, WRAP_SEARCH_OPT, WRAP_BUCKET, WRAP_RANGE = 0, 1, 2, 3
FLAG_STRICT_REFERENCE = 1
FLAG_FILTER_FIRST = 2
FLAG_WAVE_PER_QUERY = 4
FLAG_BLOCK_PER_QUERY = 8


class GrabError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"grab_anns error {code}: {msg}")
        self.code = code


class SearchParams(C.Structure):
    _fields_ = [("itopk_size", C.c_uint32), ("search_width", C.c_uint32), ("min_iterations", C.c_uint32),
                ("max_iterations", C.c_uint32), ("hash_bitlen", C.c_uint32)]


class BuildParams(C.Structure):
    _fields_ = [("intermediate_degree", C.c_uint32), ("graph_degree", C.c_uint32)]


class Counters(C.Structure):
    _fields_ = [("iterations", C.c_uint64), ("seed_dists", C.c_uint64), ("parents", C.c_uint64),
                ("filter_reads", C.c_uint64), ("child_dists", C.c_uint64), ("hash_full", C.c_uint64)]


COUNTER_FIELDS = [f[0] for f in Counters._fields_]


class SearchDesc(C.Structure):
    _fields_ = [
        ("d_dataset", C.c_void_p), ("d_graph", C.c_void_p), ("num_dataset", C.c_size_t), ("dim", C.c_uint32),
        ("graph_degree", C.c_uint32), ("active_degree", C.c_uint32), ("metric", C.c_int),
        ("d_queries", C.c_void_p), ("num_queries", C.c_size_t), ("k", C.c_uint32),
        ("itopk", C.c_uint32), ("search_width", C.c_uint32), ("max_iterations", C.c_uint32),
        ("hash_bitlen", C.c_uint32), ("n_seeds", C.c_uint32), ("d_seeds", C.c_void_p),
        ("n_provided", C.c_uint32), ("rand_xor_mask", C.c_uint64),
        ("filter_kind", C.c_int), ("d_ts", C.c_void_p), ("d_win_start", C.c_void_p), ("d_win_end", C.c_void_p),
        ("win_start", C.c_uint64), ("win_end", C.c_uint64), ("per_query_window", C.c_int),
        ("d_labels", C.c_void_p), ("d_masks", C.c_void_p), ("flags", C.c_uint32),
        ("d_out_indices", C.c_void_p), ("d_out_dists", C.c_void_p), ("d_counters", C.c_void_p),
        ("kernel_ms", C.POINTER(C.c_float)), ("stream", C.c_void_p), ("d_graph_ts", C.c_void_p),
        ("entry_layer", C.c_void_p), ("d_entry_groups", C.c_void_p), ("entry_nprobe", C.c_uint32),
        ("entry_min_rows", C.c_uint32), ("d_rank", C.c_void_p), ("d_graph_rank", C.c_void_p),
    ]


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is not built; run `make -C {_HERE}` (needs hipcc)")
    lib = C.CDLL(LIB_PATH)
    restypes = {
        "grab_last_error": C.c_char_p, "grab_reference_smem_bytes": C.c_size_t, "grab_search_lds_bytes": C.c_size_t,
        "grab_vmm_data": C.c_void_p, "grab_vmm_size": C.c_size_t, "grab_vmm_capacity": C.c_size_t,
        "grab_index_size": C.c_size_t, "grab_index_get_data": C.c_void_p, "grab_index_get_graph": C.c_void_p,
        "grab_index_ids_by_timestamp": C.c_size_t, "grab_index_last_kernel_ms": C.c_float,
    }
    for name in ("grab_vmm_destroy", "grab_index_destroy", "grab_search_plan"):
        restypes[name] = None
    for name, rt in restypes.items():
        getattr(lib, name).restype = rt  # AttributeError here = the library is stale or incomplete
    lib.grab_search_ex.argtypes = [C.POINTER(SearchDesc)]
    return lib


lib = _load()


def check(rc):
    if rc != OK:
        raise GrabError(rc, lib.grab_last_error().decode(errors="replace"))


def device_count():
    return lib.grab_device_count()


def _np_ptr(a):
    return a.ctypes.data_as(C.c_void_p)


class DeviceArray:
    """A device allocation with a numpy dtype/shape, made through the C ABI's memory helpers."""

    def __init__(self, shape, dtype):
        self.shape = tuple(np.atleast_1d(shape).tolist()) if not isinstance(shape, tuple) else shape
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = C.c_void_p()
        check(lib.grab_device_malloc(C.byref(p), C.c_size_t(self.nbytes)))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype)
        if d.nbytes:
            check(lib.grab_copy_to_device(C.c_void_p(d.ptr), _np_ptr(a), C.c_size_t(d.nbytes)))
        return d

    def numpy(self):
        out = np.empty(self.shape, self.dtype)
        if self.nbytes:
            check(lib.grab_copy_to_host(_np_ptr(out), C.c_void_p(self.ptr), C.c_size_t(self.nbytes)))
        return out

    def fill_bytes(self, value):
        check(lib.grab_device_memset(C.c_void_p(self.ptr), C.c_int(value), C.c_size_t(self.nbytes)))

    def free(self):
        if self.ptr:
            lib.grab_device_free(C.c_void_p(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def synchronize():
    check(lib.grab_device_synchronize())


class Stream:
    """A HIP stream of default priority (grab_stream_*), for stream-ordered calls."""

    def __init__(self):
        self.ptr = C.c_void_p()
        check(lib.grab_stream_create(C.byref(self.ptr)))

    def synchronize(self):
        check(lib.grab_stream_synchronize(self.ptr))

    def wait(self, other):
        """Work queued here from now on starts after everything queued on `other` so far."""
        check(lib.grab_stream_wait(self.ptr, other.ptr))

    def close(self):
        if self.ptr:
            check(lib.grab_stream_destroy(self.ptr))
            self.ptr = None


def search_plan(wrapper, k, itopk_param, search_width, degree, n_provided=0):
    it, ns, cap = C.c_uint32(), C.c_uint32(), C.c_uint32()
    lib.grab_search_plan(C.c_int(wrapper), C.c_uint32(k), C.c_uint32(itopk_param), C.c_uint32(search_width),
                         C.c_uint32(degree), C.c_uint32(n_provided), C.byref(it), C.byref(ns), C.byref(cap))
    return it.value, ns.value, cap.value


def _ptr(x):
    if x is None:
        return None
    if isinstance(x, DeviceArray):
        return x.ptr
    return int(x)


def search_ex(d_dataset, d_graph, n, dim, degree, d_queries, nq, k, itopk, search_width, max_iterations,
              hash_bitlen, n_seeds, rand_xor_mask, active_degree=None, metric=METRIC_L2, d_seeds=None,
              n_provided=0, filter_kind=FILTER_NONE, d_ts=None, win=None, d_win_start=None, d_win_end=None,
              d_labels=None, d_masks=None, flags=0, want_counters=False, want_ms=False, d_graph_ts=None, stream=None,
              d_out=None, static_tables=False, d_counters=None, entry=None, d_rank=None, d_graph_rank=None):
    """General search (grab_search_ex).  `entry` = (EntryLayer, d_groups, nprobe, min_rows): the kernel lists its own seeds.  Returns (ids int64 [nq,k], dists f32 [nq,k], counters|None, ms|None).
    With `d_out` = (DeviceArray int64 [nq,k], DeviceArray f32 [nq,k]) the search is only queued on `stream`
    (grab_search_ex_async; grab_search_ex_static with `static_tables`, which allocates nothing) and nothing is
    returned: the caller reads the arrays (and `d_counters`, a DeviceArray uint64 [nq,6]) after synchronising."""
    out_i = d_out[0] if d_out is not None else DeviceArray((nq, k), np.int64)
    out_d = d_out[1] if d_out is not None else DeviceArray((nq, k), np.float32)
    ctr = d_counters if d_counters is not None else DeviceArray((nq, 6), np.uint64) if want_counters else None
    ms = C.c_float(0.0)
    d = SearchDesc()
    d.d_dataset, d.d_graph, d.num_dataset, d.dim = _ptr(d_dataset), _ptr(d_graph), n, dim
    d.graph_degree = degree
    d.active_degree = degree if active_degree is None else active_degree
    d.metric = metric
    d.d_queries, d.num_queries, d.k = _ptr(d_queries), nq, k
    d.itopk, d.search_width, d.max_iterations, d.hash_bitlen = itopk, search_width, max_iterations, hash_bitlen
    d.n_seeds, d.d_seeds, d.n_provided, d.rand_xor_mask = n_seeds, _ptr(d_seeds), n_provided, rand_xor_mask
    d.filter_kind, d.d_ts, d.d_graph_ts = filter_kind, _ptr(d_ts), _ptr(d_graph_ts)
    if d_win_start is not None:
        d.d_win_start, d.d_win_end, d.per_query_window = _ptr(d_win_start), _ptr(d_win_end), 1
    elif win is not None:
        d.win_start, d.win_end = int(win[0]), int(win[1])
    d.d_labels, d.d_masks, d.flags = _ptr(d_labels), _ptr(d_masks), flags
    d.d_out_indices, d.d_out_dists = out_i.ptr, out_d.ptr
    d.d_counters = ctr.ptr if ctr is not None else None
    d.kernel_ms = C.pointer(ms) if want_ms else None
    d.stream = stream.ptr if stream is not None else None
    if entry is not None:
        d.entry_layer, d.d_entry_groups, d.entry_nprobe, d.entry_min_rows = entry[0].h, _ptr(entry[1]), entry[2], entry[3]
    d.d_rank, d.d_graph_rank = _ptr(d_rank), _ptr(d_graph_rank)
    if d_out is not None:
        check((lib.grab_search_ex_static if static_tables else lib.grab_search_ex_async)(C.byref(d)))
        return None
    check(lib.grab_search_ex(C.byref(d)))
    return out_i.numpy(), out_d.numpy(), (ctr.numpy() if ctr is not None else None), (ms.value if want_ms else None)


def neighbor_ranks(d_graph, d_rank, n, degree):
    """grab_neighbor_ranks: [n, degree] uint32, the place in timestamp order of every neighbour."""
    out = DeviceArray((n, degree), np.uint32)
    check(lib.grab_neighbor_ranks(C.c_void_p(_ptr(d_graph)), C.c_void_p(_ptr(d_rank)), C.c_size_t(n), C.c_uint32(degree),
                                  C.c_void_p(out.ptr), None))
    synchronize()
    return out


def neighbor_timestamps(d_graph, d_ts, n, degree):
    """grab_neighbor_timestamps: [n, degree] uint64, the timestamp of every neighbour."""
    out = DeviceArray((n, degree), np.uint64)
    check(lib.grab_neighbor_timestamps(C.c_void_p(_ptr(d_graph)), C.c_void_p(_ptr(d_ts)), C.c_size_t(n), C.c_uint32(degree),
                                       C.c_void_p(out.ptr), None))
    synchronize()
    return out


def sort_pairs(keys, vals):
    keys = np.ascontiguousarray(keys, np.float32).copy()
    vals = np.ascontiguousarray(vals, np.uint32).copy()
    check(lib.grab_sort_pairs(_np_ptr(keys), _np_ptr(vals), C.c_size_t(keys.size)))
    return keys, vals


def hash_insert_many(bitlen, keys):
    keys = np.ascontiguousarray(keys, np.uint32)
    res = np.zeros(keys.size, np.uint32)
    table = np.zeros(1 << bitlen, np.uint32)
    check(lib.grab_hash_insert_many(C.c_uint32(bitlen), _np_ptr(keys), C.c_size_t(keys.size), _np_ptr(res),
                                    _np_ptr(table)))
    return res, table


def distance_many(query, data, ids, metric=METRIC_L2):
    query = np.ascontiguousarray(query, np.float32)
    data = np.ascontiguousarray(data, np.float32)
    ids = np.ascontiguousarray(ids, np.uint32)
    out = np.zeros(ids.size, np.float32)
    check(lib.grab_distance_many(_np_ptr(query), _np_ptr(data), C.c_size_t(data.shape[0]), C.c_uint32(data.shape[1]),
                                 _np_ptr(ids), C.c_size_t(ids.size), C.c_int(metric), _np_ptr(out)))
    return out


def _stream(stream):
    return C.c_void_p(stream) if stream else None


def generate_knn_graph(d_dataset, n, dim, k, metric=METRIC_L2, want_ms=False):
    """grab_generate_knn_graph: returns (DeviceArray uint32 [n,k], ms|None)."""
    out = DeviceArray((n, k), np.uint32)
    ms = C.c_float(0.0)
    check(lib.grab_generate_knn_graph(C.c_void_p(_ptr(d_dataset)), C.c_size_t(n), C.c_uint32(dim), C.c_uint32(k),
                                      C.c_int(metric), C.c_void_p(out.ptr), C.pointer(ms) if want_ms else None, None))
    return out, (ms.value if want_ms else None)


def last_knn_stats():
    """grab_last_knn_stats: (floating-point operations of the matrix passes, rows redone by the plain pass)."""
    flop, redone = C.c_double(0.0), C.c_uint64(0)
    check(lib.grab_last_knn_stats(C.byref(flop), C.byref(redone)))
    return flop.value, redone.value


def last_knn_bf16_flop():
    """grab_last_knn_bf16_flop: bf16 matrix operations of the last kNN graph (0 where it ran on fp32 instructions)."""
    lib.grab_last_knn_bf16_flop.restype = C.c_double
    return float(lib.grab_last_knn_bf16_flop())


def knn_allow_bf16(allow):
    """grab_knn_allow_bf16: may kNN graphs form their candidates on bf16 instructions (default yes); returns the previous setting."""
    return bool(lib.grab_knn_allow_bf16(1 if allow else 0))


def last_knn_exact_rows():
    """grab_last_knn_exact_rows: rows of the last kNN graph / exact top-k that were redone against every column."""
    lib.grab_last_knn_exact_rows.restype = C.c_uint64
    return int(lib.grab_last_knn_exact_rows())


def bruteforce_topk(d_dataset, n, dim, d_queries, nq, k, metric=METRIC_L2, filter_kind=FILTER_NONE, d_ts=None,
                    win=None, d_win_start=None, d_win_end=None, d_labels=None, d_masks=None, want_ms=False):
    """grab_bruteforce_topk: exact filtered top-k.  Returns (ids int64 [nq,k], dists f32 [nq,k], ms|None)."""
    out_i = DeviceArray((nq, k), np.int64)
    out_d = DeviceArray((nq, k), np.float32)
    ms = C.c_float(0.0)
    ws, we = (int(win[0]), int(win[1])) if win is not None else (0, 0)
    check(lib.grab_bruteforce_topk(C.c_void_p(_ptr(d_dataset)), C.c_size_t(n), C.c_uint32(dim), C.c_void_p(_ptr(d_queries)),
                                   C.c_size_t(nq), C.c_uint32(k), C.c_int(metric), C.c_int(filter_kind),
                                   C.c_void_p(_ptr(d_ts)), C.c_void_p(_ptr(d_win_start)), C.c_void_p(_ptr(d_win_end)),
                                   C.c_uint64(ws), C.c_uint64(we), C.c_int(1 if d_win_start is not None else 0),
                                   C.c_void_p(_ptr(d_labels)), C.c_void_p(_ptr(d_masks)), C.c_void_p(out_i.ptr),
                                   C.c_void_p(out_d.ptr), C.pointer(ms) if want_ms else None, None))
    return out_i.numpy(), out_d.numpy(), (ms.value if want_ms else None)


def device_memory():
    """(free, total) bytes of the current device's memory."""
    f, t = C.c_size_t(), C.c_size_t()
    check(lib.grab_device_memory(C.byref(f), C.byref(t)))
    return f.value, t.value


def bucket_scan_topk(d_dataset, n, dim, bucket_offsets, d_queries, nq, k, masks, metric=METRIC_L2, want_ms=False,
                     d_out=None):
    """grab_bucket_scan_topk: exact top-k over the buckets each query's mask admits (rows stored bucket by bucket).
    Returns (ids int64 [nq,k], dists f32 [nq,k], ms|None); with d_out = (ids, dists) device arrays nothing is fetched."""
    off = np.ascontiguousarray(bucket_offsets, np.uint64)
    m = np.ascontiguousarray(masks, np.uint64)
    out_i, out_d = d_out if d_out is not None else (DeviceArray((nq, k), np.int64), DeviceArray((nq, k), np.float32))
    ms = C.c_float(0.0)
    check(lib.grab_bucket_scan_topk(C.c_void_p(_ptr(d_dataset)), C.c_size_t(n), C.c_uint32(dim), _np_ptr(off),
                                    C.c_uint32(off.size - 1), C.c_void_p(_ptr(d_queries)), C.c_size_t(nq), C.c_uint32(k),
                                    C.c_int(metric), _np_ptr(m), C.c_void_p(out_i.ptr), C.c_void_p(out_d.ptr),
                                    C.pointer(ms) if want_ms else None, None))
    if d_out is not None:
        return None, None, (ms.value if want_ms else None)
    return out_i.numpy(), out_d.numpy(), (ms.value if want_ms else None)


def window_scan_topk(d_dataset, n, dim, d_queries, nq, k, id_lo, id_hi, metric=METRIC_L2, want_ms=False, d_out=None):
    """grab_window_scan_topk: exact top-k of each query among the rows [id_lo[q], id_hi[q]) (host arrays).
    Returns (ids int64 [nq,k], dists f32 [nq,k], ms|None); with d_out = (ids, dists) device arrays nothing is fetched."""
    lo = np.ascontiguousarray(id_lo, np.uint64)
    hi = np.ascontiguousarray(id_hi, np.uint64)
    out_i, out_d = d_out if d_out is not None else (DeviceArray((nq, k), np.int64), DeviceArray((nq, k), np.float32))
    ms = C.c_float(0.0)
    check(lib.grab_window_scan_topk(C.c_void_p(_ptr(d_dataset)), C.c_size_t(n), C.c_uint32(dim), C.c_void_p(_ptr(d_queries)),
                                    C.c_size_t(nq), C.c_uint32(k), C.c_int(metric), _np_ptr(lo), _np_ptr(hi),
                                    C.c_void_p(out_i.ptr), C.c_void_p(out_d.ptr), C.pointer(ms) if want_ms else None, None))
    if d_out is not None:
        return None, None, (ms.value if want_ms else None)
    return out_i.numpy(), out_d.numpy(), (ms.value if want_ms else None)


class ScanBase:
    """grab_scan_base: a base prepared for window_topk / bucket_topk (rows split once, scratch kept between calls)."""

    def __init__(self, d_dataset, n, dim, metric=METRIC_L2):
        self.h = C.c_void_p()
        self.n, self.dim = n, dim
        self._keep = d_dataset
        lib.grab_scan_base_destroy.restype = None
        check(lib.grab_scan_base_create(C.c_void_p(_ptr(d_dataset)), C.c_size_t(n), C.c_uint32(dim), C.c_int(metric), C.byref(self.h)))

    def _run(self, call, nq, k, want_ms, d_out):
        out_i, out_d = d_out if d_out is not None else (DeviceArray((nq, k), np.int64), DeviceArray((nq, k), np.float32))
        ms = C.c_float(0.0)
        check(call(C.c_void_p(out_i.ptr), C.c_void_p(out_d.ptr), C.pointer(ms) if want_ms else None, None))
        if d_out is not None:
            return None, None, (ms.value if want_ms else None)
        return out_i.numpy(), out_d.numpy(), (ms.value if want_ms else None)

    def window_topk(self, d_queries, nq, k, id_lo, id_hi, want_ms=False, d_out=None):
        lo, hi = np.ascontiguousarray(id_lo, np.uint64), np.ascontiguousarray(id_hi, np.uint64)
        return self._run(lambda *tail: lib.grab_scan_base_window_topk(self.h, C.c_void_p(_ptr(d_queries)), C.c_size_t(nq), C.c_uint32(k),
                                                                      _np_ptr(lo), _np_ptr(hi), *tail), nq, k, want_ms, d_out)

    def bucket_topk(self, bucket_offsets, d_queries, nq, k, masks, want_ms=False, d_out=None):
        off, m = np.ascontiguousarray(bucket_offsets, np.uint64), np.ascontiguousarray(masks, np.uint64)
        return self._run(lambda *tail: lib.grab_scan_base_bucket_topk(self.h, _np_ptr(off), C.c_uint32(off.size - 1),
                                                                      C.c_void_p(_ptr(d_queries)), C.c_size_t(nq), C.c_uint32(k),
                                                                      _np_ptr(m), *tail), nq, k, want_ms, d_out)

    def close(self):
        if self.h:
            lib.grab_scan_base_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def detour_counts(d_knn, n, degree):
    out = DeviceArray((n, degree), np.uint8)
    check(lib.grab_detour_counts(C.c_void_p(_ptr(d_knn)), C.c_void_p(out.ptr), C.c_size_t(n), C.c_uint32(degree), None))
    return out


def optimize_prune(d_knn, n, in_degree, out_degree):
    out = DeviceArray((n, out_degree), np.uint32)
    check(lib.grab_optimize_prune(C.c_void_p(_ptr(d_knn)), C.c_void_p(out.ptr), C.c_size_t(n), C.c_uint32(in_degree),
                                  C.c_uint32(out_degree), None))
    return out


def optimize_create_reverse_graph(d_graph, n, degree):
    rev = DeviceArray((n, degree), np.uint32)
    cnt = DeviceArray((n,), np.uint32)
    check(lib.grab_optimize_create_reverse_graph(C.c_void_p(_ptr(d_graph)), C.c_void_p(rev.ptr), C.c_void_p(cnt.ptr),
                                                 C.c_size_t(n), C.c_uint32(degree), None))
    return rev, cnt


def optimize_merge_graphs(d_graph, d_rev, d_cnt, n, degree):
    check(lib.grab_optimize_merge_graphs(C.c_void_p(_ptr(d_graph)), C.c_void_p(_ptr(d_rev)), C.c_void_p(_ptr(d_cnt)),
                                         C.c_size_t(n), C.c_uint32(degree), None))


def build_graph(d_dataset, n, d_knn, intermediate_degree, graph_degree):
    out = DeviceArray((n, graph_degree), np.uint32)
    check(lib.grab_build_graph(C.c_void_p(_ptr(d_dataset)), C.c_size_t(n), C.c_void_p(_ptr(d_knn)),
                               BuildParams(intermediate_degree, graph_degree), C.c_void_p(out.ptr), None))
    return out


def remote_global_k(total_degree, local_degree):
    lib.grab_remote_global_k.restype = C.c_uint32
    return lib.grab_remote_global_k(C.c_uint32(total_degree), C.c_uint32(local_degree))


def build_time_partitioned_graph(d_dataset, n, dim, d_ts, bucket_sizes, total_degree, local_degree, metric=METRIC_L2):
    out = DeviceArray((n, total_degree), np.uint32)
    bs = (C.c_size_t * len(bucket_sizes))(*[int(b) for b in bucket_sizes])
    check(lib.grab_build_time_partitioned_graph(C.c_void_p(_ptr(d_dataset)), C.c_size_t(n), C.c_uint32(dim), C.c_void_p(out.ptr),
                                                C.c_void_p(_ptr(d_ts)), bs, C.c_size_t(len(bucket_sizes)), C.c_uint32(total_degree),
                                                C.c_uint32(local_degree), C.c_int(metric), None))
    return out


def update_remote_edges(d_graph, d_ts, d_cand, n, total_degree, local_degree, global_k):
    check(lib.grab_update_remote_edges(C.c_void_p(_ptr(d_graph)), C.c_void_p(_ptr(d_ts)), C.c_void_p(_ptr(d_cand)), C.c_size_t(n),
                                       C.c_uint32(total_degree), C.c_uint32(local_degree), C.c_uint32(global_k), None))


def enhance_global_connectivity(d_graph, n, total_degree, local_degree):
    check(lib.grab_enhance_global_connectivity(C.c_size_t(n), C.c_void_p(_ptr(d_graph)), C.c_uint32(total_degree),
                                               C.c_uint32(local_degree), None))


def insert(d_dataset, dim, n_existing, n_new, d_new_data, d_graph, degree, params, rng_state, metric=METRIC_L2,
           flags=0, striped_sort=0):
    """grab_insert (one cagra::insert step).  Returns the advanced rng state."""
    st = C.c_uint64(rng_state)
    check(lib.grab_insert(C.c_void_p(_ptr(d_dataset)), C.c_uint32(dim), C.c_size_t(n_existing), C.c_size_t(n_new),
                          C.c_void_p(_ptr(d_new_data)), C.c_void_p(_ptr(d_graph)), C.c_uint32(degree), params,
                          C.c_int(metric), C.byref(st), C.c_uint32(flags), C.c_int(striped_sort), None))
    return st.value


def insert_partitioned(d_dataset, d_graph, d_ts, d_seeds, n_existing, n_new, target_ts, dim, total_degree, local_degree,
                       params, n_seeds_per_query, rng_state, metric=METRIC_L2, flags=0):
    """grab_insert_partitioned (one cagra::insert step of the partitioned index).  Returns the advanced rng state."""
    st = C.c_uint64(rng_state)
    check(lib.grab_insert_partitioned(C.c_void_p(_ptr(d_dataset)), C.c_void_p(_ptr(d_graph)), C.c_void_p(_ptr(d_ts)),
                                      C.c_void_p(_ptr(d_seeds)), C.c_size_t(n_existing), C.c_size_t(n_new),
                                      C.c_uint64(target_ts), C.c_uint32(dim), C.c_uint32(total_degree),
                                      C.c_uint32(local_degree), params, C.c_uint32(n_seeds_per_query), C.c_int(metric),
                                      C.byref(st), C.c_uint32(flags), None))
    return st.value


def sample_window_seeds(d_sorted_ts, d_ids_by_ts, n, nq, n_seeds, seed, win=None, d_win_start=None, d_win_end=None):
    out = DeviceArray((nq, n_seeds), np.uint32)
    ws, we = (int(win[0]), int(win[1])) if win is not None else (0, 0)
    check(lib.grab_sample_window_seeds(C.c_void_p(_ptr(d_sorted_ts)), C.c_void_p(_ptr(d_ids_by_ts)), C.c_size_t(n),
                                       C.c_void_p(_ptr(d_win_start)), C.c_void_p(_ptr(d_win_end)), C.c_uint64(ws),
                                       C.c_uint64(we), C.c_int(1 if d_win_start is not None else 0), C.c_size_t(nq),
                                       C.c_uint32(n_seeds), C.c_uint64(seed), C.c_void_p(out.ptr), None))
    return out


class Vmm:
    """grab_vmm_*: growable device buffer (cagra::DeviceBufferVMM)."""

    def __init__(self, max_bytes):
        self.h = C.c_void_p()
        check(lib.grab_vmm_create(C.c_size_t(max_bytes), C.byref(self.h)))

    def resize(self, nbytes):
        check(lib.grab_vmm_resize(self.h, C.c_size_t(nbytes)))

    @property
    def ptr(self):
        return lib.grab_vmm_data(self.h)

    @property
    def size(self):
        return lib.grab_vmm_size(self.h)

    @property
    def capacity(self):
        return lib.grab_vmm_capacity(self.h)

    def close(self):
        if self.h:
            lib.grab_vmm_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class CagraIndex:
    """Python mirror of cagra::CagraIndex (src/cagraIndex.hpp:12-119) over the grab_index_* handle."""

    def __init__(self, dim, graph_degree=64, vmm_max_bytes=20 << 30, local_degree=0):
        self.dim, self.degree = dim, graph_degree
        self.h = C.c_void_p()
        check(lib.grab_index_create(C.c_uint32(dim), C.c_uint32(graph_degree), C.c_uint32(local_degree),
                                    C.c_size_t(vmm_max_bytes), C.byref(self.h)))

    def close(self):
        if self.h and not getattr(self, "_borrowed", False):
            lib.grab_index_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @classmethod
    def borrowed(cls, handle, dim, degree):
        """A view of a handle that something else owns (a level of a TimeStampIndex): never destroyed from here."""
        self = cls.__new__(cls)
        self.dim, self.degree, self.h, self._borrowed = dim, degree, C.c_void_p(handle), True
        return self

    def set_seed(self, seed):
        check(lib.grab_index_set_seed(self.h, C.c_uint64(seed)))

    def rng_state(self):
        v = C.c_uint64()
        check(lib.grab_index_get_rng_state(self.h, C.byref(v)))
        return v.value

    def query_params(self):
        """(itopk, search_width, min_iterations, max_iterations, hash_bitlen) in force."""
        p = SearchParams()
        check(lib.grab_index_get_query_params(self.h, C.byref(p)))
        return p.itopk_size, p.search_width, p.min_iterations, p.max_iterations, p.hash_bitlen

    def set_metric(self, metric):
        check(lib.grab_index_set_metric(self.h, C.c_int(metric)))

    def set_flags(self, flags):
        check(lib.grab_index_set_flags(self.h, C.c_uint32(flags)))

    def debug_fail_insert(self, inner_step):
        check(lib.grab_index_debug_fail_insert(self.h, C.c_int(inner_step)))

    def set_scan_below(self, fraction):
        check(lib.grab_index_set_scan_below(self.h, C.c_double(fraction)))

    def set_entry_list(self, max_rows):
        check(lib.grab_index_set_entry_list(self.h, C.c_uint32(max_rows)))

    def set_batch_chunk(self, queries_per_chunk):
        check(lib.grab_index_set_batch_chunk(self.h, C.c_size_t(queries_per_chunk)))

    def set_entry_layer(self, num_samples, seeds_per_query=16):
        check(lib.grab_index_set_entry_layer(self.h, C.c_uint32(num_samples), C.c_uint32(seeds_per_query)))

    def set_entry_groups(self, num_groups, nprobe=16, min_rows=32):
        check(lib.grab_index_set_entry_groups(self.h, C.c_uint32(num_groups), C.c_uint32(nprobe), C.c_uint32(min_rows)))

    def setBuildParams(self, inter_degree, graph_degree):
        check(lib.grab_index_set_build_params(self.h, C.c_uint32(inter_degree), C.c_uint32(graph_degree)))

    def setQueryParams(self, itopk, width, min_iter, max_iter, hash_bitlen):
        check(lib.grab_index_set_query_params(self.h, *(C.c_uint32(x) for x in (itopk, width, min_iter, max_iter, hash_bitlen))))

    def setInsertParams(self, itopk, width, min_iter, max_iter, hash_bitlen):
        check(lib.grab_index_set_insert_params(self.h, *(C.c_uint32(x) for x in (itopk, width, min_iter, max_iter, hash_bitlen))))

    def _vt(self, vectors, ts):
        v = np.ascontiguousarray(vectors, np.float32)
        t = None if ts is None else np.ascontiguousarray(ts, np.uint64)
        return v, t

    def add(self, vectors, timestamps=None):
        v, t = self._vt(vectors, timestamps)
        check(lib.grab_index_add(self.h, C.c_size_t(v.shape[0]), _np_ptr(v), None if t is None else _np_ptr(t)))

    def set_labels(self, labels):
        l = np.ascontiguousarray(labels, np.uint8)
        check(lib.grab_index_set_labels(self.h, C.c_size_t(l.size), _np_ptr(l)))

    def build(self):
        check(lib.grab_index_build(self.h))

    def build_partitioned(self):
        check(lib.grab_index_build_partitioned(self.h))

    def insert(self, vectors, timestamps=None):
        v, t = self._vt(vectors, timestamps)
        check(lib.grab_index_insert(self.h, C.c_size_t(v.shape[0]), _np_ptr(v), None if t is None else _np_ptr(t)))

    def insert_partitioned(self, vectors, timestamps):
        """CagraIndexOpt::insert: all rows are seeded from the bucket timestamps[0]."""
        v, t = self._vt(vectors, timestamps)
        check(lib.grab_index_insert_partitioned(self.h, C.c_size_t(v.shape[0]), _np_ptr(v), _np_ptr(t)))

    def _out(self, nq, k):
        return np.full((nq, k), -7, np.int64), np.full((nq, k), np.nan, np.float32)

    def query(self, queries, k, seeds=None):
        q = np.ascontiguousarray(queries, np.float32)
        ids, dist = self._out(q.shape[0], k)
        s = None if seeds is None else np.ascontiguousarray(seeds, np.uint32)
        check(lib.grab_index_search(self.h, _np_ptr(q), C.c_size_t(q.shape[0]), C.c_int(k), _np_ptr(ids), _np_ptr(dist),
                                    None if s is None else _np_ptr(s), C.c_size_t(0 if s is None else s.shape[1])))
        return ids, dist

    def query_range(self, queries, k, range_radius, start_ts, end_ts):
        q = np.ascontiguousarray(queries, np.float32)
        ids, dist = self._out(q.shape[0], k)
        check(lib.grab_index_search_range(self.h, _np_ptr(q), C.c_size_t(q.shape[0]), C.c_int(k), C.c_float(range_radius),
                                          C.c_uint64(start_ts), C.c_uint64(end_ts), _np_ptr(ids), _np_ptr(dist), None,
                                          C.c_size_t(0)))
        return ids, dist

    def query_range_batch(self, queries, k, start_ts, end_ts):
        q = np.ascontiguousarray(queries, np.float32)
        s, e = np.ascontiguousarray(start_ts, np.uint64), np.ascontiguousarray(end_ts, np.uint64)
        ids, dist = self._out(q.shape[0], k)
        check(lib.grab_index_search_range_batch(self.h, _np_ptr(q), C.c_size_t(q.shape[0]), C.c_int(k), _np_ptr(s),
                                                _np_ptr(e), _np_ptr(ids), _np_ptr(dist)))
        return ids, dist

    def scan_range_batch(self, queries, k, start_ts, end_ts):
        """grab_index_scan_range_batch: the exact top-k of every query inside its window."""
        q = np.ascontiguousarray(queries, np.float32)
        s, e = np.ascontiguousarray(start_ts, np.uint64), np.ascontiguousarray(end_ts, np.uint64)
        ids, dist = self._out(q.shape[0], k)
        check(lib.grab_index_scan_range_batch(self.h, _np_ptr(q), C.c_size_t(q.shape[0]), C.c_int(k), _np_ptr(s),
                                              _np_ptr(e), _np_ptr(ids), _np_ptr(dist)))
        return ids, dist

    def query_local(self, queries, k, target_ts):
        q = np.ascontiguousarray(queries, np.float32)
        ids, dist = self._out(q.shape[0], k)
        check(lib.grab_index_search_bucket(self.h, _np_ptr(q), C.c_size_t(q.shape[0]), C.c_int(k), C.c_uint64(target_ts),
                                           _np_ptr(ids), _np_ptr(dist)))
        return ids, dist

    def query_mask(self, queries, k, masks):
        q = np.ascontiguousarray(queries, np.float32)
        m = np.ascontiguousarray(masks, np.uint64)
        ids, dist = self._out(q.shape[0], k)
        check(lib.grab_index_search_mask(self.h, _np_ptr(q), C.c_size_t(q.shape[0]), C.c_int(k), _np_ptr(m), _np_ptr(ids),
                                         _np_ptr(dist)))
        return ids, dist

    def size(self):
        return lib.grab_index_size(self.h)

    def get_graph(self):
        p = lib.grab_index_get_graph(self.h)
        n = self.size()
        if not p or n == 0:
            return np.zeros((0, self.degree), np.uint32)
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint32)), shape=(n, self.degree)).copy()

    def get_data(self):
        p = lib.grab_index_get_data(self.h)
        n = self.size()
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_float)), shape=(n, self.dim)).copy()

    def ids_by_timestamp(self, ts):
        n = lib.grab_index_ids_by_timestamp(self.h, C.c_uint64(ts), None, C.c_size_t(0))
        out = np.zeros(n, np.uint32)
        if n:
            lib.grab_index_ids_by_timestamp(self.h, C.c_uint64(ts), _np_ptr(out), C.c_size_t(n))
        return out

    def mapped_bytes(self):
        a, b, c = C.c_size_t(), C.c_size_t(), C.c_size_t()
        check(lib.grab_index_mapped_bytes(self.h, C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    def device_ptrs(self):
        a, b, c = C.c_void_p(), C.c_void_p(), C.c_void_p()
        check(lib.grab_index_device_ptrs(self.h, C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    def last_kernel_ms(self):
        return lib.grab_index_last_kernel_ms(self.h)

    def last_build_seconds(self):
        a, b, c = C.c_double(), C.c_double(), C.c_double()
        check(lib.grab_index_last_build_seconds(self.h, C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    def save_mcag(self, path):
        check(lib.grab_index_save_mcag(self.h, path.encode()))

    def load_mcag(self, path):
        check(lib.grab_index_load_mcag(self.h, path.encode()))

    def sample_seeds_by_time(self, min_ts, max_ts, num):
        lib.grab_index_sample_seeds_by_time.restype = C.c_size_t
        out = np.zeros(num, np.uint32)
        got = lib.grab_index_sample_seeds_by_time(self.h, C.c_uint64(min_ts), C.c_uint64(max_ts), C.c_size_t(num), _np_ptr(out),
                                                  C.c_size_t(num))
        return out[:got]

    def save(self, path):
        check(lib.grab_index_save(self.h, path.encode()))

    def load(self, path):
        check(lib.grab_index_load(self.h, path.encode()))


def kmeans(data, k, niter, seed):
    """grab_kmeans: (centroids f32 [k,dim], assignment int64 [n])."""
    data = np.ascontiguousarray(data, np.float32)
    cent = np.zeros((k, data.shape[1]), np.float32)
    assign = np.zeros(data.shape[0], np.int64)
    check(lib.grab_kmeans(_np_ptr(data), C.c_size_t(data.shape[0]), C.c_uint32(data.shape[1]), C.c_uint32(k), C.c_uint32(niter),
                          C.c_uint64(seed), _np_ptr(cent), _np_ptr(assign)))
    return cent, assign


class TimeStampIndex:
    """Python mirror of timestamp::TimeStampIndex (src/timeStampIndex.cuh:47-63) over grab_tsindex_*."""

    def __init__(self, dim, degree=32, cluster_ratio=1000, vmm_max_bytes_per_bucket=1 << 30):
        self.dim, self.degree = dim, degree
        self.h = C.c_void_p()
        for f in (lib.grab_tsindex_size, lib.grab_tsindex_num_buckets, lib.grab_tsindex_num_virtual_points):
            f.restype = C.c_size_t
        lib.grab_tsindex_destroy.restype = None
        check(lib.grab_tsindex_create(C.c_uint32(dim), C.c_uint32(degree), C.c_size_t(cluster_ratio),
                                      C.c_size_t(vmm_max_bytes_per_bucket), C.byref(self.h)))

    def set_seed(self, seed):
        check(lib.grab_tsindex_set_seed(self.h, C.c_uint64(seed)))

    def insert(self, vectors, timestamps):
        v = np.ascontiguousarray(vectors, np.float32)
        t = np.ascontiguousarray(timestamps, np.uint64)
        start = C.c_uint64()
        check(lib.grab_tsindex_insert(self.h, _np_ptr(v), _np_ptr(t), C.c_size_t(v.shape[0]), C.byref(start)))
        return start.value

    def build_virtual_index(self):
        check(lib.grab_tsindex_build_virtual_index(self.h))

    def query(self, query, topk, probe_buckets=5):
        q = np.ascontiguousarray(query, np.float32)
        ids = np.full(topk, -7, np.int64)
        dist = np.full(topk, np.nan, np.float32)
        check(lib.grab_tsindex_query(self.h, _np_ptr(q), C.c_size_t(topk), _np_ptr(ids), _np_ptr(dist), C.c_int(probe_buckets)))
        return ids, dist

    def size(self):
        return lib.grab_tsindex_size(self.h)

    def num_buckets(self):
        return lib.grab_tsindex_num_buckets(self.h)

    def num_virtual_points(self):
        return lib.grab_tsindex_num_virtual_points(self.h)

    def virtual_index(self):
        """The CagraIndex over the centroids as a borrowed view (None before build_virtual_index)."""
        lib.grab_tsindex_virtual_index.restype = C.c_void_p
        h = lib.grab_tsindex_virtual_index(self.h)
        return CagraIndex.borrowed(h, self.dim, self.degree) if h else None

    def bucket_index(self, ts):
        lib.grab_tsindex_bucket_index.restype = C.c_void_p
        h = lib.grab_tsindex_bucket_index(self.h, C.c_uint64(ts))
        return CagraIndex.borrowed(h, self.dim, self.degree) if h else None

    def bucket_timestamps(self):
        lib.grab_tsindex_bucket_timestamps.restype = C.c_size_t
        out = np.zeros(self.num_buckets(), np.uint64)
        lib.grab_tsindex_bucket_timestamps(self.h, _np_ptr(out), C.c_size_t(out.size))
        return out

    def virtual_point(self, i):
        """(bucket timestamp, entry points as local ids of that bucket) of virtual point i."""
        ts, cnt = C.c_uint64(), C.c_size_t()
        ep = np.zeros(16, np.uint32)
        check(lib.grab_tsindex_virtual_point(self.h, C.c_size_t(i), C.byref(ts), _np_ptr(ep), C.c_size_t(16), C.byref(cnt)))
        return ts.value, ep[:cnt.value].copy()

    def locate(self, gid):
        ts, loc = C.c_uint64(), C.c_size_t()
        check(lib.grab_tsindex_locate(self.h, C.c_uint64(gid), C.byref(ts), C.byref(loc)))
        return ts.value, loc.value

    def close(self):
        if self.h:
            lib.grab_tsindex_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class EntryLayer:
    """grab_entry_layer_*: sample of the base + MFMA seed selection (extension)."""

    def __init__(self, d_dataset, n, dim, num_samples, d_ids_by_ts=None, d_ts=None, d_labels=None):
        self.h = C.c_void_p()
        self.dim = dim
        lib.grab_entry_layer_size.restype = C.c_uint32
        lib.grab_entry_layer_last_select_ms.restype = C.c_float
        lib.grab_entry_layer_destroy.restype = None
        check(lib.grab_entry_layer_create(C.c_void_p(_ptr(d_dataset)), C.c_size_t(n), C.c_uint32(dim),
                                          C.c_void_p(_ptr(d_ids_by_ts)), C.c_void_p(_ptr(d_ts)), C.c_void_p(_ptr(d_labels)),
                                          C.c_uint32(num_samples), C.byref(self.h)))

    @property
    def size(self):
        return lib.grab_entry_layer_size(self.h)

    @property
    def last_select_ms(self):
        return float(lib.grab_entry_layer_last_select_ms(self.h))

    def select(self, d_queries, nq, n_seeds, metric=METRIC_L2, filter_kind=FILTER_NONE, win=None, d_win_start=None,
               d_win_end=None, d_masks=None, d_out=None, want_ms=False):
        out = d_out if d_out is not None else DeviceArray((nq, n_seeds), np.uint32)
        ms = C.c_float(0.0)
        ws, we = (int(win[0]), int(win[1])) if win is not None else (0, 0)
        check(lib.grab_entry_layer_select(self.h, C.c_void_p(_ptr(d_queries)), C.c_size_t(nq), C.c_int(metric),
                                          C.c_int(filter_kind), C.c_void_p(_ptr(d_win_start)), C.c_void_p(_ptr(d_win_end)),
                                          C.c_uint64(ws), C.c_uint64(we), C.c_int(1 if d_win_start is not None else 0),
                                          C.c_void_p(_ptr(d_masks)), C.c_uint32(n_seeds), C.c_void_p(out.ptr),
                                          C.pointer(ms) if want_ms else None, None))
        synchronize()  # the call itself is stream-ordered
        return (out, ms.value) if want_ms else out

    def build_groups(self, num_groups, niter=10, seed=1):
        """grab_entry_layer_build_groups: k-means groups of the sample rows (coarse level)."""
        check(lib.grab_entry_layer_build_groups(self.h, C.c_uint32(num_groups), C.c_uint32(niter), C.c_uint64(seed)))

    @property
    def num_groups(self):
        lib.grab_entry_layer_num_groups.restype = C.c_uint32
        return lib.grab_entry_layer_num_groups(self.h)

    def select_grouped(self, d_queries, nq, n_seeds, nprobe, min_rows, metric=METRIC_L2, win=None, d_win_start=None,
                       d_win_end=None, d_out=None, want_ms=False, sync=True, d_base_ts=None, num_base=0, d_id_lo=None,
                       d_id_hi=None, stream=None):
        """grab_entry_layer_select_grouped.  `stream`: a Stream; with sync=False the call returns with the kernels queued."""
        out = d_out if d_out is not None else DeviceArray((nq, n_seeds), np.uint32)
        ms = C.c_float(0.0)
        ws, we = (int(win[0]), int(win[1])) if win is not None else (0, 0)
        check(lib.grab_entry_layer_select_grouped(self.h, C.c_void_p(_ptr(d_queries)), C.c_size_t(nq), C.c_int(metric),
                                                  C.c_void_p(_ptr(d_win_start)), C.c_void_p(_ptr(d_win_end)), C.c_uint64(ws),
                                                  C.c_uint64(we), C.c_int(1 if d_win_start is not None else 0),
                                                  C.c_void_p(_ptr(d_base_ts)), C.c_size_t(num_base), C.c_void_p(_ptr(d_id_lo)),
                                                  C.c_void_p(_ptr(d_id_hi)),
                                                  C.c_uint32(nprobe), C.c_uint32(min_rows), C.c_uint32(n_seeds),
                                                  C.c_void_p(out.ptr), C.pointer(ms) if want_ms else None,
                                                  stream.ptr if stream is not None else None))
        if sync:
            synchronize()
        return (out, ms.value) if want_ms else out

    def probe(self, d_queries, nq, nprobe, metric=METRIC_L2, d_out=None, want_ms=False, sync=True, stream=None):
        """grab_entry_layer_probe: the nprobe nearest centroids of every query, nearest first (uint32 [nq, nprobe])."""
        out = d_out if d_out is not None else DeviceArray((nq, nprobe), np.uint32)
        ms = C.c_float(0.0)
        check(lib.grab_entry_layer_probe(self.h, C.c_void_p(_ptr(d_queries)), C.c_size_t(nq), C.c_int(metric), C.c_uint32(nprobe),
                                         C.c_void_p(out.ptr), C.pointer(ms) if want_ms else None,
                                         stream.ptr if stream is not None else None))
        if sync:
            synchronize()
        return (out, ms.value) if want_ms else out

    def centroids(self):
        """The centroids of the groups, float32 [num_groups, dim]."""
        out = DeviceArray((self.num_groups, self.dim), np.float32)
        check(lib.grab_entry_layer_centroids(self.h, C.c_void_p(out.ptr)))
        return out.numpy()

    def groups(self):
        """(offsets uint32 [num_groups + 1], member row ids uint32 [size]) of the groups."""
        off = np.empty(self.num_groups + 1, np.uint32)
        ids = np.empty(self.size, np.uint32)
        check(lib.grab_entry_layer_groups(self.h, off.ctypes.data_as(C.c_void_p), ids.ctypes.data_as(C.c_void_p)))
        return off, ids

    def list_grouped(self, d_queries, nq, max_ids, nprobe, min_rows, metric=METRIC_L2, d_win_start=None, d_win_end=None,
                     d_out=None, sync=True, d_base_ts=None, num_base=0, d_id_lo=None, d_id_hi=None, stream=None, win=None):
        """grab_entry_layer_list_grouped: the in-window members of the nearest groups as they come, unscored."""
        out = d_out if d_out is not None else DeviceArray((nq, max_ids), np.uint32)
        ws, we = (int(win[0]), int(win[1])) if win is not None else (0, 0)
        check(lib.grab_entry_layer_list_grouped(self.h, C.c_void_p(_ptr(d_queries)), C.c_size_t(nq), C.c_int(metric),
                                                C.c_void_p(_ptr(d_win_start)), C.c_void_p(_ptr(d_win_end)), C.c_uint64(ws),
                                                C.c_uint64(we), C.c_int(1 if d_win_start is not None else 0),
                                                C.c_void_p(_ptr(d_base_ts)), C.c_size_t(num_base), C.c_void_p(_ptr(d_id_lo)),
                                                C.c_void_p(_ptr(d_id_hi)), C.c_uint32(nprobe), C.c_uint32(min_rows),
                                                C.c_uint32(max_ids), C.c_void_p(out.ptr), None,
                                                stream.ptr if stream is not None else None))
        if sync:
            synchronize()
        return out

    def close(self):
        if self.h:
            lib.grab_entry_layer_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def windows_to_id_ranges(d_ts, n, d_win_start, d_win_end, nq, d_lo=None, d_hi=None):
    """grab_windows_to_id_ranges: id bounds of each timestamp window (timestamps monotone in the row id)."""
    lo = d_lo if d_lo is not None else DeviceArray((nq,), np.uint64)
    hi = d_hi if d_hi is not None else DeviceArray((nq,), np.uint64)
    check(lib.grab_windows_to_id_ranges(C.c_void_p(_ptr(d_ts)), C.c_size_t(n), C.c_void_p(_ptr(d_win_start)),
                                        C.c_void_p(_ptr(d_win_end)), C.c_size_t(nq), C.c_void_p(lo.ptr), C.c_void_p(hi.ptr), None))
    return lo, hi
