"""ctypes binding of oracle/libhnsw_baseline.so, the CPU HNSW baseline (benchmark / test infrastructure only)."""
import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
lib = C.CDLL(os.path.join(ROOT, "oracle", "libhnsw_baseline.so"))
lib.hnsw_create.restype = C.c_void_p
lib.hnsw_size.restype = C.c_size_t


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


class Hnsw:
    """HNSW with the parameters of the benchmark configurations (M 32, efConstruction 200)."""

    def __init__(self, dim, M=32, ef_construction=200, seed=100):
        self.dim = dim
        self.h = C.c_void_p(lib.hnsw_create(C.c_uint32(dim), C.c_uint32(M), C.c_uint32(ef_construction), C.c_uint64(seed)))

    def add(self, rows, threads=0):
        rows = np.ascontiguousarray(rows, np.float32)
        lib.hnsw_add(self.h, C.c_size_t(rows.shape[0]), _p(rows), C.c_int(threads))

    def size(self):
        return lib.hnsw_size(self.h)

    def search(self, queries, k, ef=128, threads=0):
        q = np.ascontiguousarray(queries, np.float32)
        ids = np.zeros((q.shape[0], k), np.int64)
        dist = np.zeros((q.shape[0], k), np.float32)
        lib.hnsw_search(self.h, _p(q), C.c_size_t(q.shape[0]), C.c_uint32(k), C.c_uint32(ef), _p(ids), _p(dist), C.c_int(threads))
        return ids, dist

    def search_range(self, queries, k, timestamps, win_start, win_end, ef=128, threads=0):
        q = np.ascontiguousarray(queries, np.float32)
        ts = np.ascontiguousarray(timestamps, np.uint64)
        ws, we = np.ascontiguousarray(win_start, np.uint64), np.ascontiguousarray(win_end, np.uint64)
        ids = np.zeros((q.shape[0], k), np.int64)
        dist = np.zeros((q.shape[0], k), np.float32)
        lib.hnsw_search_range(self.h, _p(q), C.c_size_t(q.shape[0]), C.c_uint32(k), C.c_uint32(ef), _p(ts), _p(ws), _p(we),
                              _p(ids), _p(dist), None, C.c_int(threads))
        return ids, dist

    def close(self):
        if self.h:
            lib.hnsw_destroy(self.h)
            self.h = None
