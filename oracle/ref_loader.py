"""ctypes loader of oracle/_ref/libref_torch.so: the REFERENCE's own SwapManager / FeatureFilter / IdsMapper,
compiled from the reference checkout by `make -C oracle -f ref.mk`.  TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
from ctypes import c_int32, c_int64, c_uint64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_ref", "libref_torch.so")
_lib = None


def available():
    return os.path.exists(LIB_PATH)


def _p(a):
    return None if a is None else a.ctypes.data_as(c_void_p)


def lib():
    global _lib
    if _lib is None:
        import torch  # noqa: F401  (loads libtorch_cpu / libc10 the checker links against)
        L = ctypes.CDLL(LIB_PATH)
        L.ref_swap_create.restype = c_void_p
        L.ref_swap_create.argtypes = [c_int64, c_int64]
        L.ref_swap_destroy.argtypes = [c_void_p]
        L.ref_swap_compute.restype = c_int32
        L.ref_swap_compute.argtypes = [c_void_p, c_void_p, c_int64]
        L.ref_swap_result.restype = c_int64
        L.ref_swap_result.argtypes = [c_void_p, c_int32, c_void_p, c_int64]
        L.ref_swap_remove.argtypes = [c_void_p, c_void_p, c_int64]
        L.ref_filter_create.restype = c_void_p
        L.ref_filter_create.argtypes = [c_int64, c_uint64, c_uint64]
        L.ref_filter_destroy.argtypes = [c_void_p]
        L.ref_filter_statistics.argtypes = [c_void_p, c_void_p, c_void_p, c_int64]
        L.ref_filter_count_filter.argtypes = [c_void_p, c_void_p, c_int64]
        L.ref_filter_record_timestamp.restype = c_int64
        L.ref_filter_record_timestamp.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64]
        L.ref_ids_create.restype = c_void_p
        L.ref_ids_create.argtypes = [c_int64, c_void_p]
        L.ref_ids_destroy.argtypes = [c_void_p]
        L.ref_ids_parallel_unique_hash_out.restype = c_int32
        L.ref_ids_parallel_unique_hash_out.argtypes = [c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_void_p,
                                                       c_void_p, c_void_p, c_void_p, c_void_p]
        _lib = L
    return _lib


class RefSwap:
    def __init__(self, cache_size, mem_start=0):
        self.h = lib().ref_swap_create(cache_size, mem_start)

    def compute_swap_info(self, keys):
        keys = np.ascontiguousarray(keys, dtype=np.int64)
        if lib().ref_swap_compute(self.h, _p(keys), keys.size) != 0:
            raise RuntimeError("cacheSize_ too small")
        res = []
        for which in range(5):
            buf = np.empty(max(keys.size, 1), dtype=np.int64)
            m = lib().ref_swap_result(self.h, which, _p(buf), buf.size)
            res.append(buf[:m].copy())
        return tuple(res)

    def remove_keys(self, keys):
        keys = np.ascontiguousarray(keys, dtype=np.int64)
        lib().ref_swap_remove(self.h, _p(keys), keys.size)


class RefFilter:
    def __init__(self, admit_threshold=-1, evict_threshold=0, evict_step_interval=1):
        self.h = lib().ref_filter_create(admit_threshold, evict_threshold, evict_step_interval)

    def statistics_key_count(self, keys, counts=None):
        keys = np.ascontiguousarray(keys, dtype=np.int64)
        counts = None if counts is None else np.ascontiguousarray(counts, dtype=np.int64)
        lib().ref_filter_statistics(self.h, _p(keys), _p(counts), keys.size)

    def count_filter(self, keys):
        keys = np.ascontiguousarray(keys, dtype=np.int64).copy()
        lib().ref_filter_count_filter(self.h, _p(keys), keys.size)
        return keys

    def record_timestamp(self, keys, timestamps):
        """Returns the keys this call evicted (unordered set semantics in the reference)."""
        keys = np.ascontiguousarray(keys, dtype=np.int64)
        ts = np.ascontiguousarray(timestamps, dtype=np.int64)
        out = np.empty(1 << 20, dtype=np.int64)
        m = lib().ref_filter_record_timestamp(self.h, _p(keys), _p(ts), keys.size, _p(out), out.size)
        return out[:m].copy()


class RefIdsMapper:
    def __init__(self, init_max_index):
        imi = np.ascontiguousarray(init_max_index, dtype=np.int64)
        self.T = imi.size
        self.h = lib().ref_ids_create(self.T, _p(imi))

    def parallel_unique_hash_out(self, ids, offsets):
        ids = np.ascontiguousarray(ids, dtype=np.int64)
        offsets = np.ascontiguousarray(offsets, dtype=np.int64)
        n = ids.size
        bufs = [np.zeros(max(n, 1), dtype=np.int64) for _ in range(4)]
        uoff = np.zeros(self.T + 1, dtype=np.int64)
        rc = lib().ref_ids_parallel_unique_hash_out(self.h, _p(ids), n, _p(offsets), self.T, *[_p(b) for b in bufs],
                                                    _p(uoff))
        if rc != 0:
            raise RuntimeError("IdsMapper raised")
        u = int(uoff[-1])
        return bufs[0][:n], bufs[1][:u], bufs[2][:u], bufs[3][:n], uoff


def ref_unique_parallel(ids):
    ids = np.ascontiguousarray(ids, dtype=np.int64)
    out = np.zeros(max(ids.size, 1), dtype=np.int64)
    inv = np.zeros(max(ids.size, 1), dtype=np.int64)
    fn = lib().ref_unique_parallel
    fn.restype = ctypes.c_int64
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
    u = fn(_p(ids), ids.size, _p(out), _p(inv))
    return out[:u].copy(), inv[:ids.size].copy()
