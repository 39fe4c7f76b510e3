"""ctypes loader of the CPU oracle (oracle/librecsdk_oracle.so).  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package.
Build the library with `make -C oracle`.
"""
import ctypes
import os
import subprocess
from ctypes import c_float, c_int32, c_int64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "librecsdk_oracle.so")
_lib = None


def build():
    subprocess.check_call(["make", "-C", _HERE, "-s"])
    return LIB_PATH


def _ptr(a):
    return None if a is None else a.ctypes.data_as(c_void_p)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        L.orc_hash_split.restype = c_int64
        L.orc_hash_split.argtypes = [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p]
        L.orc_build_restore_vec.restype = None
        L.orc_build_restore_vec.argtypes = [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_int32]
        L.orc_global_unique.restype = c_int64
        L.orc_global_unique.argtypes = [c_void_p, c_int64, c_int32, c_int32, c_void_p, c_void_p]
        L.orc_table_create.restype = c_void_p
        L.orc_table_create.argtypes = [c_int64, c_int32, c_int64, c_int64]
        L.orc_table_destroy.restype = None
        L.orc_table_destroy.argtypes = [c_void_p]
        for name in ("orc_table_size", "orc_table_live", "orc_table_evict_count"):
            getattr(L, name).restype = c_int64
            getattr(L, name).argtypes = [c_void_p]
        L.orc_table_evict_pos.restype = None
        L.orc_table_evict_pos.argtypes = [c_void_p, c_void_p]
        L.orc_table_key2offset.restype = c_int32
        L.orc_table_key2offset.argtypes = [c_void_p, c_void_p, c_int64, c_int32]
        L.orc_table_evict.restype = c_int64
        L.orc_table_evict.argtypes = [c_void_p, c_void_p, c_int64]
        L.orc_faae_create.restype = c_void_p
        L.orc_faae_create.argtypes = [c_int32, c_int32, c_int32, c_int32]
        L.orc_faae_destroy.restype = None
        L.orc_faae_destroy.argtypes = [c_void_p]
        L.orc_faae_size.restype = c_int64
        L.orc_faae_size.argtypes = [c_void_p]
        L.orc_faae_dump.restype = c_int64
        L.orc_faae_dump.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p]
        L.orc_faae_admit.restype = c_int32
        L.orc_faae_admit.argtypes = [c_void_p, c_int32, c_void_p, c_void_p, c_int64, c_int64]
        L.orc_faae_evict.restype = c_int64
        L.orc_faae_evict.argtypes = [c_void_p, c_void_p, c_int64]
        L.orc_filter_create.restype = c_void_p
        L.orc_filter_create.argtypes = [c_int64, ctypes.c_uint64, ctypes.c_uint64]
        L.orc_filter_destroy.restype = None
        L.orc_filter_destroy.argtypes = [c_void_p]
        L.orc_filter_statistics.restype = None
        L.orc_filter_statistics.argtypes = [c_void_p, c_void_p, c_void_p, c_int64]
        L.orc_filter_count_filter.restype = None
        L.orc_filter_count_filter.argtypes = [c_void_p, c_void_p, c_int64]
        L.orc_filter_record_timestamp.restype = c_int32
        L.orc_filter_record_timestamp.argtypes = [c_void_p, c_void_p, c_void_p, c_int64]
        L.orc_filter_evicted.restype = c_int64
        L.orc_filter_evicted.argtypes = [c_void_p, c_void_p, c_int64]
        L.orc_swap_create.restype = c_void_p
        L.orc_swap_create.argtypes = [c_int64, c_int64]
        L.orc_swap_destroy.restype = None
        L.orc_swap_destroy.argtypes = [c_void_p]
        L.orc_swap_compute.restype = c_int32
        L.orc_swap_compute.argtypes = [c_void_p, c_void_p, c_int64, c_void_p]
        L.orc_swap_result.restype = c_int64
        L.orc_swap_result.argtypes = [c_void_p, c_int32, c_void_p, c_int64]
        L.orc_swap_remove.restype = None
        L.orc_swap_remove.argtypes = [c_void_p, c_void_p, c_int64]
        L.orc_unique_sharded.restype = c_int64
        L.orc_unique_sharded.argtypes = [c_void_p, c_int64, c_int32, c_int32, c_int32, c_int64, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_void_p, c_void_p]
        L.orc_unique_sorted.restype = c_int64
        L.orc_unique_sorted.argtypes = [c_void_p, c_int64, c_void_p, c_void_p]
        L.orc_om_create.restype = c_void_p
        L.orc_om_create.argtypes = [c_int64]
        L.orc_om_destroy.restype = None
        L.orc_om_destroy.argtypes = [c_void_p]
        L.orc_om_compute.restype = c_int32
        L.orc_om_compute.argtypes = [c_void_p, c_void_p, c_int64]
        L.orc_om_result.restype = c_int64
        L.orc_om_result.argtypes = [c_void_p, c_int32, c_void_p, c_int64]
        L.orc_om_remove.restype = None
        L.orc_om_remove.argtypes = [c_void_p, c_void_p, c_int64]
        L.orc_om_state.restype = None
        L.orc_om_state.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p]
        L.orc_init_create.restype = c_void_p
        L.orc_init_create.argtypes = [c_void_p, c_void_p, c_int32]
        L.orc_init_destroy.restype = None
        L.orc_init_destroy.argtypes = [c_void_p]
        L.orc_init_generate.restype = None
        L.orc_init_generate.argtypes = [c_void_p, c_void_p, c_int64, c_int32]
        L.orc_minstd_rand0.restype = None
        L.orc_minstd_rand0.argtypes = [ctypes.c_uint32, c_int64, c_void_p]
        L.orc_lookup_by_addr.restype = None
        L.orc_lookup_by_addr.argtypes = [c_void_p, c_int64, c_int32, c_int32, c_void_p]
        L.orc_update_by_addr_f32.restype = None
        L.orc_update_by_addr_f32.argtypes = [c_void_p, c_int64, c_int32, c_void_p, c_int32]
        L.orc_lazy_adam.restype = None
        L.orc_lazy_adam.argtypes = [c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_float,
                                    c_float, c_float, c_float]
        L.orc_sgd.restype = None
        L.orc_sgd.argtypes = [c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_float, c_float]
        L.orc_segment_sum.restype = None
        L.orc_segment_sum.argtypes = [c_void_p, c_void_p, c_int64, c_int32, c_int64, c_void_p]
        L.orc_byaddr_apply.restype = None
        L.orc_byaddr_apply.argtypes = [c_int32, c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p,
                                       c_int64, c_float, c_float, c_float, c_float, c_float, c_int32]
        L.orc_gather_rows.restype = None
        L.orc_gather_rows.argtypes = [c_void_p, c_int64, c_void_p, c_int64, c_int32, c_void_p]
        L.orc_tbe_forward.restype = None
        L.orc_tbe_forward.argtypes = [c_void_p, c_int32, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int32,
                                      c_int64, c_int32, c_void_p]
        L.orc_tbe_backward.restype = None
        L.orc_tbe_backward.argtypes = [c_int32, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_int64, c_void_p,
                                       c_void_p, c_void_p, c_int32, c_int64, c_int32, c_void_p, c_void_p, c_float,
                                       c_float, c_float, c_float, c_int64]
        L.orc_tbe_backward_unique.restype = None
        L.orc_tbe_backward_unique.argtypes = [c_int32, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_int64,
                                              c_void_p, c_int32, c_int64, c_int32, c_void_p, c_void_p, c_void_p,
                                              c_void_p, c_void_p, c_float, c_float, c_float, c_float, c_int64]
        _lib = L
    return _lib


# ---- numpy-level wrappers ------------------------------------------------------------------------

def hash_split(keys, rank_size=1, with_counts=True):
    """Returns (split_keys, split_offsets, restore, counts)."""
    keys = np.ascontiguousarray(keys, dtype=np.int64)
    n = keys.size
    split = np.empty(n, dtype=np.int64)
    offs = np.empty(rank_size + 1, dtype=np.int64)
    restore = np.empty(n, dtype=np.int32)
    counts = np.empty(n, dtype=np.uint32) if with_counts else None
    u = lib().orc_hash_split(_ptr(keys), n, rank_size, _ptr(split), _ptr(offs), _ptr(restore), _ptr(counts))
    return split[:u].copy(), offs, restore, (counts[:u].copy() if with_counts else None)


def build_restore_vec(keys, rank_size, block_offset, restore, hot_pos_size=0):
    keys = np.ascontiguousarray(keys, dtype=np.int64)
    block_offset = np.ascontiguousarray(block_offset, dtype=np.int32)
    restore = np.ascontiguousarray(restore, dtype=np.int32).copy()
    lib().orc_build_restore_vec(_ptr(keys), keys.size, rank_size, _ptr(block_offset), _ptr(restore), hot_pos_size)
    return restore


def read_emb_key(data, splits, table_used=None, is_timestamp=False, field_num=None):
    """Returns (sample, offsets, timestamp); raises ValueError with the reference's message on a bad timestamp."""
    data = np.ascontiguousarray(data)
    assert data.dtype in (np.int32, np.int64)
    splits = np.ascontiguousarray(splits, dtype=np.int64)
    used = None if table_used is None else np.ascontiguousarray(table_used, dtype=np.uint8)
    n_used = splits.size if used is None else int(np.count_nonzero(used))
    sample = np.empty(max(int(splits.sum()), 1), dtype=np.int64)
    offsets = np.zeros(n_used + 1, dtype=np.int64)
    ts = np.zeros(1, dtype=np.int64)
    fn = lib().orc_read_emb_key
    fn.restype = c_int64
    fn.argtypes = [c_void_p, c_int32, c_int64, c_void_p, c_void_p, c_int32, c_int32, c_int64, c_void_p, c_void_p,
                   c_void_p]
    r = fn(_ptr(data), int(data.dtype == np.int32), data.size, _ptr(splits), _ptr(used), splits.size,
           int(bool(is_timestamp)), int(splits.sum()) if field_num is None else field_num, _ptr(sample), _ptr(offsets),
           _ptr(ts))
    if r == -1:
        raise ValueError("Timestamp field not found")
    if r == -2:
        raise ValueError("Timestamp should greater than 0")
    return sample[:r].copy(), offsets, int(ts[0])


def padding_keys_mask(values, padding_keys):
    values = np.ascontiguousarray(values, dtype=np.int64)
    pad = np.ascontiguousarray(padding_keys, dtype=np.int64)
    mask = np.empty(values.size, dtype=np.int32)
    fn = lib().orc_padding_keys_mask
    fn.restype = None
    fn.argtypes = [c_void_p, c_int64, c_void_p, c_int32, c_void_p]
    fn(_ptr(values), values.size, _ptr(pad), pad.size, _ptr(mask))
    return mask


class HotKeys:
    """One table's hot-key state: HotHashSplit + UpdateHotMap for rankSize 1."""

    def __init__(self, hot_emb_tot_count):
        L = lib()
        L.orc_hot_create.restype = ctypes.c_void_p
        L.orc_hot_create.argtypes = [ctypes.c_int32]
        L.orc_hot_destroy.argtypes = [ctypes.c_void_p]
        L.orc_hot_hash_split.restype = ctypes.c_int64
        L.orc_hot_hash_split.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32] + \
            [ctypes.c_void_p] * 4
        L.orc_hot_keys.restype = ctypes.c_int64
        L.orc_hot_keys.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
        self.tot = int(hot_emb_tot_count)
        self.h = L.orc_hot_create(self.tot)

    def __del__(self):
        if lib is not None and self.h:
            lib().orc_hot_destroy(self.h)
            self.h = None

    def hot_hash_split(self, keys, refresh):
        """Returns (split_keys, restore, hot_pos, key_count)."""
        keys = np.ascontiguousarray(keys, dtype=np.int64)
        n = keys.size
        split = np.empty(max(n, 1), dtype=np.int64)
        restore = np.empty(max(n, 1), dtype=np.int32)
        hot_pos = np.empty(max(self.tot, 1), dtype=np.int32)
        cnt = np.empty(max(n, 1), dtype=np.uint32)
        u = lib().orc_hot_hash_split(self.h, _ptr(keys), n, int(bool(refresh)), _ptr(split), _ptr(restore),
                                     _ptr(hot_pos), _ptr(cnt))
        return split[:u].copy(), restore[:n].copy(), hot_pos[:self.tot].copy(), cnt[:u].copy()

    def hot_keys(self):
        out = np.empty(max(self.tot, 1), dtype=np.int64)
        m = lib().orc_hot_keys(self.h, _ptr(out), out.size)
        return out[:m].copy()


def global_unique(lookup_keys, use_static=False, use_dynamic_expansion=False):
    """Returns (unique_keys (padded when use_static), restore_vec_sec, u)."""
    lk = np.ascontiguousarray(lookup_keys, dtype=np.int64)
    m = lk.size
    uniq = np.empty(m, dtype=np.int64)
    rvs = np.empty(m, dtype=np.int32)
    u = lib().orc_global_unique(_ptr(lk), m, int(use_static), int(use_dynamic_expansion), _ptr(uniq), _ptr(rvs))
    return (uniq if use_static else uniq[:u].copy()), rvs, u


class Table:
    """EmbeddingStatic / EmbeddingDynamic key->offset map."""

    def __init__(self, dev_vocab_size, dynamic=False, arena_base=0, row_bytes=0):
        self.h = lib().orc_table_create(dev_vocab_size, int(dynamic), arena_base, row_bytes)

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_table_destroy(self.h)
            self.h = None

    def key2offset(self, keys, channel=0):
        keys = np.ascontiguousarray(keys, dtype=np.int64).copy()
        rc = lib().orc_table_key2offset(self.h, _ptr(keys), keys.size, channel)
        return keys, rc

    def evict(self, keys):
        keys = np.ascontiguousarray(keys, dtype=np.int64)
        return lib().orc_table_evict(self.h, _ptr(keys), keys.size)

    @property
    def size(self):
        return lib().orc_table_size(self.h)

    @property
    def live(self):
        return lib().orc_table_live(self.h)

    @property
    def evict_pos(self):
        n = lib().orc_table_evict_count(self.h)
        out = np.empty(n, dtype=np.int64)
        lib().orc_table_evict_pos(self.h, _ptr(out))
        return out


class Faae:
    """FeatureAdmitAndEvict history of one table."""

    def __init__(self, count_threshold, time_threshold=-1, coef=1, is_enable_sum=True):
        self.h = lib().orc_faae_create(count_threshold, time_threshold, coef, int(is_enable_sum))

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_faae_destroy(self.h)
            self.h = None

    def admit(self, keys, counts, timestamp, channel=0):
        keys = np.ascontiguousarray(keys, dtype=np.int64).copy()
        counts = np.ascontiguousarray(counts, dtype=np.uint32)
        lib().orc_faae_admit(self.h, channel, _ptr(keys), _ptr(counts), keys.size, timestamp)
        return keys

    def evict(self):
        n = lib().orc_faae_size(self.h)
        out = np.empty(max(n, 1), dtype=np.int64)
        k = lib().orc_faae_evict(self.h, _ptr(out), out.size)
        return out[:k].copy()

    def dump(self):
        n = lib().orc_faae_size(self.h)
        keys = np.empty(n, dtype=np.int64)
        counts = np.empty(n, dtype=np.uint32)
        times = np.empty(n, dtype=np.int64)
        lib().orc_faae_dump(self.h, _ptr(keys), _ptr(counts), _ptr(times))
        return keys, counts, times


class Filter:
    """torch FeatureFilter of one table."""

    def __init__(self, admit_threshold=-1, evict_threshold=0, evict_step_interval=1):
        self.h = lib().orc_filter_create(admit_threshold, evict_threshold, evict_step_interval)

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_filter_destroy(self.h)
            self.h = None

    def statistics_key_count(self, keys, counts=None):
        keys = np.ascontiguousarray(keys, dtype=np.int64)
        counts = None if counts is None else np.ascontiguousarray(counts, dtype=np.int64)
        lib().orc_filter_statistics(self.h, _ptr(keys), _ptr(counts), keys.size)

    def count_filter(self, keys):
        keys = np.ascontiguousarray(keys, dtype=np.int64).copy()
        lib().orc_filter_count_filter(self.h, _ptr(keys), keys.size)
        return keys

    def record_timestamp(self, keys, timestamps):
        """Returns the evicted keys when this call triggered an eviction, else None."""
        keys = np.ascontiguousarray(keys, dtype=np.int64)
        timestamps = np.ascontiguousarray(timestamps, dtype=np.int64)
        ran = lib().orc_filter_record_timestamp(self.h, _ptr(keys), _ptr(timestamps), keys.size)
        if not ran:
            return None
        out = np.empty(1 << 20, dtype=np.int64)
        n = lib().orc_filter_evicted(self.h, _ptr(out), out.size)
        return out[:n].copy()


class Swap:
    """torch SwapManager."""

    def __init__(self, cache_size, mem_start_offset=0):
        self.h = lib().orc_swap_create(cache_size, mem_start_offset)

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_swap_destroy(self.h)
            self.h = None

    def compute_swap_info(self, keys):
        """Returns (swapout_keys, swapout_offs, swapin_keys, swapin_offs, batch_offs) or raises on 'too small'."""
        keys = np.ascontiguousarray(keys, dtype=np.int64)
        batch = np.empty(keys.size, dtype=np.int64)
        if lib().orc_swap_compute(self.h, _ptr(keys), keys.size, _ptr(batch)) != 0:
            raise RuntimeError("cacheSize_ too small")
        res = []
        for which in range(4):
            buf = np.empty(max(keys.size, 1), dtype=np.int64)
            m = lib().orc_swap_result(self.h, which, _ptr(buf), buf.size)
            res.append(buf[:m].copy())
        return res[0], res[1], res[2], res[3], batch

    def remove_keys(self, keys):
        keys = np.ascontiguousarray(keys, dtype=np.int64)
        lib().orc_swap_remove(self.h, _ptr(keys), keys.size)


def unique_sharded(ids, shards, padding_size=0, padding_val=-1, use_mask=False):
    """AccCTR enhanced unique with sharding.  Returns a dict of the reference's EnhancedUniqueOut fields
    (unique_id, index, unique_id_in_bucket, cnt_in_bucket, id_cnt, id_cnt_fill, unique_id_cnt), or raises
    when a shard overflows padding_size (H_PADDING_SMALL)."""
    ids = np.ascontiguousarray(ids, dtype=np.int64)
    n = ids.size
    m = max(padding_size * shards, n, 1)
    uid = np.empty(m, dtype=np.int64)
    index = np.empty(max(n, 1), dtype=np.uint32)
    inb = np.empty(max(n, 1), dtype=np.int64)
    cib = np.empty(shards, dtype=np.int32)
    idc = np.empty(max(n, 1), dtype=np.int32)
    fill = np.empty(m, dtype=np.int32)
    cnt = lib().orc_unique_sharded(_ptr(ids), n, shards, 1 if use_mask else 0, padding_size, padding_val, _ptr(uid),
                                   _ptr(index), _ptr(inb), _ptr(cib), _ptr(idc), _ptr(fill))
    if cnt < 0:
        raise RuntimeError("padding size too small")
    u = int(cib.sum())
    return {"unique_id": uid[:cnt].copy(), "index": index[:n].copy(), "unique_id_in_bucket": inb[:u].copy(),
            "cnt_in_bucket": cib, "id_cnt": idc[:u].copy(),
            "id_cnt_fill": fill[:cnt].copy() if padding_size > 0 else None, "unique_id_cnt": int(cnt)}


def unique_sorted(ids):
    """hybrid::UniqueParallel: (sorted distinct ids, inverse int64)."""
    ids = np.ascontiguousarray(ids, dtype=np.int64)
    out = np.empty(max(ids.size, 1), dtype=np.int64)
    inv = np.empty(max(ids.size, 1), dtype=np.int64)
    u = lib().orc_unique_sorted(_ptr(ids), ids.size, _ptr(out), _ptr(inv))
    return out[:u].copy(), inv[:ids.size].copy()


class OffsetMapper:
    """AccCTR EmbCache::OffsetMapper (HBM-cache planner of the TF path)."""

    def __init__(self, max_cache_size):
        self.h = lib().orc_om_create(max_cache_size)

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_om_destroy(self.h)
            self.h = None

    def get_swap_pairs_and_key2offset(self, keys):
        """Returns (offsets, swapin_keys, swapin_pos, swapout_keys, swapout_pos); raises on 'cache too small'."""
        keys = np.array(keys, dtype=np.int64)
        if lib().orc_om_compute(self.h, _ptr(keys), keys.size) != 0:
            raise RuntimeError("max cache size too small")
        res = []
        for which in range(4):
            buf = np.empty(max(keys.size, 1), dtype=np.int64)
            m = lib().orc_om_result(self.h, which, _ptr(buf), buf.size)
            res.append(buf[:m].copy())
        return keys, res[0], res[1], res[2], res[3]

    def remove(self, keys):
        keys = np.ascontiguousarray(keys, dtype=np.int64)
        lib().orc_om_remove(self.h, _ptr(keys), keys.size)

    def state(self):
        st = np.zeros(3, dtype=np.int64)
        lib().orc_om_state(self.h, _ptr(st), None, None)
        k = np.empty(max(int(st[2]), 1), dtype=np.int64)
        v = np.empty(max(int(st[2]), 1), dtype=np.int64)
        lib().orc_om_state(self.h, _ptr(st), _ptr(k), _ptr(v))
        return {"use_length": int(st[0]), "evict_size": int(st[1]), "keys": k[:st[2]].copy(), "slots": v[:st[2]].copy()}


INIT_CONSTANT, INIT_RANDOM_NORMAL, INIT_TRUNCATED_NORMAL = 0, 1, 2


class Initializer:
    """A list of row initializers (AccCTR InitializerInfo): descs = [(kind, start, len, value_or_mean, stddev, seed,
    init_k), ...]; generate(rows, ext_dim) fills consecutive rows, the generators keep their state."""

    def __init__(self, descs):
        ints = np.array([[d[0], d[1], d[2], d[5]] for d in descs], dtype=np.int64).reshape(-1)
        floats = np.array([[d[3], d[4], d[6]] for d in descs], dtype=np.float32).reshape(-1)
        self.h = lib().orc_init_create(_ptr(ints), _ptr(floats), len(descs))

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_init_destroy(self.h)
            self.h = None

    def generate(self, rows, ext_dim, fill=0.0):
        out = np.full((rows, ext_dim), fill, dtype=np.float32)
        lib().orc_init_generate(self.h, _ptr(out), rows, ext_dim)
        return out


def minstd_rand0(seed, n):
    out = np.empty(n, dtype=np.uint32)
    lib().orc_minstd_rand0(seed, n, _ptr(out))
    return out


def std_normal(seed, mean, stddev, n):
    """n values of std::normal_distribution<float>(mean, stddev) over std::default_random_engine(seed), drawn from the
    std classes themselves"""
    out = np.empty(n, dtype=np.float32)
    fn = lib().orc_std_normal
    fn.restype = None
    fn.argtypes = [ctypes.c_uint32, ctypes.c_float, ctypes.c_float, ctypes.c_int64, ctypes.c_void_p]
    fn(int(seed), float(mean), float(stddev), int(n), _ptr(out))
    return out


class HostRows:
    """EmbLocalTable (AccCTR emb_local_table.cpp:106-335) with the single-refill-thread pool order: the j-th row ever
    created gets the j-th row of the initializer stream.  Pure Python over the initializer above (small cases)."""

    def __init__(self, vocab_size, ext_dim, descs):
        self.vocab = vocab_size
        self.ext = ext_dim
        self.init = Initializer(descs)
        self.rows = {}

    def _row(self, key):
        key = int(key)
        if key not in self.rows:
            if len(self.rows) >= self.vocab:
                raise RuntimeError("host vocab size too small")
            self.rows[key] = self.init.generate(1, self.ext)[0]
        return self.rows[key]

    def gather(self, keys):
        return np.stack([self._row(k).copy() for k in keys]) if len(keys) else np.zeros((0, self.ext), np.float32)

    def scatter(self, keys, src):
        for k, r in zip(keys, src):
            self._row(k)[:] = r

    def gather_and_remove(self, keys):
        out = []
        for k in keys:
            k = int(k)
            if k in self.rows:
                out.append(self.rows.pop(k))
            else:
                out.append(self.init.generate(1, self.ext)[0])
        return np.stack(out) if out else np.zeros((0, self.ext), np.float32)

    def remove(self, keys):
        for k in keys:
            self.rows.pop(int(k), None)

    def export(self):
        ks = sorted(self.rows)
        return np.array(ks, dtype=np.int64), (np.stack([self.rows[k] for k in ks]) if ks
                                              else np.zeros((0, self.ext), np.float32))

    def serialize(self):
        """EmbLocalTable::Serialize, emb_local_table.cpp:361-376: per key [key u64][ext floats]; ascending key here."""
        out = bytearray()
        for k in sorted(self.rows):
            out += np.array([k], dtype=np.int64).view(np.uint64).tobytes() + self.rows[k].astype(np.float32).tobytes()
        return bytes(out)

    def deserialize(self, data):
        """EmbLocalTable::Deserialize, emb_local_table.cpp:379-402; returns False on a cut record ("get data failed")."""
        i = 0
        while i < len(data):
            if i + 8 > len(data):
                return False
            key = int(np.frombuffer(data[i:i + 8], dtype=np.uint64)[0].astype(np.int64))
            i += 8
            row = self._row(key)     # FindAndPutIfNotFound
            for j in range(self.ext):
                if i + 4 > len(data):
                    return False
                row[j] = np.frombuffer(data[i:i + 4], dtype=np.float32)[0]
                i += 4
        return True

    def torch_files(self, emb_dim, optim_num):
        """EmbcacheManager::Save + WriteAttributeFile, embcache_manager.cpp:342-458, for one table: relative file
        name -> bytes; a row is [embedding | momentum1 | momentum2], keys ascending."""
        ks = sorted(self.rows)
        count = len(ks)
        files = {"key/slice.data": np.array(ks, dtype=np.int64).tobytes(),
                 "key/slice.attribute": np.array([8, count], dtype=np.int64).tobytes()}
        parts = [("embedding", 0)]
        if optim_num > 0:
            parts.append(("momentum1", emb_dim))
        if optim_num > 1:
            parts.append(("momentum2", optim_num * emb_dim))
        for name, at in parts:
            files[name + "/slice.data"] = b"".join(self.rows[k][at:at + emb_dim].astype(np.float32).tobytes() for k in ks)
            files[name + "/slice.attribute"] = np.array([4, count, emb_dim], dtype=np.int64).tobytes()
        return files

    def torch_load(self, files, emb_dim, optim_num):
        """EmbcacheManager::Load -> InsertOrAssign, embcache_manager.cpp:460-527."""
        keys = np.frombuffer(files["key/slice.data"], dtype=np.int64)
        names = ["embedding", "momentum1", "momentum2"][:optim_num + 1]
        mats = [np.frombuffer(files[n + "/slice.data"], dtype=np.float32).reshape(keys.size, emb_dim) for n in names]
        for i, k in enumerate(keys):
            row = self._row(k)
            for p, m in enumerate(mats):
                row[p * emb_dim:(p + 1) * emb_dim] = m[i]


# ---- checkpoint files of the device tables ------------------------------------------------------------------------

def ckpt_filter_keys(file_keys, rank_id, rank_size, is_dp):
    """EmbeddingStatic::LoadKey / EmbeddingDynamic::LoadKey, embedding_static.cpp:216-225: (kept keys, loadOffset).
    The test is C++'s `key % rankSize != rankId` (remainder takes the sign of the key)."""
    file_keys = np.ascontiguousarray(file_keys, dtype=np.int64)
    keys, load_offset = [], []
    for i, k in enumerate(file_keys.tolist()):
        rem = abs(k) % rank_size
        rem = -rem if k < 0 else rem
        if not is_dp and rem != rank_id:
            continue
        keys.append(k)
        load_offset.append(i)
    return np.array(keys, dtype=np.int64), np.array(load_offset, dtype=np.int64)


def ckpt_static_load(file_keys, rank_id, rank_size, is_dp):
    """keyOffsetMap after EmbeddingStatic::LoadKey on a fresh table: kept key j -> offset j."""
    keys, load_offset = ckpt_filter_keys(file_keys, rank_id, rank_size, is_dp)
    return {int(k): j for j, k in enumerate(keys)}, load_offset


def ckpt_row_file(rows, emb_size, at=0):
    """LocalFileSystem::WriteEmbedding, local_file_system.cpp:165-224: embSize floats per address, back to back."""
    rows = np.ascontiguousarray(rows, dtype=np.float32)
    return rows[:, at:at + emb_size].astype(np.float32).tobytes()


def ckpt_read_rows(file_bytes, load_offset, emb_size, ext_emb_size, out):
    """LocalFileSystem::ReadEmbedding, local_file_system.cpp:317-381: file row loadOffset[i] -> out[i, :embSize]
    (out is [n, extEmbSize] starting at firstAddress)."""
    mat = np.frombuffer(file_bytes, dtype=np.float32).reshape(-1, emb_size)
    load_offset = np.asarray(load_offset, dtype=np.int64)
    out[:load_offset.size, :emb_size] = mat[load_offset]
    return out


def history_record(table_timestamp, keys, counts, last_times):
    """FeatAdmitNEvictCkpt::SetHistRecTrans, feat_admit_n_evict_ckpt.cpp:112-131: int64 [timestamp, (featureId, count,
    lastTime)*]."""
    out = [int(table_timestamp)]
    for k, c, t in zip(keys, counts, last_times):
        out += [int(k), int(c), int(t)]
    return np.array(out, dtype=np.int64)


def lookup_by_addr(address, dim, out_dtype=np.float32):
    address = np.ascontiguousarray(address, dtype=np.int64)
    y = np.empty((address.size, dim), dtype=out_dtype)
    lib().orc_lookup_by_addr(_ptr(address), address.size, dim, y.dtype.itemsize, _ptr(y))
    return y


def update_by_addr(address, emb, update_type):
    address = np.ascontiguousarray(address, dtype=np.int64)
    emb = np.ascontiguousarray(emb, dtype=np.float32)
    lib().orc_update_by_addr_f32(_ptr(address), address.size, emb.shape[1], _ptr(emb), update_type)


def lazy_adam(grad, indices, m, v, var, lr, beta1, beta2, eps):
    """In place on m, v, var (float32 C-contiguous [rows, dim])."""
    grad = np.ascontiguousarray(grad, dtype=np.float32)
    indices = np.ascontiguousarray(indices, dtype=np.int32)
    lib().orc_lazy_adam(_ptr(grad), _ptr(indices), indices.size, grad.shape[1], _ptr(m), _ptr(v), _ptr(var), lr, beta1,
                        beta2, eps)


def sgd(grad, indices, var, lr, weight_decay=0.0):
    grad = np.ascontiguousarray(grad, dtype=np.float32)
    indices = np.ascontiguousarray(indices, dtype=np.int32)
    lib().orc_sgd(_ptr(grad), _ptr(indices), indices.size, grad.shape[1], _ptr(var), lr, weight_decay)


def segment_sum(grad, seg, num_seg):
    grad = np.ascontiguousarray(grad, dtype=np.float32)
    seg = np.ascontiguousarray(seg, dtype=np.int32)
    out = np.empty((num_seg, grad.shape[1]), dtype=np.float32)
    lib().orc_segment_sum(_ptr(grad), _ptr(seg), seg.size, grad.shape[1], num_seg, _ptr(out))
    return out


def byaddr_apply(optim, g, slots, w, s1, s2, stride, lr_t, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0,
                 delta_form=True):
    """In place on w/s1/s2 (numpy float32 buffers sharing one row stride, in elements)."""
    g = np.ascontiguousarray(g, dtype=np.float32)
    slots = np.ascontiguousarray(slots, dtype=np.int64)
    lib().orc_byaddr_apply(optim, _ptr(g), _ptr(slots), slots.size, g.shape[1], _ptr(w), _ptr(s1), _ptr(s2), stride,
                           lr_t, beta1, beta2, eps, weight_decay, int(delta_form))


def gather_rows(w, stride, slots, dim):
    slots = np.ascontiguousarray(slots, dtype=np.int64)
    out = np.empty((slots.size, dim), dtype=np.float32)
    lib().orc_gather_rows(_ptr(w), stride, _ptr(slots), slots.size, dim, _ptr(out))
    return out


def tbe_forward(dev_weights, weights_offsets, d_offsets, total_d, indices, offsets, T, B, pooling_mode, bf16=False):
    weights_offsets = np.ascontiguousarray(weights_offsets, dtype=np.int64)
    d_offsets = np.ascontiguousarray(d_offsets, dtype=np.int32)
    indices = np.ascontiguousarray(indices, dtype=np.int64)
    offsets = np.ascontiguousarray(offsets, dtype=np.int64)
    if pooling_mode == 2:
        out = np.empty((indices.size, total_d // T), dtype=np.float32)
    else:
        out = np.empty((B, total_d), dtype=np.float32)
    lib().orc_tbe_forward(_ptr(dev_weights), int(bf16), _ptr(weights_offsets), _ptr(d_offsets), total_d, _ptr(indices),
                          _ptr(offsets), T, B, pooling_mode, _ptr(out))
    return out


def tbe_backward(optim, grad_output, dev_weights, weights_offsets, d_offsets, total_d, hash_size_cumsum, indices,
                 offsets, T, B, pooling_mode, momentum1, momentum2, lr, eps=1e-8, beta1=0.9, beta2=0.999, it=1,
                 bf16=False):
    """In place on dev_weights / momentum1 / momentum2."""
    grad_output = np.ascontiguousarray(grad_output, dtype=np.float32)
    weights_offsets = np.ascontiguousarray(weights_offsets, dtype=np.int64)
    d_offsets = np.ascontiguousarray(d_offsets, dtype=np.int32)
    hash_size_cumsum = np.ascontiguousarray(hash_size_cumsum, dtype=np.int64)
    indices = np.ascontiguousarray(indices, dtype=np.int64)
    offsets = np.ascontiguousarray(offsets, dtype=np.int64)
    lib().orc_tbe_backward(optim, _ptr(grad_output), _ptr(dev_weights), int(bf16), _ptr(weights_offsets),
                           _ptr(d_offsets), total_d, _ptr(hash_size_cumsum), _ptr(indices), _ptr(offsets), T, B,
                           pooling_mode, _ptr(momentum1), _ptr(momentum2), lr, eps, beta1, beta2, it)


def tbe_backward_unique(optim, grad_output, dev_weights, weights_offsets, d_offsets, total_d, offsets, T, B,
                        pooling_mode, unique_ids, unique_offsets, unique_inverse, momentum1, momentum2, lr, eps=1e-8,
                        beta1=0.9, beta2=0.999, it=1, bf16=False):
    """The unique variant (the caller brings the distinct rows and the inverse index).  In place."""
    grad_output = np.ascontiguousarray(grad_output, dtype=np.float32)
    weights_offsets = np.ascontiguousarray(weights_offsets, dtype=np.int64)
    d_offsets = np.ascontiguousarray(d_offsets, dtype=np.int32)
    offsets = np.ascontiguousarray(offsets, dtype=np.int64)
    unique_ids = np.ascontiguousarray(unique_ids, dtype=np.int64)
    unique_offsets = np.ascontiguousarray(unique_offsets, dtype=np.int64)
    unique_inverse = np.ascontiguousarray(unique_inverse, dtype=np.int64)
    assert unique_offsets.size == T + 1 and unique_ids.size >= unique_offsets[T]
    lib().orc_tbe_backward_unique(optim, _ptr(grad_output), _ptr(dev_weights), int(bf16), _ptr(weights_offsets),
                                  _ptr(d_offsets), total_d, _ptr(offsets), T, B, pooling_mode, _ptr(unique_ids),
                                  _ptr(unique_offsets), _ptr(unique_inverse), _ptr(momentum1), _ptr(momentum2), lr,
                                  eps, beta1, beta2, it)
