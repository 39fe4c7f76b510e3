"""Host-side mirror of the reference's interfaces for the sparse-embedding hot path, over the C ABI.

Class and method names follow the reference so that tests read like the reference's own:
  KeyProcess.hash_split / global_unique        training/tf_rec_v1/src/core/key_process/key_process.{h,cpp}
  EmbeddingTables.key2offset / evict_keys      training/tf_rec_v1/src/core/emb_table/embedding_{static,dynamic,table}.cpp
  embedding_lookup_by_address / ..._update_... cust_op/framework/tf_plugin/src/cust_embedding_by_address.cpp
  lazy_adam / sgd                              cust_op/framework/tf_plugin/src/{lazy_adam,sgd}.cpp
torch is used for device memory and streams only; all compute goes through librecsdk_hip.so.
"""
import ctypes
from ctypes import c_int32, c_int64, c_void_p

import numpy as np
import torch

from . import capi
from .capi import check, lib

_TORCH_TO_DT = {torch.float32: capi.DT_F32, torch.float16: capi.DT_F16, torch.int32: capi.DT_I32,
                torch.bfloat16: capi.DT_BF16}


def _stream():
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "device pointers must come from contiguous CUDA tensors"
    return c_void_p(t.data_ptr())


# ---- by-address ops (TF custom-op surface) --------------------------------------------------------

def embedding_lookup_by_address(address, embedding_dim, embedding_type=torch.float32):
    """y[i, :] = row at device address[i]; address 0 gives a zero row."""
    n = address.numel()
    y = torch.empty((n, embedding_dim), dtype=embedding_type, device=address.device)
    check(lib().recsdk_lookup_by_addr(_p(address), n, embedding_dim, _TORCH_TO_DT[embedding_type], _p(y), _stream()))
    return y


def embedding_update_by_address(address, embedding, update_type=0):
    """row at address[i] += embedding[i, :] (update_type 0, atomic) or = embedding[i, :] (update_type 1)."""
    n, dim = embedding.shape
    check(lib().recsdk_update_by_addr(_p(address), n, dim, _TORCH_TO_DT[embedding.dtype], _p(embedding), update_type,
                                      _stream()))


def lazy_adam(gradient, indices, input_m, input_v, input_var, lr, beta1, beta2, epsilon):
    n, dim = gradient.shape
    check(lib().recsdk_lazy_adam(_p(gradient), _p(indices), n, dim, _p(input_m), _p(input_v), _p(input_var), lr, beta1,
                                 beta2, epsilon, _stream()))
    return input_m, input_v, input_var


def sgd(gradient, indices, input_var, lr, weight_decay=0.0):
    n, dim = gradient.shape
    check(lib().recsdk_sgd(_p(gradient), _p(indices), n, dim, _p(input_var), lr, weight_decay, _stream()))
    return input_var


# ---- batch ingestion ------------------------------------------------------------------------------------

def read_emb_key(sample, splits, table_used=None, is_timestamp=False, field_num=None):
    """ReadEmbKeyV2: one int32/int64 device tensor [timestamp?][table 0 keys][table 1 keys]... -> (keys int64 [n],
    offsets int64 [used+1] on the device, offsets as numpy, timestamp or -1).  field_num defaults to sum(splits)."""
    splits = np.ascontiguousarray(splits, dtype=np.int64)
    used = None if table_used is None else np.ascontiguousarray(table_used, dtype=np.uint8)
    n_used = splits.size if used is None else int(np.count_nonzero(used))
    total = int(splits.sum() if used is None else splits[used != 0].sum())
    keys = torch.empty(max(total, 1), dtype=torch.int64, device=sample.device)
    d_off = torch.empty(n_used + 1, dtype=torch.int64, device=sample.device)
    h_off = np.zeros(n_used + 1, dtype=np.int64)
    ts = c_int64(-1)
    dt = {torch.int32: capi.DT_I32, torch.int64: capi.DT_I64}.get(sample.dtype, -1)
    check(lib().recsdk_read_emb_key(_p(sample), dt, sample.numel(), splits.ctypes.data_as(c_void_p),
                                    None if used is None else used.ctypes.data_as(c_void_p), splits.size,
                                    1 if is_timestamp else 0, int(splits.sum()) if field_num is None else field_num,
                                    _p(keys), _p(d_off), h_off.ctypes.data_as(c_void_p), ctypes.byref(ts), _stream()))
    return keys[:total], d_off, h_off, ts.value


def padding_keys_mask(values, padding_keys):
    """PushPaddingKeysTensors: int32 mask, 0 where values[i] is one of padding_keys, else 1."""
    pad = np.ascontiguousarray(padding_keys, dtype=np.int64)
    mask = torch.empty(max(values.numel(), 1), dtype=torch.int32, device=values.device)
    check(lib().recsdk_padding_keys_mask(_p(values), values.numel(), pad.ctypes.data_as(c_void_p), pad.size, _p(mask),
                                         _stream()))
    return mask[:values.numel()]


_ONE_TABLE_OFFSETS = {}


def _one_table_offsets(n, device):
    """The offsets [0, n] of a one-table batch as a device tensor.  Kept per (n, device): building it is two small
    host-to-device copies, a tenth of a millisecond in front of every call otherwise.  Read-only for every user."""
    key = (int(n), str(device))
    t = _ONE_TABLE_OFFSETS.get(key)
    if t is None:
        if len(_ONE_TABLE_OFFSETS) >= 64:
            _ONE_TABLE_OFFSETS.clear()
        t = torch.tensor([0, int(n)], dtype=torch.int64, device=device)
        _ONE_TABLE_OFFSETS[key] = t
    return t


GRAPH_NODE_KINDS = {0: "kernel", 1: "memcpy", 2: "memset", 3: "host", 4: "graph", 5: "empty", 6: "wait_event",
                    7: "event_record", 8: "semaphore_signal", 9: "semaphore_wait", 10: "mem_alloc", 11: "mem_free",
                    12: "memcpy_from_symbol", 13: "memcpy_to_symbol"}


def graph_node_kinds(raw_graph):
    """Names of the node types of a captured HIP graph (torch.cuda.CUDAGraph(keep_graph=True).raw_cuda_graph())."""
    count = c_int64()
    check(lib().recsdk_graph_node_kinds(c_void_p(int(raw_graph)), None, 0, ctypes.byref(count)))
    kinds = (c_int32 * max(count.value, 1))()
    check(lib().recsdk_graph_node_kinds(c_void_p(int(raw_graph)), kinds, count.value, ctypes.byref(count)))
    return [GRAPH_NODE_KINDS.get(int(k), str(int(k))) for k in kinds[:count.value]]


# ---- radix sort ---------------------------------------------------------------------------------------

class Sorter:
    """Stable radix sort of (key, uint32 value) pairs on the device (workspace handle); keys int32/uint32 or
    int64/uint64 tensors holding non-negative values below 2**bits."""

    def __init__(self, max_pairs, key_bytes=4):
        self.h = c_void_p()
        self.key_bytes = key_bytes
        check(lib().recsdk_sorter_create(int(max_pairs), key_bytes, ctypes.byref(self.h)))

    def close(self):
        if self.h:
            lib().recsdk_sorter_destroy(self.h)
            self.h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def sort_pairs(self, keys, values, bits, descending=False):
        """-> (sorted keys, values in the same order); inputs are left as they are"""
        import torch
        assert keys.element_size() == self.key_bytes and values.element_size() == 4
        keys_out, values_out = torch.empty_like(keys), torch.empty_like(values)
        check(lib().recsdk_sort_pairs(self.h, _p(keys), _p(keys_out), _p(values), _p(values_out), keys.numel(), int(bits),
                                      1 if descending else 0, _stream()))
        return keys_out, values_out


# ---- dedup ------------------------------------------------------------------------------------------

class Unique:
    """Multi-table first-occurrence dedup (workspace handle)."""

    def __init__(self, max_keys, max_tables=1, position_lists=True, early_counts=True, max_table_keys=0):
        """early_counts=False: counts arrive with the position lists (KeyProcess::HashSplit has none at all)."""
        self.h = c_void_p()
        check(lib().recsdk_unique_create(max_keys, max_tables, ctypes.byref(self.h)))
        if not position_lists:
            check(lib().recsdk_unique_set_lists(self.h, 0))
        if not early_counts:
            check(lib().recsdk_unique_set_counts(self.h, 0))
        if max_table_keys:
            check(lib().recsdk_unique_set_max_table_keys(self.h, int(max_table_keys)))
        self.n = 0
        self.T = 0
        self._keep = None

    def close(self):
        if self.h:
            lib().recsdk_unique_destroy(self.h)
            self.h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def run(self, keys, offsets, in_counts=None, skip_key=None):
        """keys: int64 [n] device; offsets: int64 [T+1] device (table t = keys[offsets[t]:offsets[t+1]])."""
        self.n = keys.numel()
        self.T = offsets.numel() - 1
        self._keep = (keys, offsets, in_counts)  # inputs are read by later kernels (gather / apply)
        check(lib().recsdk_unique_run(self.h, _p(keys), _p(in_counts), _p(offsets), self.T, self.n,
                                      0 if skip_key is None else 1, 0 if skip_key is None else int(skip_key),
                                      _stream()))
        return self

    def total(self):
        out = c_int64()
        check(lib().recsdk_unique_total(self.h, _stream(), ctypes.byref(out)))
        return out.value

    def fetch(self):
        """Returns (unique_keys[U], unique_offsets[T+1], inverse[n], counts[U]) as new device tensors."""
        dev = self._keep[0].device
        uk = torch.empty(max(self.n, 1), dtype=torch.int64, device=dev)
        uo = torch.empty(self.T + 1, dtype=torch.int64, device=dev)
        inv = torch.empty(max(self.n, 1), dtype=torch.int32, device=dev)
        cnt = torch.empty(max(self.n, 1), dtype=torch.int32, device=dev)
        check(lib().recsdk_unique_fetch(self.h, _p(uk), _p(uo), _p(inv), _p(cnt), _stream()))
        u = self.total()
        return uk[:u], uo, inv[:self.n], cnt[:u]


def unique_expand(unique, values, fill=-1):
    """values[U] (per distinct key, all tables back to back) -> int64 [n] per key."""
    out = torch.empty(max(unique.n, 1), dtype=torch.int64, device=values.device)
    check(lib().recsdk_unique_expand(unique.h, _p(values), fill, _p(out), _stream()))
    return out[:unique.n]


class KeyProcess:
    """The dedup half of KeyProcess for one rank (rankSize 1)."""

    def __init__(self, max_keys, max_tables=1):
        self.max_keys = max_keys
        self.hot = None
        self.unique = Unique(max_keys, max_tables)

    def hash_split(self, keys, offsets=None):
        """HashSplitWithFAAE with rankSize 1: returns (split_keys, restore, key_count, unique_offsets)."""
        if offsets is None:
            offsets = _one_table_offsets(keys.numel(), keys.device)
        uk, uo, inv, cnt = self.unique.run(keys, offsets).fetch()
        return uk, inv, cnt, uo

    def enable_hot_keys(self, hot_counts, hot_emb_update_step=1000):
        """Turns on hot-key staging: hot_counts[t] = hotEmbTotCount of table t, refresh of the hot sets every
        hot_emb_update_step batches (HOT_EMB_UPDATE_STEP, default 1000)."""
        hc = np.ascontiguousarray(hot_counts, dtype=np.int32)
        self.hot_counts = hc
        self.hot_step = int(hot_emb_update_step)
        self.hot = c_void_p()
        check(lib().recsdk_hot_create(hc.size, hc.ctypes.data_as(c_void_p), self.max_keys, ctypes.byref(self.hot)))

    def close(self):
        if getattr(self, "hot", None):
            lib().recsdk_hot_destroy(self.hot)
            self.hot = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def hot_hash_split(self, keys, batch_id, offsets=None):
        """HotHashSplit with rankSize 1: returns (split_keys, restore, hot_pos, key_count, unique_offsets);
        hot_pos holds the tables' hot_counts[t] entries back to back."""
        if offsets is None:
            offsets = _one_table_offsets(keys.numel(), keys.device)
        uk, uo, _, cnt = self.unique.run(keys, offsets).fetch()
        restore = torch.empty(max(keys.numel(), 1), dtype=torch.int32, device=keys.device)
        hot_pos = torch.empty(max(int(self.hot_counts.sum()), 1), dtype=torch.int32, device=keys.device)
        check(lib().recsdk_hot_split(self.hot, self.unique.h, _p(restore), _p(hot_pos),
                                     1 if batch_id % self.hot_step == 0 else 0, _stream()))
        return uk, restore[:keys.numel()], hot_pos[:int(self.hot_counts.sum())], cnt, uo

    def global_unique(self, lookup_keys, use_static=False, use_dynamic_expansion=False):
        """GlobalUnique: returns (unique_keys, restore_vec_sec); with use_static the padding key is skipped
        and unique_keys is padded to len(lookup_keys) with it."""
        offsets = _one_table_offsets(lookup_keys.numel(), lookup_keys.device)
        pad = 0 if use_dynamic_expansion else -1
        uk, _, inv, _ = self.unique.run(lookup_keys, offsets, skip_key=pad if use_static else None).fetch()
        if use_static:
            full = torch.full((lookup_keys.numel(),), pad, dtype=torch.int64, device=lookup_keys.device)
            full[:uk.numel()] = uk
            uk = full
        return uk, inv


# ---- key -> slot tables --------------------------------------------------------------------------------

class EmbeddingTables:
    """A group of EmbeddingStatic / EmbeddingDynamic key->offset maps living on the device."""

    def __init__(self, dev_vocab_sizes, max_keys, dynamic=None, arena_bases=None, row_bytes=None):
        T = len(dev_vocab_sizes)
        self.T = T
        self.h = c_void_p()
        arr = lambda ct, xs: (ct * T)(*xs) if xs is not None else None
        check(lib().recsdk_tables_create(T, arr(c_int64, dev_vocab_sizes), arr(c_int32, dynamic),
                                         arr(c_int64, arena_bases), arr(c_int64, row_bytes), max_keys,
                                         ctypes.byref(self.h)))

    def close(self):
        if self.h:
            lib().recsdk_tables_destroy(self.h)
            self.h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def key2offset(self, keys, offsets, channel=capi.CHANNEL_TRAIN, n=None):
        """In place on `keys` (distinct per table, -1 allowed)."""
        check(lib().recsdk_tables_key2offset(self.h, _p(keys), _p(offsets), self.T, keys.numel() if n is None else n,
                                             channel, _stream()))
        return keys

    def evict_keys(self, keys, offsets):
        check(lib().recsdk_tables_evict(self.h, _p(keys), _p(offsets), self.T, keys.numel(), _stream()))

    def maintain(self):
        """Rebuilds the maps that evictions (also those replayed from a graph) have filled with erased entries;
        returns the number of tables rebuilt.  Synchronous."""
        rebuilt = c_int32()
        check(lib().recsdk_tables_maintain(self.h, _stream(), ctypes.byref(rebuilt)))
        return rebuilt.value

    def stats(self):
        """Returns (max_offset[T], live[T], evicted[T]); raises RecsdkError(EOVERFLOW) on vocabulary overflow."""
        mo = (c_int64 * self.T)()
        lv = (c_int64 * self.T)()
        ev = (c_int64 * self.T)()
        check(lib().recsdk_tables_stats(self.h, _stream(), mo, lv, ev))
        return list(mo), list(lv), list(ev)

    def evict_pos(self, t, cap=1 << 20):
        out = (c_int64 * cap)()
        cnt = c_int64()
        check(lib().recsdk_tables_evict_pos(self.h, t, _stream(), out, cap, ctypes.byref(cnt)))
        return list(out[:min(cnt.value, cap)])


# ---- rows + fused sparse step ----------------------------------------------------------------------------

class Rows:
    """Where each table's rows live: w / s1 / s2 tensors and a common row stride (elements)."""

    def __init__(self, dim, w, s1=None, s2=None, strides=None):
        T = len(w)
        self.T = T
        self.dim = dim
        self._keep = (w, s1, s2)
        strides = strides if strides is not None else [dim] * T
        pw = (c_void_p * T)(*[t.data_ptr() for t in w])
        ps1 = (c_void_p * T)(*[t.data_ptr() for t in s1]) if s1 is not None else None
        ps2 = (c_void_p * T)(*[t.data_ptr() for t in s2]) if s2 is not None else None
        self.h = c_void_p()
        check(lib().recsdk_rows_create(T, dim, pw, ps1, ps2, (c_int64 * T)(*strides), ctypes.byref(self.h)))

    def close(self):
        if self.h:
            lib().recsdk_rows_destroy(self.h)
            self.h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def gather_unique(rows, unique, slots, out=None):
    if out is None:
        out = torch.empty((unique.n, rows.dim), dtype=torch.float32, device=slots.device)
    check(lib().recsdk_gather_unique(rows.h, unique.h, _p(slots), _p(out), _stream()))
    return out


def sparse_apply(rows, unique, slots, grad, optim, lr, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0):
    """lr: a float, or a one-element float32 device tensor that the kernels read when they run (a step recorded into a
    HIP graph takes the rate of each replay from there)"""
    if isinstance(lr, torch.Tensor):
        check(lib().recsdk_sparse_apply_lr_dev(rows.h, unique.h, _p(slots), _p(grad), optim, _p(lr), beta1, beta2, eps,
                                               weight_decay, _stream()))
        return
    check(lib().recsdk_sparse_apply(rows.h, unique.h, _p(slots), _p(grad), optim, lr, beta1, beta2, eps, weight_decay,
                                    _stream()))


# ---- split-embedding (fbgemm schema) ops -------------------------------------------------------------------

def split_embedding_codegen_forward_unweighted(dev_weights, weights_offsets, D_offsets, total_D, max_D, indices,
                                               offsets, pooling_mode):
    """Pooled lookup; arguments as fbgemm::split_embedding_codegen_forward_unweighted_cuda (unused ones omitted)."""
    T = weights_offsets.numel()
    B = (offsets.numel() - 1) // T
    nnz = indices.numel()
    if pooling_mode == capi.POOL_NONE:
        out = torch.empty((nnz, total_D // T), dtype=torch.float32, device=indices.device)
    else:
        out = torch.empty((B, total_D), dtype=torch.float32, device=indices.device)
    dt = capi.DT_BF16 if dev_weights.dtype == torch.bfloat16 else capi.DT_F32
    check(lib().recsdk_tbe_forward(_p(dev_weights), dt, dev_weights.numel(), _p(weights_offsets), _p(D_offsets),
                                   total_D, max_D, _p(indices), _p(offsets), T, B, nnz, pooling_mode, _p(out),
                                   _stream()))
    return out


class SplitEmbeddingBackward:
    """Workspace + entry point of split_embedding_backward_codegen_{sgd,adagrad,adam}_unweighted_exact."""

    def __init__(self, max_tables, max_nnz):
        self.h = c_void_p()
        check(lib().recsdk_tbe_create(max_tables, max_nnz, ctypes.byref(self.h)))

    def close(self):
        if self.h:
            lib().recsdk_tbe_destroy(self.h)
            self.h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __call__(self, optim, grad_output, dev_weights, weights_offsets, D_offsets, total_D, max_D, hash_size_cumsum,
                 indices, offsets, pooling_mode, momentum1=None, momentum2=None, learning_rate=0.01, eps=1e-8,
                 beta1=0.9, beta2=0.999, iter=1, hash_indices=None, unique_ids=None, unique_offsets=None,
                 unique_inverse=None):
        """hash_indices (when given) replaces indices; unique_ids / unique_offsets / unique_inverse (when given) select
        the unique variant, as in the reference's operators."""
        T = weights_offsets.numel()
        B = (offsets.numel() - 1) // T
        dt = capi.DT_BF16 if dev_weights.dtype == torch.bfloat16 else capi.DT_F32
        if hash_indices is not None and hash_indices.numel() > 0:
            indices = hash_indices
        if unique_ids is not None and unique_ids.numel() > 0:
            check(lib().recsdk_tbe_backward_unique(self.h, optim, _p(grad_output), _p(dev_weights), dt,
                                                   _p(weights_offsets), _p(D_offsets), total_D, max_D,
                                                   _p(hash_size_cumsum), _p(offsets), T, B, unique_inverse.numel(),
                                                   pooling_mode, _p(unique_ids), _p(unique_offsets),
                                                   _p(unique_inverse), unique_ids.numel(), _p(momentum1),
                                                   _p(momentum2), learning_rate, eps, beta1, beta2, iter, _stream()))
            return
        check(lib().recsdk_tbe_backward(self.h, optim, _p(grad_output), _p(dev_weights), dt, _p(weights_offsets),
                                        _p(D_offsets), total_D, max_D, _p(hash_size_cumsum), _p(indices), _p(offsets),
                                        T, B, indices.numel(), pooling_mode, _p(momentum1), _p(momentum2),
                                        learning_rate, eps, beta1, beta2, iter, _stream()))


# ---- feature admission / eviction -----------------------------------------------------------------------------

class FeatureAdmitAndEvict:
    """Device-resident admission/eviction history of T tables (ThresholdValue per table)."""

    def __init__(self, capacities, count_thresholds, time_thresholds=None, coefs=None, enable_sum=None,
                 max_keys=1 << 20):
        T = len(capacities)
        self.T = T
        self.max_keys = max_keys
        arr = lambda ct, xs: (ct * T)(*xs) if xs is not None else None
        self.h = c_void_p()
        check(lib().recsdk_faae_create(T, arr(c_int64, capacities), arr(c_int32, count_thresholds),
                                       arr(c_int32, time_thresholds), arr(c_int32, coefs),
                                       arr(c_int32, [int(x) for x in enable_sum] if enable_sum is not None else None),
                                       max_keys, ctypes.byref(self.h)))

    def close(self):
        if self.h:
            lib().recsdk_faae_destroy(self.h)
            self.h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def feature_admit(self, channel, keys, counts, offsets, timestamps, distinct=False):
        """In place on keys; counts int32/uint32 per occurrence; timestamps: one per table (host ints).  distinct:
        the keys are distinct inside each table already (a unique run's output), no merge pass is needed."""
        ts = (c_int64 * self.T)(*timestamps)
        fn = lib().recsdk_faae_admit_distinct if distinct else lib().recsdk_faae_admit
        check(fn(self.h, channel, _p(keys), _p(counts), _p(offsets), self.T, keys.numel(), ts, _stream()))
        return keys

    def statistics_key_count(self, keys, counts, offsets):
        check(lib().recsdk_faae_count_add(self.h, _p(keys), _p(counts), _p(offsets), self.T, keys.numel(), _stream()))

    def count_filter(self, keys, offsets):
        check(lib().recsdk_faae_count_filter(self.h, _p(keys), _p(offsets), self.T, keys.numel(), _stream()))
        return keys

    def record_timestamp(self, keys, timestamps, offsets):
        check(lib().recsdk_faae_record_timestamp(self.h, _p(keys), _p(timestamps), _p(offsets), self.T, keys.numel(),
                                                 _stream()))

    def feature_evict(self, strict=False, cap=None, device="cuda:0"):
        """Returns (evicted_keys tensor, offsets list[T+1])."""
        cap = cap if cap is not None else self.max_keys
        out = torch.empty(max(cap, 1), dtype=torch.int64, device=device)
        offs = (c_int64 * (self.T + 1))()
        check(lib().recsdk_faae_evict(self.h, int(strict), _p(out), cap, offs, _stream()))
        offs = list(offs)
        return out[:offs[-1]], offs

    def stats(self):
        live = (c_int64 * self.T)()
        latest = (c_int64 * self.T)()
        check(lib().recsdk_faae_stats(self.h, _stream(), live, latest))
        return list(live), list(latest)

    def dump(self, t, cap=1 << 20, device="cuda:0"):
        """Records of table t sorted by key: (keys, counts, times) numpy arrays."""
        k = torch.empty(cap, dtype=torch.int64, device=device)
        c = torch.empty(cap, dtype=torch.int32, device=device)
        ts = torch.empty(cap, dtype=torch.int64, device=device)
        n = c_int64()
        check(lib().recsdk_faae_dump(self.h, t, _p(k), _p(c), _p(ts), cap, ctypes.byref(n), _stream()))
        m = min(n.value, cap)
        kk = k[:m].cpu().numpy()
        order = kk.argsort(kind="stable")
        return kk[order], c[:m].cpu().numpy().view("uint32")[order], ts[:m].cpu().numpy()[order]


# ---- torch-side key mapping and HBM-cache planning ----------------------------------------------------------------

class IdsMapper:
    """hybrid::IdsMapper for T tables (hybrid_torchrec/src/ids_process/ids_mapper.cpp:176-285): ids get dense indices
    in first-seen order per table; returns per-table unique / inverse like ParallelUniqueHashOut."""

    def __init__(self, init_max_index, max_keys):
        self.T = len(init_max_index)
        self.unique = Unique(max_keys, self.T, position_lists=False)
        self.tables = EmbeddingTables(list(init_max_index), max_keys)

    def parallel_unique_hash_out(self, global_ids, offsets):
        """Returns (hash_indices[n], unique[U], unique_ids[U], unique_inverse[n], unique_offset[T+1])."""
        unique_ids, unique_offset, inverse, _ = self.unique.run(global_ids, offsets).fetch()
        unique = unique_ids.clone()
        self.tables.key2offset(unique, unique_offset, capi.CHANNEL_TRAIN)
        hash_indices = unique_expand(self.unique, unique)
        return hash_indices, unique, unique_ids, inverse.to(torch.int64), unique_offset

    def max_index(self):
        """Raises RecsdkError(EOVERFLOW) when a table reached its init_max_index ("Ids map reached maxIndex")."""
        return self.tables.stats()[0]


class SwapManager:
    """Embcache::SwapManager on the device."""

    def __init__(self, cache_size, mem_start_offset=0, max_keys=1 << 20):
        self.max_keys = max_keys
        self.h = c_void_p()
        check(lib().recsdk_swap_create(cache_size, mem_start_offset, max_keys, ctypes.byref(self.h)))

    def close(self):
        if self.h:
            lib().recsdk_swap_destroy(self.h)
            self.h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def compute_swap_info(self, keys):
        """Returns (swapout_keys, swapout_offs, swapin_keys, swapin_offs, batch_offs) device tensors."""
        n = keys.numel()
        dev = keys.device
        bufs = [torch.empty(max(n, 1), dtype=torch.int64, device=dev) for _ in range(5)]
        check(lib().recsdk_swap_compute(self.h, _p(keys), n, *[_p(b) for b in bufs], _stream()))
        so, si, _ = self.counts()
        return bufs[0][:so], bufs[1][:so], bufs[2][:si], bufs[3][:si], bufs[4][:n]

    def counts(self):
        a, b, c = c_int64(), c_int64(), c_int64()
        check(lib().recsdk_swap_counts(self.h, _stream(), ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)))
        return a.value, b.value, c.value

    def remove_keys(self, keys):
        check(lib().recsdk_swap_remove(self.h, _p(keys), keys.numel(), _stream()))


class OffsetMapper:
    """EmbCache::OffsetMapper on the device (AccCTR offset_mapper.h:36-325): one table's HBM-cache planner."""

    def __init__(self, max_cache_size, max_keys=1 << 20):
        self.max_cache_size = max_cache_size
        self.h = c_void_p()
        check(lib().recsdk_om_create(max_cache_size, max_keys, ctypes.byref(self.h)))

    def close(self):
        if self.h:
            lib().recsdk_om_destroy(self.h)
            self.h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def get_swap_pairs_and_key2offset(self, keys):
        """keys (int64 device, distinct apart from -1) become slots IN PLACE.
        Returns (swapin_keys, swapin_pos, swapout_keys, swapout_pos) device tensors."""
        n = keys.numel()
        bufs = [torch.empty(max(n, 1), dtype=torch.int64, device=keys.device) for _ in range(4)]
        check(lib().recsdk_om_compute(self.h, _p(keys), n, *[_p(b) for b in bufs], _stream()))
        si, so, _, _ = self.counts()
        return bufs[0][:si], bufs[1][:si], bufs[2][:so], bufs[3][:so]

    def counts(self):
        """(swap-ins, swap-outs of the last call, slots ever used, freed slots waiting); raises RecsdkError when the
        last call did not fit the cache."""
        v = [c_int64() for _ in range(4)]
        check(lib().recsdk_om_counts(self.h, _stream(), *[ctypes.byref(x) for x in v]))
        return tuple(x.value for x in v)

    def remove(self, keys):
        check(lib().recsdk_om_remove(self.h, _p(keys), keys.numel(), _stream()))

    def export_sorted_kv_pairs(self):
        """(keys, slots) of the cached keys in slot order."""
        buf = torch.empty(self.max_cache_size, dtype=torch.int64, device="cuda")
        check(lib().recsdk_om_export(self.h, _p(buf), _stream()))
        slots = torch.nonzero(buf != -1).flatten()
        return buf[slots], slots


class ShardedUnique:
    """ock::ctr::Unique with the enhanced outputs (AccCTR include/unique.h:49-131) over one id stream."""

    def __init__(self, max_keys, sharding_num=1, use_sharding=False, use_padding=False, padding_size=0,
                 padding_val=-1, use_id_count=False, performance=False):
        if use_padding and not use_sharding:
            raise ValueError("padding needs sharding")  # Initialize returns H_ERROR (unique_test.cpp:109-128)
        if use_sharding and sharding_num <= 0:
            raise ValueError("shardingNum must be positive")
        if use_padding and padding_size <= 0:
            raise ValueError("paddingSize must be positive")
        self.shards = sharding_num if use_sharding else 1
        self.padding = padding_size if use_padding else 0
        self.padding_val = padding_val
        self.use_id_count = use_id_count
        self.performance = performance
        self.unique = Unique(max_keys, 1, position_lists=False)
        self.g = c_void_p()
        check(lib().recsdk_regroup_create(max_keys, ctypes.byref(self.g)))

    def close(self):
        if self.g:
            lib().recsdk_regroup_destroy(self.g)
            self.g = c_void_p()
        self.unique.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def do_enhanced_unique(self, ids):
        """Returns a dict with the fields of EnhancedUniqueOut (device tensors; unique_id_cnt an int)."""
        n = ids.numel()
        dev = ids.device
        offsets = _one_table_offsets(n, dev)
        self.unique.run(ids, offsets)
        m = max(self.padding * self.shards, n, 1)
        uid = torch.empty(m, dtype=torch.int64, device=dev)
        index = torch.empty(max(n, 1), dtype=torch.int32, device=dev)
        inb = torch.empty(max(n, 1), dtype=torch.int64, device=dev)
        cib = torch.empty(self.shards, dtype=torch.int32, device=dev)
        idc = torch.empty(max(n, 1), dtype=torch.int32, device=dev) if self.use_id_count else None
        fill = torch.empty(m, dtype=torch.int32, device=dev) if (self.use_id_count and self.padding) else None
        cnt = ctypes.c_int32()
        check(lib().recsdk_unique_sharded(self.g, self.unique.h, self.shards, 1 if self.performance else 0,
                                          self.padding, self.padding_val, _p(uid), _p(index), _p(inb), _p(cib),
                                          _p(idc), _p(fill), _stream(), ctypes.byref(cnt)))
        u = int(cib.sum().item())
        return {"unique_id": uid[:cnt.value], "index": index[:n], "unique_id_in_bucket": inb[:u],
                "cnt_in_bucket": cib, "id_cnt": None if idc is None else idc[:u],
                "id_cnt_fill": None if fill is None else fill[:cnt.value], "unique_id_cnt": cnt.value}


def unique_parallel(ids, unique=None, regroup=None):
    """hybrid::UniqueParallel (unique.cpp:110-118): (sorted distinct ids, inverse int64)."""
    n = ids.numel()
    dev = ids.device
    own = unique is None
    if own:
        unique = Unique(max(n, 1), 1, position_lists=False)
        regroup = c_void_p()
        check(lib().recsdk_regroup_create(max(n, 1), ctypes.byref(regroup)))
    try:
        offsets = _one_table_offsets(n, dev)
        unique.run(ids, offsets)
        out = torch.empty(max(n, 1), dtype=torch.int64, device=dev)
        inv = torch.empty(max(n, 1), dtype=torch.int64, device=dev)
        check(lib().recsdk_unique_sorted(regroup, unique.h, _p(out), _p(inv), _stream()))
        u = unique.total()
        return out[:u], inv[:n]
    finally:
        if own:
            torch.cuda.synchronize()
            lib().recsdk_regroup_destroy(regroup)
            unique.close()


def _hp(a):
    """pointer to a contiguous host numpy array"""
    return None if a is None else c_void_p(a.ctypes.data)


class Initializer:
    """A table's row initializers (AccCTR InitializerInfo list): descs = [(kind, start, len, value_or_mean, stddev,
    seed, init_k), ...].  Host side only."""

    def __init__(self, descs):
        self.h = c_void_p()
        self._descs = capi.initializer_descs(descs)
        check(lib().recsdk_initializer_create(self._descs, len(descs), ctypes.byref(self.h)))

    def close(self):
        if self.h:
            lib().recsdk_initializer_destroy(self.h)
            self.h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def generate(self, rows, ext_dim, fill=0.0):
        import numpy as np
        out = np.full((rows, ext_dim), fill, dtype=np.float32)
        check(lib().recsdk_initializer_generate(self.h, _hp(out), rows, ext_dim))
        return out


class EmbLocalTable:
    """Host-DRAM row store behind the HBM cache (AccCTR EmbLocalTable): pinned rows, host key map, device kernels
    for the swaps.  keys / rows on the host side are numpy arrays."""

    def __init__(self, vocab_size, ext_dim, descs):
        self.ext = ext_dim
        self.h = c_void_p()
        self._descs = capi.initializer_descs(descs)
        check(lib().recsdk_hostrows_create(vocab_size, ext_dim, self._descs, len(descs), ctypes.byref(self.h)))

    def close(self):
        if self.h:
            lib().recsdk_hostrows_destroy(self.h)
            self.h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @staticmethod
    def _keys(keys):
        import numpy as np
        return np.ascontiguousarray(keys, dtype=np.int64)

    def gather(self, keys, threads=1):
        import numpy as np
        keys = self._keys(keys)
        out = np.empty((keys.size, self.ext), dtype=np.float32)
        check(lib().recsdk_hostrows_gather(self.h, _hp(keys), keys.size, _hp(out), threads))
        return out

    def scatter(self, keys, src, threads=1):
        import numpy as np
        keys = self._keys(keys)
        src = np.ascontiguousarray(src, dtype=np.float32)
        check(lib().recsdk_hostrows_scatter(self.h, _hp(keys), keys.size, _hp(src), threads))

    def gather_and_remove(self, keys):
        import numpy as np
        keys = self._keys(keys)
        out = np.empty((keys.size, self.ext), dtype=np.float32)
        check(lib().recsdk_hostrows_gather_and_remove(self.h, _hp(keys), keys.size, _hp(out)))
        return out

    def remove(self, keys):
        keys = self._keys(keys)
        check(lib().recsdk_hostrows_remove(self.h, _hp(keys), keys.size))

    def size(self):
        v = c_int64()
        check(lib().recsdk_hostrows_size(self.h, ctypes.byref(v)))
        return v.value

    def export(self):
        import numpy as np
        n = self.size()
        keys = np.empty(max(n, 1), dtype=np.int64)
        rows = np.empty((max(n, 1), self.ext), dtype=np.float32)
        cnt = c_int64()
        check(lib().recsdk_hostrows_export(self.h, _hp(keys), _hp(rows), n, ctypes.byref(cnt)))
        return keys[:n], rows[:n]

    def serialize(self):
        """EmbLocalTable::Serialize: bytes of [key u64 | ext floats] records, ascending key."""
        n = c_int64()
        check(lib().recsdk_hostrows_serialize(self.h, None, 0, ctypes.byref(n)))
        buf = np.empty(max(n.value, 1), dtype=np.uint8)
        check(lib().recsdk_hostrows_serialize(self.h, buf.ctypes.data_as(c_void_p), buf.size, ctypes.byref(n)))
        return buf[:n.value].tobytes()

    def deserialize(self, data):
        buf = np.frombuffer(data, dtype=np.uint8)
        check(lib().recsdk_hostrows_deserialize(self.h, buf.ctypes.data_as(c_void_p) if buf.size else None, buf.size))

    def save(self, path, table_name, rank, emb_dim, optim_num):
        """EmbcacheManager::Save for this table: <path>/<table_name>/rank<rank>/{key,embedding,momentum1,momentum2}/."""
        prefix = "%s/%s/rank%d" % (path, table_name, rank)
        check(lib().recsdk_hostrows_save(self.h, prefix.encode(), emb_dim, optim_num))
        return prefix

    def load(self, path, table_name, rank, emb_dim, optim_num):
        prefix = "%s/%s/rank%d" % (path, table_name, rank)
        check(lib().recsdk_hostrows_load(self.h, prefix.encode(), emb_dim, optim_num))
        return prefix

    def swap_out(self, keys, slots, cache):
        """cache[slots[i]] (device rows, [cache_rows, stride] float32) -> host rows of keys[i]; keys: a device tensor
        of distinct keys (no host work) or host keys"""
        if isinstance(keys, torch.Tensor) and keys.is_cuda:
            check(lib().recsdk_hostrows_swap_out_dev(self.h, _p(keys), keys.numel(), _p(slots), _p(cache),
                                                     cache.stride(0), _stream()))
            return
        keys = self._keys(keys)
        check(lib().recsdk_hostrows_swap_out(self.h, _hp(keys), keys.size, _p(slots), _p(cache), cache.stride(0),
                                             _stream()))

    def on_link_start(self, event):
        """event: a recorded-once torch.cuda.Event (or None) that every later swap() records right before its link
        kernel, after the kernels that prepare the move"""
        check(lib().recsdk_hostrows_on_link_start(self.h, c_void_p(event.cuda_event) if event is not None else None))

    def swap(self, out_keys, out_slots, in_keys, in_slots, cache):
        """swap_out(out_keys, out_slots) then swap_in(in_keys, in_slots) with both directions of the host link busy at
        once; device tensors of distinct keys, no key in both lists (the lists of one cache-planner call)"""
        check(lib().recsdk_hostrows_swap_dev(self.h, _p(out_keys), out_keys.numel(), _p(out_slots), _p(in_keys),
                                             in_keys.numel(), _p(in_slots), _p(cache), cache.stride(0), _stream()))

    def swap_in(self, keys, slots, cache):
        """host rows of keys[i] (created with initial values when new) -> cache[slots[i]]"""
        if isinstance(keys, torch.Tensor) and keys.is_cuda:
            check(lib().recsdk_hostrows_swap_in_dev(self.h, _p(keys), keys.numel(), _p(slots), _p(cache),
                                                    cache.stride(0), _stream()))
            return
        keys = self._keys(keys)
        check(lib().recsdk_hostrows_swap_in(self.h, _hp(keys), keys.size, _p(slots), _p(cache), cache.stride(0),
                                            _stream()))
