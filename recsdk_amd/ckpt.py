"""Checkpoints in the reference's on-disk layout, over the C ABI.

  save_table / load_table        EmbeddingStatic / EmbeddingDynamic ::Save / ::Load
                                 (training/tf_rec_v1/src/core/emb_table/embedding_{static,dynamic}.cpp)
  merge_table_slices             what the Python saver does after every rank wrote its slice
                                 (training/tf_rec_v1/python/saver/saver.py:290-330,815-890): slice_<rank>.data ->
                                 slice.data (+ slice.attribute)
  save_history / load_history    FeatAdmitNEvictCkpt (training/tf_rec_v1/src/core/ckpt_data_handler/
                                 feat_admit_n_evict_ckpt/feat_admit_n_evict_ckpt.cpp:82-210)
  save_filter / load_filter      EmbcacheManager::Save/LoadFeatureAdmitAndEvictInfo
                                 (training/torch_rec_v1/torchrec_embcache/src/torchrec_embcache/csrc/embedding_cache/
                                 embcache_manager.cpp:824-950)
The row / key files themselves are written and read by librecsdk_hip.so (recsdk_ckpt_*, recsdk_hostrows_save/load).
"""
import ctypes
import os
from ctypes import c_int64, c_void_p

import numpy as np
import torch

from .capi import check, lib

INT64_MIN = -(1 << 63)


def _stream():
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return None if t is None else c_void_p(t.data_ptr())


def _path(*parts):
    return os.path.join(*parts).encode()


def export_table(tables, t, device="cuda:0"):
    """(keys, values) of table t as device tensors, ascending value."""
    _, live, _ = tables.stats()
    cap = max(live[t], 1)
    keys = torch.empty(cap, dtype=torch.int64, device=device)
    vals = torch.empty(cap, dtype=torch.int64, device=device)
    n = c_int64()
    check(lib().recsdk_tables_export(tables.h, t, _p(keys), _p(vals), cap, _stream(), ctypes.byref(n)))
    return keys[:n.value], vals[:n.value]


def save_table(save_path, name, rank_id, tables, t, emb_size=None, optim_name=None, optim_params=()):
    """EmbeddingStatic::Save (emb_size None: key file only; returns the device offsets of the keys, which the caller
    uses to slice the table variable) or EmbeddingDynamic::Save (key file + embedding + one file per optimizer
    state, rows read at the exported device addresses)."""
    keys, vals = export_table(tables, t)
    n = keys.numel()
    fname = "slice_%d.data" % rank_id
    check(lib().recsdk_ckpt_write_keys(_path(save_path, name, "key", fname), _p(keys), n, _stream()))
    if emb_size is None:
        return vals
    check(lib().recsdk_ckpt_write_rows(_path(save_path, name, "embedding", fname), _p(vals), n, emb_size, 0, _stream()))
    for p, param in enumerate(optim_params, start=1):
        check(lib().recsdk_ckpt_write_rows(_path(save_path, name, "%s_%s" % (optim_name, param), fname), _p(vals), n,
                                           emb_size, p * emb_size * 4, _stream()))
    return vals


def merge_table_slices(save_path, name, data_types, emb_size, is_dp=False):
    """slice_*.data of every rank -> slice.data + slice.attribute per data type ("key", "embedding", "<optim>_<param>").
    Model parallel: the slices are concatenated in file-name order; data parallel: the first one is kept."""
    for data_type in data_types:
        upper = os.path.join(save_path, name, data_type)
        files = sorted(f for f in os.listdir(upper) if f.startswith("slice_"))
        if not files:
            raise RuntimeError("rename and remove file failed, slice*.data do not exist in %s." % upper)
        out = os.path.join(upper, "slice.data")
        if is_dp:
            os.replace(os.path.join(upper, files[0]), out)
            for f in files[1:]:
                os.remove(os.path.join(upper, f))
        else:
            with open(out, "wb") as dst:
                for f in files:
                    with open(os.path.join(upper, f), "rb") as src:
                        while True:
                            block = src.read(1 << 24)
                            if not block:
                                break
                            dst.write(block)
                    os.remove(os.path.join(upper, f))
        size = os.path.getsize(out)
        if data_type == "key":
            attribute = np.array([size // 8, 8], dtype=np.int64)
        else:
            attribute = np.array([size // 4 // emb_size, emb_size, 4], dtype=np.int64)
        attribute.tofile(os.path.join(upper, "slice.attribute"))


def load_table(save_path, name, rank_id, rank_size, tables, t, is_dp=False, emb_size=None, ext_emb_size=None,
               first_address=None, optim_name=None, optim_params=()):
    """EmbeddingStatic::Load (emb_size None; returns (keys, load_offset): row load_offset[i] of the saved variable
    belongs at device offset i) or EmbeddingDynamic::Load (rows and optimizer states are read into the arena at
    first_address, ext_emb_size floats apart)."""
    key_file = _path(save_path, name, "key", "slice.data")
    n = c_int64()
    size = os.path.getsize(key_file.decode()) if os.path.exists(key_file.decode()) else 0
    cap = max(size // 8, 1)
    keys = np.empty(cap, dtype=np.int64)
    load_offset = np.empty(cap, dtype=np.int64)
    check(lib().recsdk_ckpt_read_keys(key_file, rank_id, rank_size, int(is_dp), keys.ctypes.data_as(c_void_p),
                                      load_offset.ctypes.data_as(c_void_p), cap, ctypes.byref(n)))
    keys, load_offset = keys[:n.value].copy(), load_offset[:n.value].copy()
    d_keys = torch.from_numpy(keys).to("cuda:0")
    check(lib().recsdk_tables_load_keys(tables.h, t, _p(d_keys), n.value, _stream()))
    if emb_size is None:
        return keys, load_offset
    lo = load_offset.ctypes.data_as(c_void_p)
    check(lib().recsdk_ckpt_read_rows(_path(save_path, name, "embedding", "slice.data"), lo, n.value, emb_size,
                                      c_void_p(first_address), ext_emb_size, _stream()))
    for p, param in enumerate(optim_params, start=1):
        check(lib().recsdk_ckpt_read_rows(_path(save_path, name, "%s_%s" % (optim_name, param), "slice.data"), lo,
                                          n.value, emb_size, c_void_p(first_address + p * emb_size * 4), ext_emb_size,
                                          _stream()))
    return keys, load_offset


# ---- admission / eviction history -------------------------------------------------------------------------------

def save_history(save_path, name, rank_id, faae, t, thresholds):
    """HashTable-side files of one table: table_2_threshold/slice_<rank>.data = int32 [countThreshold, timeThreshold,
    isEnableSum]; history_record/slice_<rank>.data = int64 [tableTimestamp, (featureId, count, lastTime)*]."""
    keys, counts, times = faae.dump(t)
    _, latest = faae.stats()
    rec = np.empty(1 + 3 * keys.size, dtype=np.int64)
    rec[0] = latest[t]
    rec[1::3] = keys
    rec[2::3] = counts.astype(np.int64)
    rec[3::3] = times
    for sub, arr in (("table_2_threshold", np.asarray(thresholds, dtype=np.int32)), ("history_record", rec)):
        d = os.path.join(save_path, name, sub)
        os.makedirs(d, exist_ok=True)
        arr.tofile(os.path.join(d, "slice_%d.data" % rank_id))
    return keys.size


def write_history_attributes(save_path, name, n_records):
    """The attribute files the loader wants next to slice.data: [3, 4] and [n_records, 8]."""
    np.array([3, 4], dtype=np.int64).tofile(os.path.join(save_path, name, "table_2_threshold", "slice.attribute"))
    np.array([n_records, 8], dtype=np.int64).tofile(os.path.join(save_path, name, "history_record", "slice.attribute"))


def load_history(save_path, name, faae, t, device="cuda:0"):
    """Returns the saved [countThreshold, timeThreshold, isEnableSum]; the records replace table t's.  Returns None
    when the checkpoint holds no admission data (no attribute file: noFeatAdmitAndEvictData)."""
    d = os.path.join(save_path, name, "history_record")
    if not os.path.exists(os.path.join(d, "slice.attribute")):
        return None
    attribute = np.fromfile(os.path.join(d, "slice.attribute"), dtype=np.int64)
    rec = np.fromfile(os.path.join(d, "slice.data"), dtype=np.int64)
    if rec.size == 0 or attribute.size == 0:
        raise RuntimeError("TransArr or attribute is empty. Please check the implementations.")
    n = int(attribute[0])
    body = rec[1:1 + 3 * n].reshape(n, 3)
    keys = torch.from_numpy(np.ascontiguousarray(body[:, 0])).to(device)
    counts = torch.from_numpy(np.ascontiguousarray(body[:, 1]).astype(np.uint32).view(np.int32)).to(device)
    times = torch.from_numpy(np.ascontiguousarray(body[:, 2])).to(device)
    check(lib().recsdk_faae_load(faae.h, t, _p(keys), _p(counts), _p(times), n, 1, int(rec[0]), _stream()))
    torch.cuda.current_stream().synchronize()
    return np.fromfile(os.path.join(save_path, name, "table_2_threshold", "slice.data"), dtype=np.int32)


def save_filter(prefix, faae, t, save_keys, admit=True, evict=True):
    """Torch-side feature filter files under prefix = <path>/<table>/rank<rank>: admit_count/slice.data = the count of
    every saved key (-1 without a record), attribute {8, len(save_keys)}; evict_timestamp/slice_evict_key.data,
    slice_evict_ts.data = the timestamp records, attribute {8, records}."""
    keys, counts, times = faae.dump(t)
    if admit:
        d = os.path.join(prefix, "admit_count")
        os.makedirs(d, exist_ok=True)
        have = {int(k): int(c) for k, c in zip(keys, counts) if c != 0xFFFFFFFF}
        out = np.array([have.get(int(k), -1) for k in save_keys], dtype=np.int64)
        np.array([8, out.size], dtype=np.int64).tofile(os.path.join(d, "slice.attribute"))
        out.tofile(os.path.join(d, "slice.data"))
    if evict:
        d = os.path.join(prefix, "evict_timestamp")
        os.makedirs(d, exist_ok=True)
        sel = times != INT64_MIN
        np.array([8, int(sel.sum())], dtype=np.int64).tofile(os.path.join(d, "slice.attribute"))
        keys[sel].tofile(os.path.join(d, "slice_evict_key.data"))
        times[sel].tofile(os.path.join(d, "slice_evict_ts.data"))


def _read_counted(attr_file, data_file):
    attribute = np.fromfile(attr_file, dtype=np.int64)
    if attribute.size < 2 or attribute[1] < 0 or attribute[1] > 10 ** 9:
        raise RuntimeError("Read key attribute file error, keys count is invalid, file:%s." % attr_file)
    data = np.fromfile(data_file, dtype=np.int64)
    if os.path.getsize(data_file) % 8 != 0 or data.size != attribute[1]:
        raise RuntimeError("Key file bytes is not an integer multiple of type int64_t, key file:%s" % data_file)
    return data


def load_filter(prefix, faae, t, save_keys, admit=True, evict=True, device="cuda:0"):
    """LoadFeatureRecords (count of save_keys[i] = file value i) and LoadTimestampRecords, into table t."""
    if admit:
        d = os.path.join(prefix, "admit_count")
        counts = _read_counted(os.path.join(d, "slice.attribute"), os.path.join(d, "slice.data"))
        save_keys = np.ascontiguousarray(save_keys, dtype=np.int64)
        if save_keys.size != counts.size:
            raise RuntimeError("Failed to load key count info, vector size is not same between keys and counts.")
        k = torch.from_numpy(save_keys).to(device)
        c = torch.from_numpy(counts.astype(np.uint32).view(np.int32)).to(device)
        check(lib().recsdk_faae_load(faae.h, t, _p(k), _p(c), None, k.numel(), 0, INT64_MIN, _stream()))
    if evict:
        d = os.path.join(prefix, "evict_timestamp")
        attr = os.path.join(d, "slice.attribute")
        keys = _read_counted(attr, os.path.join(d, "slice_evict_key.data"))
        times = _read_counted(attr, os.path.join(d, "slice_evict_ts.data"))
        k = torch.from_numpy(keys).to(device)
        ts = torch.from_numpy(times).to(device)
        check(lib().recsdk_faae_load(faae.h, t, _p(k), None, _p(ts), k.numel(), 0, INT64_MIN, _stream()))
    torch.cuda.current_stream().synchronize()
