"""Pins the oracle's restatement of the checkpoint byte layouts.

The layouts are fixed by the reference's readers and writers (raw little-endian arrays); each restatement is checked
against Python's struct module on hand-written tiny cases (an independent encoder), against the reference's own
serialize tests (AccCTR emb_cache_test.cpp:1414-1482: garbage and truncated buffers fail, a round trip reproduces the
bytes) and against the round trip load(save(x)) == x."""
import struct

import numpy as np
import pytest

import oracle

CONST = [(oracle.INIT_CONSTANT, 0, 6, 0.5, 0.0, 0, 1.0)]


def test_serialize_layout_by_struct():
    hr = oracle.HostRows(8, 6, CONST)
    hr.scatter([7, -2], np.arange(12, dtype=np.float32).reshape(2, 6))
    want = struct.pack("<q6f", -2, *range(6, 12)) + struct.pack("<q6f", 7, *range(0, 6))
    assert hr.serialize() == want


def test_reference_serialize_cases():
    ext = 26
    descs = [(oracle.INIT_CONSTANT, 0, ext, 0.0, 0.0, 0, 1.0)]
    hr = oracle.HostRows(5, ext, descs)
    assert hr.deserialize(b"AB12") is False                     # 4 bytes: not even a key
    keys = [0, 1, 2, 3, 4]
    hr = oracle.HostRows(5, ext, descs)
    hr.scatter(keys, (0.01 * np.arange(5 * ext, dtype=np.float32)).reshape(5, ext))
    b1 = hr.serialize()
    assert len(b1) == 5 * (8 + 4 * ext)
    assert hr.deserialize(b1[:len(b1) // 2]) is False            # cut in the middle of a record
    hr2 = oracle.HostRows(5, ext, descs)
    hr2.scatter(keys, (0.01 * np.arange(5 * ext, dtype=np.float32)).reshape(5, ext))
    b1 = hr2.serialize()
    assert hr2.deserialize(b1) is True
    assert hr2.serialize() == b1


def test_torch_files_layout_by_struct():
    hr = oracle.HostRows(8, 6, CONST)                              # emb_dim 2, two optimizer states
    hr.scatter([3, 1], np.arange(12, dtype=np.float32).reshape(2, 6))
    f = hr.torch_files(2, 2)
    assert f["key/slice.data"] == struct.pack("<2q", 1, 3)
    assert f["key/slice.attribute"] == struct.pack("<2q", 8, 2)
    assert f["embedding/slice.data"] == struct.pack("<4f", 6, 7, 0, 1)
    assert f["momentum1/slice.data"] == struct.pack("<4f", 8, 9, 2, 3)
    assert f["momentum2/slice.data"] == struct.pack("<4f", 10, 11, 4, 5)
    for name in ("embedding", "momentum1", "momentum2"):
        assert f[name + "/slice.attribute"] == struct.pack("<3q", 4, 2, 2)
    assert "momentum2/slice.data" not in hr.torch_files(2, 1)
    hr2 = oracle.HostRows(8, 6, CONST)
    hr2.torch_load(f, 2, 2)
    k1, r1 = hr.export()
    k2, r2 = hr2.export()
    np.testing.assert_array_equal(k1, k2)
    np.testing.assert_array_equal(r1, r2)


def test_filter_keys_uses_cpp_remainder():
    file_keys = np.array([8, -3, 5, 0, -4, 7, 9, 2], dtype=np.int64)
    keys, lo = oracle.ckpt_filter_keys(file_keys, 1, 4, False)
    # C++: 5 % 4 == 1, 9 % 4 == 1, -3 % 4 == -3 (not 1)
    np.testing.assert_array_equal(keys, [5, 9])
    np.testing.assert_array_equal(lo, [2, 6])
    keys, lo = oracle.ckpt_filter_keys(file_keys, 0, 4, False)
    np.testing.assert_array_equal(keys, [8, 0, -4])
    keys, lo = oracle.ckpt_filter_keys(file_keys, 3, 4, True)
    np.testing.assert_array_equal(keys, file_keys)
    np.testing.assert_array_equal(lo, np.arange(8))
    m, lo = oracle.ckpt_static_load(file_keys, 1, 4, False)
    assert m == {5: 0, 9: 1}


def test_row_file_round_trip():
    rng = np.random.default_rng(0)
    rows = rng.standard_normal((9, 12)).astype(np.float32)       # [emb 4 | m 4 | v 4]
    for p in range(3):
        data = oracle.ckpt_row_file(rows, 4, 4 * p)
        assert data == struct.pack("<36f", *rows[:, 4 * p:4 * p + 4].reshape(-1))
    lo = np.array([7, 0, 3], dtype=np.int64)
    out = np.zeros((3, 12), dtype=np.float32)
    oracle.ckpt_read_rows(oracle.ckpt_row_file(rows, 4, 4), lo, 4, 12, out[:, 4:])
    np.testing.assert_array_equal(out[:, 4:8], rows[lo, 4:8])
    assert not out[:, :4].any() and not out[:, 8:].any()


def test_history_record_layout():
    rec = oracle.history_record(1700, [5, -1], [3, 9], [1600, 1650])
    assert rec.tobytes() == struct.pack("<7q", 1700, 5, 3, 1600, -1, 9, 1650)
