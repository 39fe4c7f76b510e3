"""GPU parity: checkpoint files in the reference's layout through the C ABI.

Files written by the library are compared byte for byte with the oracle's restatement of the layout; loads are
compared with the oracle's loaders; and a table that was saved and loaded must go on behaving like the original."""
import os

import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, ckpt, host
from recsdk_amd.synth import zipf_ranks
from tests.util import splitmix64

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
C, N = capi.INIT_CONSTANT, capi.INIT_RANDOM_NORMAL


def dev(a, dt=torch.int64):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV).to(dt)


def k2o(tg, keys, channel=0):
    dk = dev(np.asarray(keys, dtype=np.int64))
    tg.key2offset(dk, dev(np.array([0, dk.numel()], dtype=np.int64)), channel)
    return dk.cpu().numpy()


def evict(tg, keys):
    dk = dev(np.asarray(keys, dtype=np.int64))
    tg.evict_keys(dk, dev(np.array([0, dk.numel()], dtype=np.int64)))


def read(*parts):
    with open(os.path.join(*parts), "rb") as f:
        return f.read()


def test_static_table_save_merge_load(tmp_path):
    path = str(tmp_path)
    tg = host.EmbeddingTables([5000], 4096)
    keys = splitmix64(np.arange(3000, dtype=np.uint64)).astype(np.int64)
    keys[7] = np.int64(-(1 << 63))            # the key whose bits equal the erased-slot marker
    offs = k2o(tg, keys)
    evict(tg, keys[100:600])                  # holes: the export must skip erased keys
    more = splitmix64(np.arange(10**6, 10**6 + 200, dtype=np.uint64)).astype(np.int64)
    offs2 = k2o(tg, more)                      # reuse evicted slots
    live = {int(k): int(o) for k, o in zip(keys, offs)}
    for k in keys[100:600]:
        del live[int(k)]
    live.update({int(k): int(o) for k, o in zip(more, offs2)})
    dev_offsets = ckpt.save_table(path, "t0", 0, tg, 0).cpu().numpy()
    want_keys = np.array(sorted(live, key=live.get), dtype=np.int64)
    assert read(path, "t0", "key", "slice_0.data") == want_keys.tobytes()
    np.testing.assert_array_equal(dev_offsets, np.array(sorted(live.values()), dtype=np.int64))
    # a second rank's slice, then the merge the Python saver does
    other = np.array([11, -5, 22, 33, 44, 8], dtype=np.int64)
    other.tofile(os.path.join(path, "t0", "key", "slice_1.data"))
    ckpt.merge_table_slices(path, "t0", ["key"], emb_size=0, is_dp=False)
    merged = np.concatenate([want_keys, other])
    assert read(path, "t0", "key", "slice.data") == merged.tobytes()
    assert read(path, "t0", "key", "slice.attribute") == np.array([merged.size, 8], dtype=np.int64).tobytes()
    assert sorted(os.listdir(os.path.join(path, "t0", "key"))) == ["slice.attribute", "slice.data"]
    for rank_id, rank_size, is_dp in ((0, 1, False), (1, 3, False), (2, 3, False), (1, 3, True)):
        tg2 = host.EmbeddingTables([5000], 4096)
        got_keys, got_lo = ckpt.load_table(path, "t0", rank_id, rank_size, tg2, 0, is_dp=is_dp)
        want_map, want_lo = oracle.ckpt_static_load(merged, rank_id, rank_size, is_dp)
        np.testing.assert_array_equal(got_lo, want_lo)
        np.testing.assert_array_equal(got_keys, merged[want_lo])
        probe = np.concatenate([merged, [123456789]])
        got = k2o(tg2, probe, channel=capi.CHANNEL_EVAL)
        np.testing.assert_array_equal(got, [want_map.get(int(k), -1) for k in probe])
        mo, lv, ev = tg2.stats()
        assert mo == [len(want_map)] and lv == [len(want_map)] and ev == [0]
        # the loaded table goes on like a table that got these keys in one call
        fresh = k2o(tg2, np.array([987654321, 987654322]))
        assert fresh.tolist() == [len(want_map), len(want_map) + 1]


def test_static_load_rejects_too_many_keys(tmp_path):
    path = str(tmp_path)
    os.makedirs(os.path.join(path, "t", "key"))
    np.arange(100, dtype=np.int64).tofile(os.path.join(path, "t", "key", "slice.data"))
    tg = host.EmbeddingTables([50], 256)
    with pytest.raises(RuntimeError, match="exceeds device vocab size"):
        ckpt.load_table(path, "t", 0, 1, tg, 0)
    with pytest.raises(RuntimeError, match="Failed to open read file"):
        ckpt.load_table(path, "missing", 0, 1, tg, 0)


@pytest.mark.parametrize("n,emb", [(700, 16), (150000, 128)])        # the second spans several staging chunks
def test_dynamic_table_save_load(tmp_path, n, emb):
    path = str(tmp_path)
    ext = 3 * emb                                                       # [embedding | m | v]
    vocab = n + 64
    arena = torch.randn(vocab, ext, device=DEV)
    tg = host.EmbeddingTables([vocab], n, dynamic=[1], arena_bases=[arena.data_ptr()], row_bytes=[ext * 4])
    keys = splitmix64(np.arange(n, dtype=np.uint64)).astype(np.int64)
    addr = k2o(tg, keys)
    rows_of = (addr - arena.data_ptr()) // (ext * 4)
    np.testing.assert_array_equal(rows_of, np.arange(n))
    ckpt.save_table(path, "d", 0, tg, 0, emb_size=emb, optim_name="LazyAdam", optim_params=("m", "v"))
    host_arena = arena.cpu().numpy()
    assert read(path, "d", "key", "slice_0.data") == keys.tobytes()
    for p, sub in enumerate(("embedding", "LazyAdam_m", "LazyAdam_v")):
        assert read(path, "d", sub, "slice_0.data") == oracle.ckpt_row_file(host_arena[:n], emb, p * emb), sub
    ckpt.merge_table_slices(path, "d", ["key", "embedding", "LazyAdam_m", "LazyAdam_v"], emb_size=emb, is_dp=True)
    assert read(path, "d", "embedding", "slice.attribute") == np.array([n, emb, 4], dtype=np.int64).tobytes()
    for rank_id, rank_size in ((0, 1), (2, 3)):
        arena2 = torch.full((vocab, ext), -7.0, device=DEV)
        tg2 = host.EmbeddingTables([vocab], n, dynamic=[1], arena_bases=[arena2.data_ptr()], row_bytes=[ext * 4])
        got_keys, got_lo = ckpt.load_table(path, "d", rank_id, rank_size, tg2, 0, emb_size=emb, ext_emb_size=ext,
                                           first_address=arena2.data_ptr(), optim_name="LazyAdam",
                                           optim_params=("m", "v"))
        want_keys, want_lo = oracle.ckpt_filter_keys(keys, rank_id, rank_size, False)
        np.testing.assert_array_equal(got_keys, want_keys)
        np.testing.assert_array_equal(got_lo, want_lo)
        m = want_keys.size
        want = np.full((vocab, ext), -7.0, dtype=np.float32)
        for p, sub in enumerate(("embedding", "LazyAdam_m", "LazyAdam_v")):
            oracle.ckpt_read_rows(read(path, "d", sub, "slice.data"), want_lo, emb, ext, want[:m, p * emb:])
        np.testing.assert_array_equal(arena2.cpu().numpy(), want)
        got_addr = k2o(tg2, want_keys, channel=capi.CHANNEL_EVAL)
        np.testing.assert_array_equal(got_addr, arena2.data_ptr() + np.arange(m) * ext * 4)
        # new keys take the rows after the loaded ones
        assert k2o(tg2, np.array([424242]))[0] == arena2.data_ptr() + m * ext * 4


def test_host_rows_serialize_reference_cases():
    ext = 28        # the reference's case has 26 floats a row; rows of this store are a multiple of 4 floats
    descs = [(C, 0, ext, 0.0, 0.0, 0, 1.0)]
    tab = host.EmbLocalTable(5, ext, descs)
    with pytest.raises(RuntimeError, match="get data failed"):
        tab.deserialize(b"AB12")
    keys = np.arange(5, dtype=np.int64)
    emb = (0.01 * np.arange(5 * ext, dtype=np.float32)).reshape(5, ext)
    tab, orc = host.EmbLocalTable(5, ext, descs), oracle.HostRows(5, ext, descs)
    tab.scatter(keys, emb)
    orc.scatter(keys, emb)
    b1 = tab.serialize()
    assert b1 == orc.serialize()
    with pytest.raises(RuntimeError, match="get data failed"):
        tab.deserialize(b1[:len(b1) // 2])
    tab = host.EmbLocalTable(5, ext, descs)
    tab.scatter(keys, emb)
    tab.deserialize(b1)
    assert tab.serialize() == b1


def test_host_rows_serialize_into_fresh_store_matches_oracle():
    ext = 12
    descs = [(N, 0, 4, 0.0, 0.05, 3, 1.0), (C, 4, 8, 0.25, 0.0, 0, 1.0)]
    rng = np.random.default_rng(2)
    src, osrc = host.EmbLocalTable(300, ext, descs), oracle.HostRows(300, ext, descs)
    keys = rng.choice(10**6, 200, replace=False).astype(np.int64) - 500
    upd = rng.normal(0, 1, (200, ext)).astype(np.float32)
    src.scatter(keys, upd)
    osrc.scatter(keys, upd)
    data = src.serialize()
    assert data == osrc.serialize()
    dst, odst = host.EmbLocalTable(300, ext, descs), oracle.HostRows(300, ext, descs)
    dst.gather(keys[:20])                      # some rows exist already, with initial values
    odst.gather(keys[:20])
    dst.deserialize(data)
    assert odst.deserialize(data) is True
    for a, b in zip(dst.export(), odst.export()):
        np.testing.assert_array_equal(a, b)
    # rows created after the load draw from the same place of the initializer stream
    np.testing.assert_array_equal(dst.gather([10**7, 10**7 + 1]), odst.gather([10**7, 10**7 + 1]))
    small = host.EmbLocalTable(10, ext, descs)
    with pytest.raises(RuntimeError, match="too small"):
        small.deserialize(data)


@pytest.mark.parametrize("optim_num", [0, 1, 2])
def test_host_rows_torch_save_load(tmp_path, optim_num):
    path = str(tmp_path)
    emb = 8
    ext = emb * (1 + optim_num)
    descs = [(N, 0, emb, 0.0, 0.1, 5, 1.0)] + ([(C, emb, ext - emb, 0.0, 0.0, 0, 1.0)] if optim_num else [])
    rng = np.random.default_rng(3)
    tab, orc = host.EmbLocalTable(600, ext, descs), oracle.HostRows(600, ext, descs)
    keys = rng.choice(10**9, 500, replace=False).astype(np.int64)
    upd = rng.normal(0, 1, (500, ext)).astype(np.float32)
    tab.scatter(keys, upd)
    orc.scatter(keys, upd)
    prefix = tab.save(path, "tbl", 3, emb, optim_num)
    assert prefix == os.path.join(path, "tbl", "rank3")
    files = orc.torch_files(emb, optim_num)
    on_disk = sorted(os.path.join(d, f)[len(prefix) + 1:] for d, _, fs in os.walk(prefix) for f in fs)
    assert on_disk == sorted(files)
    for name, want in files.items():
        assert read(prefix, name) == want, name
    tab2, orc2 = host.EmbLocalTable(600, ext, descs), oracle.HostRows(600, ext, descs)
    tab2.load(path, "tbl", 3, emb, optim_num)
    orc2.torch_load(files, emb, optim_num)
    for a, b in zip(tab2.export(), orc2.export()):
        np.testing.assert_array_equal(a, b)
    for a, b in zip(tab2.export(), tab.export()):
        np.testing.assert_array_equal(a, b)
    # the checks the reference's loader makes
    with pytest.raises(RuntimeError, match="dim error"):
        host.EmbLocalTable(600, 2 * ext, descs).load(path, "tbl", 3, 2 * emb if optim_num == 0 else emb // 2, optim_num)
    np.array([8, 499], dtype=np.int64).tofile(os.path.join(prefix, "key", "slice.attribute"))
    with pytest.raises(RuntimeError, match="Key file bytes"):
        host.EmbLocalTable(600, ext, descs).load(path, "tbl", 3, emb, optim_num)
    with pytest.raises(RuntimeError, match="Failed to open read file"):
        host.EmbLocalTable(600, ext, descs).load(path, "nope", 3, emb, optim_num)


def faae_batches(rng, steps, n, start=0):
    hot = splitmix64(np.arange(400, dtype=np.uint64)).astype(np.int64)
    for step in range(start, start + steps):
        fresh = splitmix64(np.arange(10**6 + step * n, 10**6 + (step + 1) * n, dtype=np.uint64)).astype(np.int64)
        keys = np.where(rng.random(n) < 0.7, hot[zipf_ranks(rng, 1.2, 400, n)], fresh)
        yield step, keys, rng.integers(1, 4, n)


def test_history_records_save_load_and_continue(tmp_path):
    path = str(tmp_path)
    n = 2000
    o = dev(np.array([0, n], dtype=np.int64))
    a = host.FeatureAdmitAndEvict([30000], [2], [4], max_keys=n)
    rng = np.random.default_rng(4)
    for step, keys, cnt in faae_batches(rng, 6, n):
        a.feature_admit(capi.CHANNEL_TRAIN, dev(keys), dev(cnt, torch.int32), o, [1000 + step])
    records = ckpt.save_history(path, "t", 0, a, 0, [2, 4, 1])
    k, c, ts = a.dump(0, 1 << 16)
    assert records == k.size
    assert read(path, "t", "history_record", "slice_0.data") == oracle.history_record(1005, k, c, ts).tobytes()
    assert read(path, "t", "table_2_threshold", "slice_0.data") == np.array([2, 4, 1], dtype=np.int32).tobytes()
    b = host.FeatureAdmitAndEvict([30000], [2], [4], max_keys=n)
    assert ckpt.load_history(path, "t", b, 0) is None             # no merged files yet: no admission data
    ckpt.merge_table_slices(path, "t", ["history_record", "table_2_threshold"], emb_size=1, is_dp=True)
    ckpt.write_history_attributes(path, "t", records)
    # stale records in the target are dropped by the load
    b.feature_admit(capi.CHANNEL_TRAIN, dev(np.arange(n)), dev(np.ones(n), torch.int32), o, [5])
    assert ckpt.load_history(path, "t", b, 0).tolist() == [2, 4, 1]
    for x, y in zip(a.dump(0, 1 << 16), b.dump(0, 1 << 16)):
        np.testing.assert_array_equal(x, y)
    assert a.stats() == b.stats()
    rng_a, rng_b = np.random.default_rng(5), np.random.default_rng(5)
    for (step, keys, cnt), (_, keys_b, cnt_b) in zip(faae_batches(rng_a, 6, n, 6), faae_batches(rng_b, 6, n, 6)):
        ga = a.feature_admit(capi.CHANNEL_TRAIN, dev(keys), dev(cnt, torch.int32), o, [1000 + step]).cpu().numpy()
        gb = b.feature_admit(capi.CHANNEL_TRAIN, dev(keys_b), dev(cnt_b, torch.int32), o, [1000 + step]).cpu().numpy()
        np.testing.assert_array_equal(ga, gb)
        if step % 2 == 1:
            ea, eb = a.feature_evict(cap=1 << 16), b.feature_evict(cap=1 << 16)
            np.testing.assert_array_equal(ea[0].cpu().numpy(), eb[0].cpu().numpy())
    for x, y in zip(a.dump(0, 1 << 16), b.dump(0, 1 << 16)):
        np.testing.assert_array_equal(x, y)


def test_feature_filter_save_load(tmp_path):
    prefix = os.path.join(str(tmp_path), "tbl", "rank0")
    n = 1500
    o = dev(np.array([0, n], dtype=np.int64))
    rng = np.random.default_rng(6)
    a = host.FeatureAdmitAndEvict([20000], [3], [4], max_keys=8 * n)
    seen = set()
    for step in range(5):
        keys = np.where(rng.random(n) < 0.6, zipf_ranks(rng, 1.1, 300, n), rng.integers(10**6, 10**9, n)).astype(np.int64)
        a.statistics_key_count(dev(keys), dev(rng.integers(0, 3, n), torch.int32), o)
        if step % 2 == 0:                      # some keys have a count but no timestamp
            a.record_timestamp(dev(keys), dev((step + rng.integers(0, 2, n)).astype(np.int64)), o)
        seen.update(keys.tolist())
    save_keys = np.array(sorted(seen) + [-12345], dtype=np.int64)      # one saved key the filter never saw
    ckpt.save_filter(prefix, a, 0, save_keys)
    k, c, ts = a.dump(0, 1 << 16)
    count_of = {int(x): int(y) for x, y in zip(k, c) if y != 0xFFFFFFFF}
    want_counts = np.array([count_of.get(int(x), -1) for x in save_keys], dtype=np.int64)
    assert read(prefix, "admit_count", "slice.data") == want_counts.tobytes()
    assert read(prefix, "admit_count", "slice.attribute") == np.array([8, save_keys.size], dtype=np.int64).tobytes()
    has_ts = ts != ckpt.INT64_MIN
    assert read(prefix, "evict_timestamp", "slice_evict_key.data") == k[has_ts].tobytes()
    assert read(prefix, "evict_timestamp", "slice_evict_ts.data") == ts[has_ts].tobytes()
    assert read(prefix, "evict_timestamp", "slice.attribute") == np.array([8, int(has_ts.sum())], np.int64).tobytes()
    b = host.FeatureAdmitAndEvict([20000], [3], [4], max_keys=8 * n)
    ckpt.load_filter(prefix, b, 0, save_keys)
    kb, cb, tb = b.dump(0, 1 << 16)
    # every saved key has a record now; the key the filter never saw carries the saved -1 as its count
    assert set(kb.tolist()) == set(k.tolist()) | {-12345}
    got = {int(x): (int(y), int(z)) for x, y, z in zip(kb, cb, tb)}
    for x, y, z in zip(k, c, ts):
        assert got[int(x)] == (int(y) if y != 0xFFFFFFFF else 0xFFFFFFFF, int(z))
    assert got[-12345] == (0xFFFFFFFF, ckpt.INT64_MIN)
    probe = dev(save_keys.copy())
    oo = dev(np.array([0, save_keys.size], dtype=np.int64))
    np.testing.assert_array_equal(a.count_filter(dev(save_keys.copy()), oo).cpu().numpy()[:-1],
                                  b.count_filter(probe, oo).cpu().numpy()[:-1])
