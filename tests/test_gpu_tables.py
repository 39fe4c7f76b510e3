"""GPU parity: key -> slot / address tables (Key2Offset, EvictKeys) through the C ABI vs the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host
from tests.util import splitmix64

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def k2o(tg, tables, channel=0):
    keys = np.concatenate(tables + [np.zeros(0, np.int64)]).astype(np.int64)
    offs = np.concatenate([[0], np.cumsum([len(t) for t in tables])]).astype(np.int64)
    dk = torch.from_numpy(keys).to(DEV)
    tg.key2offset(dk, torch.from_numpy(offs).to(DEV), channel)
    out = dk.cpu().numpy()
    return [out[offs[t]:offs[t + 1]] for t in range(len(tables))]


def evict(tg, tables):
    keys = np.concatenate(tables + [np.zeros(0, np.int64)]).astype(np.int64)
    offs = np.concatenate([[0], np.cumsum([len(t) for t in tables])]).astype(np.int64)
    if keys.size:
        tg.evict_keys(torch.from_numpy(keys).to(DEV), torch.from_numpy(offs).to(DEV))


def test_key2offset_kat():
    # key_process_test.cpp:925-954 on distinct keys (the dedup in front removes the repeats)
    tg = host.EmbeddingTables([1000], 64)
    assert k2o(tg, [np.array([4, 16, 28, 24, 20])])[0].tolist() == [0, 1, 2, 3, 4]
    assert k2o(tg, [np.array([24, 4, 99])])[0].tolist() == [3, 0, 5]
    assert k2o(tg, [np.array([5, 17, 29, 25, 21])], channel=1)[0].tolist() == [-1] * 5
    assert tg.stats()[0] == [6]


def test_fill_overflow_eval_and_evict_reuse():
    # embedding_static_test.cpp:78-160
    tg = host.EmbeddingTables([100], 256)
    assert k2o(tg, [np.arange(100)])[0].tolist() == list(range(100))
    mo, live, ev = tg.stats()
    assert (mo, live, ev) == ([100], [100], [0])
    evict(tg, [np.arange(100)])
    assert tg.stats() == ([100], [0], [100])
    assert k2o(tg, [np.arange(10)])[0].tolist() == list(range(99, 89, -1))
    assert tg.evict_pos(0) == list(range(90))
    # overflow: the 101st key gets no slot and the group reports the overflow
    tg2 = host.EmbeddingTables([100], 256)
    out = k2o(tg2, [np.arange(101)])[0]
    assert out[:100].tolist() == list(range(100)) and out[100] == -1
    with pytest.raises(capi.RecsdkError) as e:
        tg2.stats()
    assert e.value.code == capi.EOVERFLOW
    tg3 = host.EmbeddingTables([100], 256)
    assert (k2o(tg3, [np.arange(100)], channel=1)[0] == -1).all()


def test_random_sequence_with_evictions_matches_oracle():
    rng = np.random.default_rng(0)
    vocab = [5000, 300, 70000]
    T = len(vocab)
    tg = host.EmbeddingTables(vocab, 40000)
    orc = [oracle.Table(v) for v in vocab]
    universe = [splitmix64(np.arange(v * 3, dtype=np.uint64) + np.uint64(t << 40)) for t, v in enumerate(vocab)]
    universe[0][7] = -2**63  # the erased-slot marker value is a legal key
    live = [set() for _ in range(T)]
    for step in range(12):
        tables = []
        for t in range(T):
            n = int(rng.integers(0, max(2, vocab[t] // 6)))
            k = rng.choice(universe[t], size=n, replace=False)
            k = np.where(rng.random(n) < 0.05, -1, k)
            # stay within capacity
            new = [x for x in dict.fromkeys(k.tolist()) if x != -1 and x not in live[t]]
            room = vocab[t] - len(live[t])
            drop = set(new[room:]) if len(new) > room else set()
            k = np.array([x for x in k.tolist() if x not in drop], dtype=np.int64)
            live[t].update(x for x in k.tolist() if x != -1)
            tables.append(k)
        channel = 1 if step % 5 == 4 else 0
        if channel == 1:
            for t in range(T):
                live[t].intersection_update(set())  # recomputed below from the oracle
        got = k2o(tg, tables, channel)
        for t in range(T):
            want, rc = orc[t].key2offset(tables[t], channel)
            assert rc == 0
            np.testing.assert_array_equal(got[t], want)
        if step % 3 == 2:
            ev = []
            for t in range(T):
                cur = np.array(sorted(live[t]), dtype=np.int64) if live[t] else np.zeros(0, np.int64)
                pick = rng.choice(cur, size=cur.size // 3, replace=False) if cur.size else cur
                pick = np.concatenate([pick, np.array([123456789, -1], dtype=np.int64)])  # absent / invalid keys
                ev.append(pick)
                orc[t].evict(pick)
                live[t].difference_update(pick.tolist())
            evict(tg, ev)
        mo, lv, evc = tg.stats()
        for t in range(T):
            assert mo[t] == orc[t].size and lv[t] == orc[t].live
            np.testing.assert_array_equal(np.array(tg.evict_pos(t), dtype=np.int64), orc[t].evict_pos)
        if channel == 1:
            # eval lookups insert nothing: rebuild the live sets from what the oracle holds
            for t in range(T):
                live[t] = {x for x in universe[t].tolist() if orc[t].key2offset([x], 1)[0][0] != -1}


def test_dynamic_tables_mint_addresses():
    base, rb = 0x7000000000, 3 * 32 * 4
    tg = host.EmbeddingTables([1000, 1000], 256, dynamic=[1, 0], arena_bases=[base, 0], row_bytes=[rb, 0])
    orc = oracle.Table(1000, dynamic=True, arena_base=base, row_bytes=rb)
    a = np.array([9, -1, 5, 11], dtype=np.int64)
    got = k2o(tg, [a, np.array([9, 5])])
    np.testing.assert_array_equal(got[0], orc.key2offset(a, 0)[0])
    assert got[1].tolist() == [0, 1]
    evict(tg, [np.array([9]), np.zeros(0, np.int64)])
    orc.evict([9])
    b = np.array([9, 6], dtype=np.int64)
    np.testing.assert_array_equal(k2o(tg, [b, np.zeros(0, np.int64)])[0], orc.key2offset(b, 0)[0])
    assert k2o(tg, [np.array([77]), np.array([77])], channel=1)[0].tolist() == [0]


def test_many_evictions_trigger_compaction_and_lookups_survive():
    vocab = 2400  # 1500 + 7 * 100 fresh slots are needed
    tg = host.EmbeddingTables([vocab], 4096)
    orc = oracle.Table(vocab)
    rng = np.random.default_rng(1)
    nxt = 0
    for _ in range(8):
        keys = splitmix64(np.arange(nxt, nxt + 1500, dtype=np.uint64))
        nxt += 1500
        got = k2o(tg, [keys])[0]
        want, _ = orc.key2offset(keys, 0)
        np.testing.assert_array_equal(got, want)
        evict(tg, [keys[:1400]])
        orc.evict(keys[:1400])
    survivors = np.concatenate([splitmix64(np.arange(s + 1400, s + 1500, dtype=np.uint64)) for s in range(0, nxt, 1500)])
    got = k2o(tg, [survivors], channel=1)[0]
    want, _ = orc.key2offset(survivors, 1)
    np.testing.assert_array_equal(got, want)
    assert (got >= 0).all()


def test_a_new_key_listed_twice_is_reported():
    """key2offset takes keys that are distinct per table (KeyProcess hands it the dedup's output).  A duplicated new
    key cannot be resolved by the rank-based slot assignment; the call flags it and stats() reports the table as bad
    instead of handing one key two slots silently."""
    tg = host.EmbeddingTables([100], 64)
    keys = torch.tensor([7, 8, 9], dtype=torch.int64, device=DEV)
    offs = torch.tensor([0, 3], dtype=torch.int64, device=DEV)
    tg.key2offset(keys, offs)
    tg.stats()
    dup = torch.tensor([7, 50, 51, 50], dtype=torch.int64, device=DEV)
    tg.key2offset(dup, torch.tensor([0, 4], dtype=torch.int64, device=DEV))
    with pytest.raises(capi.RecsdkError) as e:
        tg.stats()
    assert e.value.code == capi.EINVAL and "twice" in str(e.value)


def test_evictions_replayed_from_a_graph_are_counted_and_maintain_rebuilds_the_map():
    """A captured evict never re-enters host code, so the erased entries are counted on the device; the eager
    maintenance call reads the count, rebuilds the map, and every live key still resolves to its slot."""
    vocab = 4000                       # map of 8192 entries: a rebuild is due above 2048 erased ones
    tg = host.EmbeddingTables([vocab], 4096)
    orc = oracle.Table(vocab)
    kbuf = torch.zeros(900, dtype=torch.int64, device=DEV)
    obuf = torch.tensor([0, 900], dtype=torch.int64, device=DEV)
    # first eviction eagerly: the evicted-slot stack is allocated on first use
    keys = splitmix64(np.arange(0, 1000, dtype=np.uint64))
    np.testing.assert_array_equal(k2o(tg, [keys])[0], orc.key2offset(keys, 0)[0])
    kbuf.copy_(torch.from_numpy(keys[:900].astype(np.int64)))
    tg.evict_keys(kbuf, obuf)
    orc.evict(keys[:900])
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph(keep_graph=True)
    with torch.cuda.graph(g):
        tg.evict_keys(kbuf, obuf)
    assert "memset" not in host.graph_node_kinds(g.raw_cuda_graph())
    g.instantiate()
    assert tg.maintain() == 0          # 900 erased entries so far: nothing to do
    nxt = 1000
    for _ in range(3):
        keys = splitmix64(np.arange(nxt, nxt + 1000, dtype=np.uint64))
        nxt += 1000
        np.testing.assert_array_equal(k2o(tg, [keys])[0], orc.key2offset(keys, 0)[0])
        kbuf.copy_(torch.from_numpy(keys[:900].astype(np.int64)))
        g.replay()
        orc.evict(keys[:900])
    torch.cuda.synchronize()
    assert tg.maintain() == 1          # 3600 erased entries, 2700 of them by replays the host never saw
    assert tg.maintain() == 0
    survivors = np.concatenate([splitmix64(np.arange(s + 900, s + 1000, dtype=np.uint64)) for s in range(0, nxt, 1000)])
    got = k2o(tg, [survivors], channel=1)[0]
    want, _ = orc.key2offset(survivors, 1)
    np.testing.assert_array_equal(got, want)
    assert (got >= 0).all()
    # and the table goes on: new keys take the evicted slots last-evicted-first, as the oracle's
    more = splitmix64(np.arange(nxt, nxt + 500, dtype=np.uint64))
    np.testing.assert_array_equal(k2o(tg, [more])[0], orc.key2offset(more, 0)[0])
