"""Pins the CPU oracle's integer half against the reference's own known-answer vectors and brute force.

KAT sources (reference checkout):
  training/tf_rec_v1/src/tests/key_process/key_process_test.cpp:744-787   HashSplit / HashSplitWithFAAE
  training/tf_rec_v1/src/tests/key_process/key_process_test.cpp:855-885   BuildRestoreVec, 4 ranks
  training/tf_rec_v1/src/tests/key_process/key_process_test.cpp:925-954   Key2Offset train / eval
  training/tf_rec_v1/src/tests/emb_table/embedding_static_test.cpp:78-160 fill, overflow, eval, evict + reuse
  training/tf_rec_v1/src/tests/key_process/feature_admit_and_evict_test.cpp:283-325,405-421 admit / evict
"""
import numpy as np
import pytest

import oracle

BATCH = [1, 4, 23, 14, 16, 7, 2, 21, 21, 29]


def test_hash_split_kat():
    split, offs, restore, counts = oracle.hash_split(BATCH, rank_size=4)
    buckets = [split[offs[d]:offs[d + 1]].tolist() for d in range(4)]
    assert buckets == [[4, 16], [1, 21, 29], [14, 2], [23, 7]]
    assert restore.tolist() == [0, 0, 0, 0, 1, 1, 1, 1, 1, 2]
    cnt = [counts[offs[d]:offs[d + 1]].tolist() for d in range(4)]
    assert cnt == [[1, 1], [1, 2, 1], [1, 1], [1, 1]]


def test_build_restore_vec_kat_4_ranks():
    all_keys = [[1, 4, 23, 14, 16, 7, 2, 21, 21, 29],
                [5, 17, 26, 9, 27, 22, 27, 28, 15, 3],
                [10, 4, 22, 17, 24, 13, 24, 26, 29, 11],
                [14, 21, 18, 25, 21, 4, 20, 24, 13, 19]]
    all_ss = [[0, 2, 5, 7, 9], [0, 1, 4, 6], [0, 2, 5, 8], [0, 3, 6, 8]]
    expect = [[2, 0, 7, 5, 1, 8, 6, 3, 3, 4],
              [1, 2, 4, 3, 6, 5, 6, 0, 7, 8],
              [5, 0, 6, 2, 1, 3, 1, 7, 4, 8],
              [6, 3, 7, 4, 3, 0, 1, 2, 5, 8]]
    for keys, ss, exp in zip(all_keys, all_ss, expect):
        _, _, restore, _ = oracle.hash_split(keys, rank_size=4)
        out = oracle.build_restore_vec(keys, 4, ss[:4], restore)
        assert out.tolist() == exp


def first_occurrence_unique(keys):
    """Brute force with numpy: distinct keys in order of first occurrence, inverse, counts."""
    keys = np.asarray(keys, dtype=np.int64)
    uniq_sorted, first_idx, inv_sorted, cnt_sorted = np.unique(keys, return_index=True, return_inverse=True,
                                                               return_counts=True)
    order = np.argsort(first_idx, kind="stable")
    rank_of_sorted = np.empty_like(order)
    rank_of_sorted[order] = np.arange(order.size)
    return uniq_sorted[order], rank_of_sorted[inv_sorted], cnt_sorted[order]


@pytest.mark.parametrize("seed,n,hi", [(0, 1, 3), (1, 1000, 50), (2, 5000, 10**12), (3, 4096, 4)])
def test_hash_split_rank1_matches_numpy_bruteforce(seed, n, hi):
    rng = np.random.default_rng(seed)
    keys = rng.integers(-hi, hi, n)
    split, offs, restore, counts = oracle.hash_split(keys, rank_size=1)
    u, inv, cnt = first_occurrence_unique(keys)
    assert split.tolist() == u.tolist()
    assert restore.tolist() == inv.tolist()
    assert counts.tolist() == cnt.tolist()
    assert offs.tolist() == [0, u.size]


def test_hash_split_negative_keys_bucket_by_abs_mod():
    keys = np.array([-5, 5, -6, 7, -5], dtype=np.int64)
    split, offs, restore, _ = oracle.hash_split(keys, rank_size=4)
    buckets = [split[offs[d]:offs[d + 1]].tolist() for d in range(4)]
    assert buckets == [[], [-5, 5], [-6], [7]]
    assert restore.tolist() == [0, 1, 0, 0, 0]


@pytest.mark.parametrize("use_static,dyn", [(False, False), (True, False), (True, True)])
def test_global_unique_matches_bruteforce(use_static, dyn):
    rng = np.random.default_rng(7)
    keys = rng.integers(-1, 6, 200)  # contains the padding values -1 and 0
    uniq, rvs, u = oracle.global_unique(keys, use_static, dyn)
    pad = 0 if dyn else -1
    valid = np.ones(keys.size, bool) if not use_static else keys != pad
    bu, binv, _ = first_occurrence_unique(keys[valid])
    assert u == bu.size
    assert uniq[:u].tolist() == bu.tolist()
    assert rvs[valid].tolist() == binv.tolist()
    assert (rvs[~valid] == -1).all()
    if use_static:
        assert uniq.size == keys.size and (uniq[u:] == pad).all()


def test_key2offset_kat():
    t = oracle.Table(1000)
    out, rc = t.key2offset([4, 16, 28, 4, 24, 4, 20, 24], channel=0)
    assert rc == 0 and out.tolist() == [0, 1, 2, 0, 3, 0, 4, 3]
    out, rc = t.key2offset([5, 17, 29, 5, 25, 5, 21, 25], channel=1)
    assert out.tolist() == [-1] * 8
    assert t.size == 5


def test_static_table_fill_overflow_eval_and_evict_reuse():
    t = oracle.Table(100)
    out, rc = t.key2offset(np.arange(100), 0)
    assert rc == 0 and out.tolist() == list(range(100)) and t.size == 100
    t2 = oracle.Table(100)
    _, rc = t2.key2offset(np.arange(101), 0)
    assert rc == -1  # the reference throws std::runtime_error here
    t3 = oracle.Table(100)
    out, _ = t3.key2offset(np.arange(100), 1)
    assert (out == -1).all()
    # evict everything, then 10 new keys reuse evicted slots last-evicted-first: 90 left
    assert t.evict(np.arange(100)) == 100
    out, rc = t.key2offset(np.arange(10), 0)
    assert rc == 0 and out.tolist() == list(range(99, 89, -1))
    assert t.evict_pos.tolist() == list(range(90))
    assert t.size == 100


def test_static_table_skips_invalid_and_reuses_once_per_distinct_key():
    t = oracle.Table(10)
    t.key2offset([1, 2, 3], 0)
    t.evict([2, -1, 99])
    out, _ = t.key2offset([-1, 7, 7, 8], 0)
    assert out.tolist() == [-1, 1, 1, 3]


def test_dynamic_table_mints_addresses_in_order_and_never_reuses():
    base, rb = 0x10000, 48
    t = oracle.Table(1000, dynamic=True, arena_base=base, row_bytes=rb)
    out, _ = t.key2offset([9, -1, 5, 9], 0)
    assert out.tolist() == [base, 0, base + rb, base]
    t.evict([9])
    out, _ = t.key2offset([9, 6], 0)
    assert out.tolist() == [base + 2 * rb, base + 3 * rb]
    out, _ = t.key2offset([77], 1)
    assert out.tolist() == [0]


def test_feature_admit_and_evict_kat():
    t0 = 1000
    aaa = oracle.Faae(2, 5)
    bbb = oracle.Faae(3, 7)
    r = aaa.admit([11, 11, 33, 44, 11, 55, 88, 55], [1, 2, 1, 3, 1, 1, 4, 1], t0)
    assert r.tolist() == [11, 11, -1, 44, 11, 55, 88, 55]
    r = aaa.admit([11, 12, 33, 21, 11, 12], [1, 2, 1, 1, 2, 3], t0 + 1)
    assert r.tolist() == [11, 12, 33, -1, 11, 12]
    assert aaa.evict().size == 0  # nothing is idle yet (table time is the last batch's timestamp)
    r = bbb.admit([123, 121, 121, 212, 211], [1, 2, 1, 1, 2], t0 + 3)
    assert r.tolist() == [-1, 121, 121, -1, -1]
    r = aaa.admit([11, 11, 33, 44, 55, 88, 55], [1, 2, 3, 2, 1, 2, 1], t0 + 9)
    assert r.tolist() == [11, 11, 33, 44, 55, 88, 55]
    r = bbb.admit([125, 121, 122, 212, 211], [1, 2, 1, 3, 1], t0 + 11)
    assert r.tolist() == [-1, 121, -1, 212, 211]
    assert sorted(aaa.evict().tolist()) == [12, 21]
    assert sorted(bbb.evict().tolist()) == [123]
    k, c, _ = aaa.dump()
    assert dict(zip(k.tolist(), c.tolist())) == {11: 10, 33: 5, 44: 5, 55: 4, 88: 6}
    k, c, _ = bbb.dump()
    assert dict(zip(k.tolist(), c.tolist())) == {121: 5, 122: 1, 125: 1, 211: 3, 212: 4}


def test_faae_eval_channel_and_no_sum_do_not_touch_history():
    f = oracle.Faae(2, 5)
    assert f.admit([7, 8], [5, 5], 10, channel=1).tolist() == [-1, -1]
    assert f.dump()[0].size == 0
    g = oracle.Faae(2, 5, coef=3, is_enable_sum=True)
    assert g.admit([7], [1], 10).tolist() == [7]  # 1 * coef 3 >= 2
    h = oracle.Faae(2, 5, is_enable_sum=False)
    assert h.admit([7], [9], 10).tolist() == [-1]


def test_torch_feature_filter_against_dict_model():
    """The reference holds no known-answer vector for FeatureFilter; the oracle is checked against a plain
    dict model written from feature_filter.cpp:27-80,112-160 on a random stream (parity otherwise unpinned)."""
    rng = np.random.default_rng(11)
    f = oracle.Filter(admit_threshold=3, evict_threshold=4, evict_step_interval=2)
    cnt, ts, latest, batch = {}, {}, 0, 0
    for step in range(12):
        keys = rng.integers(0, 60, 40)
        counts = rng.integers(-1, 4, 40)
        f.statistics_key_count(keys, counts)
        for k, c in zip(keys.tolist(), counts.tolist()):
            cnt[k] = cnt.get(k, 0) + max(c, 0)
        got = f.count_filter(keys)
        want = np.array([-1 if (k in cnt and cnt[k] < 3) else k for k in keys.tolist()])
        np.testing.assert_array_equal(got, want)
        stamps = np.full(40, step) + rng.integers(0, 2, 40)
        ev = f.record_timestamp(keys, stamps)
        for k, t in zip(keys.tolist(), stamps.tolist()):
            ts[k] = t
            latest = max(latest, t)
        if batch > 0 and (batch + 1) % 2 == 0:
            gone = sorted((t, k) for k, t in ts.items() if latest - t > 4)
            assert ev.tolist() == [k for _, k in gone]
            for _, k in gone:
                del ts[k]
                cnt.pop(k, None)
        else:
            assert ev is None
        batch += 1
