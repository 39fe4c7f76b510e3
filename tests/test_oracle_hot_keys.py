"""Pins the oracle's hot-key restatement (KeyProcess::HotHashSplit / UpdateHotMap, rankSize 1).

The reference holds no known-answer test for this path (key_process_test.cpp only prints the results), so the
restatement is checked against an independent model built from what the operation means rather than how it loops:
numpy first-occurrence dedup, a cumulative count over "is hot" flags, and a plain sort for the top-k refresh; plus
invariants that a dropped offset, an off-by-one in the non-hot branch or a wrong tie-break would break."""
import collections

import numpy as np
import pytest

import oracle


def model_split(keys, hot_set, tot):
    uniq, first, inverse, counts = np.unique(keys, return_index=True, return_inverse=True, return_counts=True)
    order = np.argsort(first, kind="stable")          # distinct keys by first occurrence
    rank_of = np.empty_like(order)
    rank_of[order] = np.arange(order.size)
    split = uniq[order]
    is_hot = np.array([k in hot_set for k in split.tolist()], dtype=bool)
    hot_index = np.cumsum(is_hot) - 1
    per_unique = np.where(is_hot, hot_index, np.arange(split.size) + tot).astype(np.int32)
    restore = per_unique[rank_of[inverse]] if keys.size else np.zeros(0, np.int32)
    hot_pos = np.zeros(tot, dtype=np.int32)
    hot_pos[:int(is_hot.sum())] = np.nonzero(is_hot)[0]
    return split, restore, hot_pos, counts[order].astype(np.uint32)


def model_refresh(keys, tot):
    c = collections.Counter(keys.tolist())
    return set(k for k, _ in sorted(c.items(), key=lambda kv: (-kv[1], kv[0]))[:tot])


def zipf_keys(rng, n, universe, a=1.2):
    return (rng.zipf(a, size=n) % universe).astype(np.int64) * 7919 - 3


@pytest.mark.parametrize("seed,n,universe,tot", [(0, 0, 10, 4), (1, 1, 10, 4), (2, 300, 40, 8), (3, 5000, 700, 64),
                                                 (4, 5000, 50, 64), (5, 4096, 100000, 0), (6, 777, 3, 1)])
def test_hot_hash_split_matches_model(seed, n, universe, tot):
    rng = np.random.default_rng(seed)
    orc = oracle.HotKeys(tot)
    hot_set = set()
    for batch_id in range(7):
        keys = zipf_keys(rng, n, universe)
        refresh = batch_id % 3 == 0
        split, restore, hot_pos, cnt = orc.hot_hash_split(keys, refresh)
        m_split, m_restore, m_hot_pos, m_cnt = model_split(keys, hot_set, tot)
        np.testing.assert_array_equal(split, m_split)
        np.testing.assert_array_equal(restore, m_restore)
        np.testing.assert_array_equal(hot_pos, m_hot_pos)
        np.testing.assert_array_equal(cnt, m_cnt)
        if refresh:
            hot_set = model_refresh(keys, tot)
        np.testing.assert_array_equal(orc.hot_keys(), np.array(sorted(hot_set), dtype=np.int64))


def test_first_batch_has_no_hot_keys_and_refresh_takes_effect_next_batch():
    orc = oracle.HotKeys(2)
    keys = np.array([5, 9, 5, 7, 9, 5, 1], dtype=np.int64)
    split, restore, hot_pos, cnt = orc.hot_hash_split(keys, True)
    # hot set empty: restore = unique index + hotOffset, hot_pos all zero
    np.testing.assert_array_equal(split, [5, 9, 7, 1])
    np.testing.assert_array_equal(restore, [2, 3, 2, 4, 3, 2, 5])
    np.testing.assert_array_equal(hot_pos, [0, 0])
    np.testing.assert_array_equal(cnt, [3, 2, 1, 1])
    np.testing.assert_array_equal(orc.hot_keys(), [5, 9])
    # next batch: 9 first -> hot index 0 at unique position 1; 5 -> hot index 1 at unique position 2
    keys = np.array([4, 9, 5, 9, 4, 8], dtype=np.int64)
    split, restore, hot_pos, _ = orc.hot_hash_split(keys, False)
    np.testing.assert_array_equal(split, [4, 9, 5, 8])
    np.testing.assert_array_equal(restore, [2, 0, 1, 0, 2, 5])
    np.testing.assert_array_equal(hot_pos, [1, 2])
    np.testing.assert_array_equal(orc.hot_keys(), [5, 9])   # no refresh: unchanged


def test_refresh_tie_goes_to_smaller_key():
    orc = oracle.HotKeys(2)
    orc.hot_hash_split(np.array([30, 10, 20, 20, 10, 30, 40], dtype=np.int64), True)
    np.testing.assert_array_equal(orc.hot_keys(), [10, 20])


@pytest.mark.parametrize("seed", range(4))
def test_restore_gathers_back_the_keys(seed):
    """Staging invariant: with the hot rows laid out first (hot_pos picks them from the distinct keys) and the
    distinct keys after them, indexing that layout with restore gives back the batch."""
    rng = np.random.default_rng(100 + seed)
    tot = 16
    orc = oracle.HotKeys(tot)
    for batch_id in range(4):
        keys = zipf_keys(rng, 2000, 300)
        split, restore, hot_pos, cnt = orc.hot_hash_split(keys, batch_id % 2 == 0)
        staged = np.concatenate([split[hot_pos], split])
        np.testing.assert_array_equal(staged[restore], keys)
        assert cnt.sum() == keys.size
