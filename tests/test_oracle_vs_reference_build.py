"""The CPU oracle's restatement of the torch-side planners checked against the REFERENCE's own code, compiled from
the reference checkout into oracle/_ref/libref_torch.so (make -C oracle -f ref.mk).  Skipped where that library
is absent."""
import numpy as np
import pytest

import oracle
from oracle import ref_loader

pytestmark = pytest.mark.skipif(not ref_loader.available(), reason="oracle/_ref/libref_torch.so not built")


@pytest.mark.parametrize("cache,mem_start,universe", [(64, 0, 200), (300, 1, 1000), (50, 0, 40)])
def test_swap_manager_sequences_match_reference(cache, mem_start, universe):
    rng = np.random.default_rng(cache)
    ref = ref_loader.RefSwap(cache, mem_start)
    orc = oracle.Swap(cache, mem_start)
    for step in range(60):
        n = int(rng.integers(1, max(2, (cache - mem_start) // 3)))
        keys = rng.integers(0, universe, n)
        keys = np.where(rng.random(n) < 0.05, -1, keys)
        try:
            want = ref.compute_swap_info(keys)
        except RuntimeError:
            with pytest.raises(RuntimeError):
                orc.compute_swap_info(keys)
            break
        got = orc.compute_swap_info(keys)
        for g, w in zip(got, want):
            np.testing.assert_array_equal(g, w)
        if step % 7 == 6:
            rm = rng.integers(0, universe, 10)
            ref.remove_keys(rm)
            orc.remove_keys(rm)


def test_swap_manager_too_small_raises_like_reference():
    ref = ref_loader.RefSwap(8)
    orc = oracle.Swap(8)
    ref.compute_swap_info(np.arange(8))
    orc.compute_swap_info(np.arange(8))
    with pytest.raises(RuntimeError):
        ref.compute_swap_info(np.arange(100, 105))
    with pytest.raises(RuntimeError):
        orc.compute_swap_info(np.arange(100, 105))


def test_feature_filter_matches_reference():
    rng = np.random.default_rng(3)
    ref = ref_loader.RefFilter(3, 4, 2)
    orc = oracle.Filter(3, 4, 2)
    for step in range(14):
        keys = rng.integers(0, 80, 50)
        counts = rng.integers(-1, 4, 50)
        ref.statistics_key_count(keys, counts)
        orc.statistics_key_count(keys, counts)
        np.testing.assert_array_equal(orc.count_filter(keys), ref.count_filter(keys))
        stamps = step + rng.integers(0, 2, 50)
        ev_ref = ref.record_timestamp(keys, stamps)
        ev_orc = orc.record_timestamp(keys, stamps)
        # the reference emits evicted keys in hash-map order: compare as sets
        assert sorted(ev_ref.tolist()) == sorted([] if ev_orc is None else ev_orc.tolist())


def test_ids_mapper_matches_dedup_plus_slot_assignment():
    """ParallelUniqueHashOut == first-occurrence dedup per table + first-seen slot numbers (oracle.hash_split +
    oracle.Table.key2offset), which is how the device path composes it."""
    rng = np.random.default_rng(4)
    T = 3
    ref = ref_loader.RefIdsMapper([10**6] * T)
    tabs = [oracle.Table(10**6) for _ in range(T)]
    for _ in range(5):
        lens = rng.integers(0, 400, T)
        offs = np.concatenate([[0], np.cumsum(lens)])
        ids = rng.integers(0, 300, int(offs[-1]))
        hash_idx, uniq, uniq_ids, inv, uoff = ref.parallel_unique_hash_out(ids, offs)
        for t in range(T):
            seg = ids[offs[t]:offs[t + 1]]
            split, _, restore, _ = oracle.hash_split(seg, 1)
            slots, _ = tabs[t].key2offset(split, 0)
            assert uoff[t + 1] - uoff[t] == split.size
            np.testing.assert_array_equal(uniq_ids[uoff[t]:uoff[t + 1]], split)
            np.testing.assert_array_equal(uniq[uoff[t]:uoff[t + 1]], slots)
            np.testing.assert_array_equal(inv[offs[t]:offs[t + 1]], restore)
            np.testing.assert_array_equal(hash_idx[offs[t]:offs[t + 1]], slots[restore])
