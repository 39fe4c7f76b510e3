"""GPU parity: version-clock HBM-cache planner (SwapManager) and IdsMapper through the C ABI vs the CPU oracle
(which tests/test_oracle_vs_reference_build.py checks against the reference's own code)."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host
from recsdk_amd.synth import zipf_ranks

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)).to(DEV)


def check_step(sm, orc, keys):
    want = orc.compute_swap_info(keys)
    got = sm.compute_swap_info(dev(keys))
    for g, w in zip(got, want):
        np.testing.assert_array_equal(g.cpu().numpy(), w)


@pytest.mark.parametrize("cache,mem_start,universe,alpha", [(64, 0, 200, None), (300, 1, 1000, None),
                                                           (5000, 0, 40000, 1.05), (2048, 1, 3000, 1.2)])
def test_sequences_match_oracle(cache, mem_start, universe, alpha):
    rng = np.random.default_rng(cache)
    sm = host.SwapManager(cache, mem_start, max_keys=4096)
    orc = oracle.Swap(cache, mem_start)
    for step in range(40):
        n = int(rng.integers(1, max(2, (cache - mem_start) // 3)))
        keys = zipf_ranks(rng, alpha, universe, n) if alpha else rng.integers(0, universe, n)
        keys = np.where(rng.random(n) < 0.05, -1, keys)
        check_step(sm, orc, keys)
        if step % 7 == 6:
            rm = rng.integers(0, universe, 20)
            orc.remove_keys(rm)
            sm.remove_keys(dev(rm))
    assert sm.counts()[2] <= cache


def test_empty_batch_and_all_invalid():
    sm = host.SwapManager(16, max_keys=64)
    orc = oracle.Swap(16)
    check_step(sm, orc, np.zeros(0, np.int64))
    check_step(sm, orc, np.full(5, -1))
    check_step(sm, orc, np.array([3, 3, -1, 4]))


def test_cache_too_small_is_reported_and_state_kept():
    sm = host.SwapManager(8, max_keys=64)
    orc = oracle.Swap(8)
    check_step(sm, orc, np.arange(8))
    with pytest.raises(RuntimeError):
        orc.compute_swap_info(np.arange(100, 105))
    with pytest.raises(capi.RecsdkError) as e:
        sm.compute_swap_info(dev(np.arange(100, 105)))
    assert e.value.code == capi.EOVERFLOW
    # the resident keys are still where they were
    bufs = [torch.empty(8, dtype=torch.int64, device=DEV) for _ in range(5)]
    keys = dev(np.arange(8))
    capi.check(capi.lib().recsdk_swap_compute(sm.h, keys.data_ptr(), 8, *[b.data_ptr() for b in bufs], None))
    torch.cuda.synchronize()
    assert bufs[4].cpu().tolist() == list(range(8))


def test_fresh_slots_of_the_same_call_are_never_victims():
    """A batch whose misses first fill the never-used slots and then need victims: the slots being filled in this very
    call carry the current version in the sequential planner (swap_manager.cpp:88-96), so the sweep may not hand them
    out a second time.  cache 10, [1,2,3,4] twice, then [1,2,3,4,11..18]: 6 fresh slots, 2 victims needed, none
    eligible (slots 0-3 were used in the batch before) -> "cacheSize_ too small", state as it was."""
    sm = host.SwapManager(10, max_keys=64)
    orc = oracle.Swap(10)
    check_step(sm, orc, np.array([1, 2, 3, 4]))
    check_step(sm, orc, np.array([1, 2, 3, 4]))
    big = np.array([1, 2, 3, 4, 11, 12, 13, 14, 15, 16, 17, 18])
    with pytest.raises(RuntimeError):
        orc.compute_swap_info(big)
    with pytest.raises(capi.RecsdkError) as e:
        sm.compute_swap_info(dev(big))
    assert e.value.code == capi.EOVERFLOW
    import ctypes
    occ = ctypes.c_int64()
    rc = capi.lib().recsdk_swap_counts(sm.h, None, None, None, ctypes.byref(occ))   # still reports the failed batch
    assert rc == capi.EOVERFLOW and occ.value == 4   # occupied as before
    # the planner goes on from the state it had: the failed batch left only its hit stamps and one version tick, which
    # is what a batch of its hits alone leaves in a fresh sequential planner (the reference's is half updated by now)
    orc3 = oracle.Swap(10)
    for _ in range(3):
        orc3.compute_swap_info(np.array([1, 2, 3, 4]))
    check_step(sm, orc3, np.array([1, 2, 3, 4, 11, 12]))
    check_step(sm, orc3, np.array([1, 2]))
    check_step(sm, orc3, np.array([30, 31, 32, 33, 34, 35]))   # 4 never-used slots, then 2 victims
    # a variant that does fit: old occupied slots exist, fresh slots are filled first, victims come from the old ones
    sm2 = host.SwapManager(10, max_keys=64)
    orc2 = oracle.Swap(10)
    for keys in ([1, 2, 3, 4], [5, 6], [7], [20, 21, 22, 23, 24, 25], [1, 30, 31, 32]):
        check_step(sm2, orc2, np.array(keys))


def test_many_steps_rebuild_the_map():
    """Churn far beyond the map's capacity: the key -> offset map is rebuilt on the way and stays consistent."""
    cache = 256
    rng = np.random.default_rng(9)
    sm = host.SwapManager(cache, max_keys=128)
    orc = oracle.Swap(cache)
    for step in range(120):
        keys = rng.integers(step * 50, step * 50 + 400, 100)
        check_step(sm, orc, keys)


def test_ids_mapper_matches_oracle_composition():
    rng = np.random.default_rng(4)
    T = 3
    im = host.IdsMapper([10**5] * T, 4096)
    tabs = [oracle.Table(10**5) for _ in range(T)]
    for _ in range(5):
        lens = rng.integers(0, 900, T)
        offs = np.concatenate([[0], np.cumsum(lens)])
        ids = rng.integers(0, 500, int(offs[-1]))
        hash_idx, uniq, uniq_ids, inv, uoff = im.parallel_unique_hash_out(dev(ids), dev(offs))
        hash_idx, uniq, uniq_ids, inv, uoff = (x.cpu().numpy() for x in (hash_idx, uniq, uniq_ids, inv, uoff))
        for t in range(T):
            seg = ids[offs[t]:offs[t + 1]]
            split, _, restore, _ = oracle.hash_split(seg, 1)
            slots, _ = tabs[t].key2offset(split, 0)
            np.testing.assert_array_equal(uniq_ids[uoff[t]:uoff[t + 1]], split)
            np.testing.assert_array_equal(uniq[uoff[t]:uoff[t + 1]], slots)
            np.testing.assert_array_equal(inv[offs[t]:offs[t + 1]], restore)
            np.testing.assert_array_equal(hash_idx[offs[t]:offs[t + 1]], slots[restore])
    assert im.max_index() == [t.size for t in tabs]


@pytest.mark.parametrize("seed", range(12))
def test_sequences_with_random_geometry_match_oracle(seed):
    """Cache sizes, reserved prefixes, key universes and skews drawn at random."""
    rng = np.random.default_rng(900 + seed)
    cache = int(rng.integers(16, 12000))
    mem_start = int(rng.integers(0, 2))
    universe = int(rng.integers(cache // 2 + 2, cache * 8))
    alpha = [None, 1.05, 1.2][int(rng.integers(0, 3))]
    test_sequences_match_oracle(cache, mem_start, universe, alpha)
