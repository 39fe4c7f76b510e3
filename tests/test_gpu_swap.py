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
