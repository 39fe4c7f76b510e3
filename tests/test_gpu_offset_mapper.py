"""GPU parity: the TF path's HBM-cache planner (AccCTR OffsetMapper) through the C ABI, bit-exact against the CPU
oracle (which tests/test_oracle_offset_mapper.py pins)."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)).to(DEV)


def check_step(om, orc, keys):
    want = orc.get_swap_pairs_and_key2offset(keys)
    d = dev(keys)
    got = om.get_swap_pairs_and_key2offset(d)
    np.testing.assert_array_equal(d.cpu().numpy(), want[0], err_msg="offsets")
    for name, g, w in zip(("swapin_keys", "swapin_pos", "swapout_keys", "swapout_pos"), got, want[1:]):
        np.testing.assert_array_equal(g.cpu().numpy(), w, err_msg=name)


def check_state(om, orc):
    st = orc.state()
    _, _, use, ev = om.counts()
    assert (use, ev) == (st["use_length"], st["evict_size"])
    k, s = om.export_sorted_kv_pairs()
    np.testing.assert_array_equal(k.cpu().numpy(), st["keys"])
    np.testing.assert_array_equal(s.cpu().numpy(), st["slots"])


def test_reference_cases():
    om, orc = host.OffsetMapper(10, max_keys=64), oracle.OffsetMapper(10)
    for keys in ([0, 1, 2, 3, 4], [1, 2, 3], list(range(10))):
        check_step(om, orc, np.array(keys))
    with pytest.raises(RuntimeError):
        orc.get_swap_pairs_and_key2offset(np.arange(11))
    with pytest.raises(capi.RecsdkError) as e:
        om.get_swap_pairs_and_key2offset(dev(np.arange(11)))
    assert e.value.code == capi.EOVERFLOW
    om, orc = host.OffsetMapper(10, max_keys=64), oracle.OffsetMapper(10)
    for keys in ([0, 1, 2, 3, 4], [5, 6, 7, 8, 9], [10, 11, 12, 13, 14]):
        check_step(om, orc, np.array(keys))
    check_state(om, orc)
    om, orc = host.OffsetMapper(10, max_keys=64), oracle.OffsetMapper(10)
    check_step(om, orc, np.full(5, -1))
    check_step(om, orc, np.zeros(0, np.int64))


def test_remove_and_reuse():
    om, orc = host.OffsetMapper(10, max_keys=64), oracle.OffsetMapper(10)
    check_step(om, orc, np.arange(10))
    orc.remove(np.arange(10))
    om.remove(dev(np.arange(10)))
    check_state(om, orc)
    check_step(om, orc, np.array([9, 10, 11, 12, 13]))
    orc.remove(np.array([9, 10, 11, 3]))
    om.remove(dev([9, 10, 11, 3]))
    check_step(om, orc, np.arange(8))
    check_step(om, orc, np.array([15]))
    check_state(om, orc)


@pytest.mark.parametrize("cache,universe,batch", [(64, 200, 20), (500, 5000, 150), (30000, 100000, 9500),
                                                  (4096, 6000, 1300)])
def test_sequences_match_oracle(cache, universe, batch):
    rng = np.random.default_rng(cache)
    om, orc = host.OffsetMapper(cache, max_keys=batch + 64), oracle.OffsetMapper(cache)
    for step in range(40):
        n = int(rng.integers(batch // 2, batch + 1))
        keys = rng.choice(universe, size=n, replace=False).astype(np.int64)
        keys = np.where(rng.random(n) < 0.03, -1, keys)
        check_step(om, orc, keys)
        if step % 6 == 5:
            rm = rng.choice(universe, size=min(batch, universe) // 4, replace=False).astype(np.int64)
            orc.remove(rm)
            om.remove(dev(rm))
    check_state(om, orc)


def test_map_rebuild_keeps_sequence():
    # small cache, many calls: the key->slot map is rebuilt several times on the way
    rng = np.random.default_rng(9)
    om, orc = host.OffsetMapper(128, max_keys=64), oracle.OffsetMapper(128)
    for step in range(300):
        keys = rng.choice(4000, size=40, replace=False).astype(np.int64)
        check_step(om, orc, keys)
    check_state(om, orc)


@pytest.mark.parametrize("seed", range(12))
def test_sequences_with_random_geometry_match_oracle(seed):
    """Cache sizes, key universes and batch sizes drawn at random."""
    rng = np.random.default_rng(700 + seed)
    cache = int(rng.integers(32, 20000))
    universe = int(rng.integers(cache * 2, cache * 10))
    batch = int(rng.integers(4, max(5, cache // 3)))
    test_sequences_match_oracle(cache, universe, batch)
