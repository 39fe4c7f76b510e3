"""GPU parity: sharded unique (AccCTR DoEnhancedUnique outputs) and sorted unique (UniqueParallel) through the C ABI,
bit-exact against the CPU oracle."""
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


def compare(got, want):
    for name in ("unique_id", "index", "unique_id_in_bucket", "cnt_in_bucket", "id_cnt", "id_cnt_fill"):
        if want[name] is None:
            continue
        np.testing.assert_array_equal(got[name].cpu().numpy().astype(np.int64), want[name].astype(np.int64), err_msg=name)
    assert got["unique_id_cnt"] == want["unique_id_cnt"]


def test_reference_known_answer_padding():
    ids = np.array([4, 4, 5, 6, 4, 0], dtype=np.int64)
    su = host.ShardedUnique(64, sharding_num=2, use_sharding=True, use_padding=True, padding_size=4, padding_val=-1,
                            use_id_count=True)
    compare(su.do_enhanced_unique(dev(ids)), oracle.unique_sharded(ids, 2, 4, -1))


@pytest.mark.parametrize("n,universe,shards,padding,mask", [(1000, 700, 1, 0, False), (1000, 700, 7, 0, False),
                                                           (50000, 20000, 8, 0, True), (50000, 20000, 4, 6000, False),
                                                           (200000, 1 << 40, 64, 0, True), (3000, 100, 1024, 2, False)])
def test_random_matches_oracle(n, universe, shards, padding, mask):
    rng = np.random.default_rng(n + shards)
    ids = rng.integers(0, universe, n).astype(np.int64)
    su = host.ShardedUnique(n, sharding_num=shards, use_sharding=True, use_padding=padding > 0, padding_size=padding,
                            padding_val=-7, use_id_count=True, performance=mask)
    compare(su.do_enhanced_unique(dev(ids)), oracle.unique_sharded(ids, shards, padding, -7, use_mask=mask))
    # the handle is reusable: a second, smaller call
    ids2 = ids[: n // 3]
    compare(su.do_enhanced_unique(dev(ids2)), oracle.unique_sharded(ids2, shards, padding, -7, use_mask=mask))


def test_padding_too_small_reports_capacity():
    su = host.ShardedUnique(64, sharding_num=2, use_sharding=True, use_padding=True, padding_size=1, use_id_count=True)
    with pytest.raises(capi.RecsdkError) as e:
        su.do_enhanced_unique(dev([0, 2, 1]))
    assert e.value.code == capi.ECAPACITY


def test_empty_input():
    su = host.ShardedUnique(64, sharding_num=4, use_sharding=True, use_id_count=True)
    r = su.do_enhanced_unique(dev(np.zeros(0, np.int64)))
    assert r["unique_id_cnt"] == 0 and r["cnt_in_bucket"].cpu().tolist() == [0, 0, 0, 0]


@pytest.mark.parametrize("n", [1, 100, 65536, 300000])
def test_sorted_unique_matches_oracle(n):
    rng = np.random.default_rng(n)
    ids = rng.integers(-(1 << 62), 1 << 62, n).astype(np.int64)
    ids[rng.integers(0, n, n // 2)] = ids[0]
    ids[rng.integers(0, n, n // 8)] = -1
    got_u, got_inv = host.unique_parallel(dev(ids))
    want_u, want_inv = oracle.unique_sorted(ids)
    np.testing.assert_array_equal(got_u.cpu().numpy(), want_u)
    np.testing.assert_array_equal(got_inv.cpu().numpy(), want_inv)


@pytest.mark.parametrize("case", ["one_key", "two_keys_low_bit", "below_2_32", "negative_only", "around_zero",
                                  "shared_high_bits", "extremes"])
def test_sorted_unique_key_ranges(case):
    """The sort runs over the bits in which the distinct keys differ: ranges that make that one bit, 32 bits, the
    sign bit alone, a window in the middle of the word, and all 64."""
    rng = np.random.default_rng(11)
    n = 20000
    if case == "one_key":
        ids = np.full(n, 123456789012345, np.int64)
    elif case == "two_keys_low_bit":
        ids = (rng.integers(0, 2, n) + (1 << 40)).astype(np.int64)
    elif case == "below_2_32":
        ids = rng.integers(0, 1 << 32, n).astype(np.int64)
    elif case == "negative_only":
        ids = -rng.integers(1, 1 << 20, n).astype(np.int64)
    elif case == "around_zero":
        ids = rng.integers(-3, 4, n).astype(np.int64)
    elif case == "shared_high_bits":
        ids = ((0x5A5A << 44) + (rng.integers(0, 1 << 12, n) << 20) + 77).astype(np.int64)
    else:
        ids = rng.choice(np.array([np.iinfo(np.int64).min, np.iinfo(np.int64).max, 0, -1, 1], np.int64), n)
    got_u, got_inv = host.unique_parallel(dev(ids))
    want_u, want_inv = oracle.unique_sorted(ids)
    np.testing.assert_array_equal(got_u.cpu().numpy(), want_u)
    np.testing.assert_array_equal(got_inv.cpu().numpy(), want_inv)


def test_sorted_unique_zipf_full_batch():
    rng = np.random.default_rng(0)
    ids = zipf_ranks(rng, 1.05, 8_000_000, 65536 * 26).astype(np.int64)
    got_u, got_inv = host.unique_parallel(dev(ids))
    # size-independent properties: sorted, strictly increasing, inverse restores the input
    assert bool((got_u[1:] > got_u[:-1]).all())
    assert bool((got_u[got_inv] == dev(ids)).all())
