"""CPU checks that pin the oracle's sharded unique (AccCTR DoEnhancedUnique) and sorted unique (UniqueParallel).

Sharded unique: the known-answer inputs and every assertion of the reference's tests
(AccCTR/tests/ut/src/unique_test.cpp:573-655 sharding, :716-797 padding, :866-945 seven shards), plus a numpy brute
force of the layout.  Sorted unique: numpy.unique, and the reference's own UniqueParallel where oracle/_ref is built.
"""
import numpy as np
import pytest

import oracle
from oracle import ref_loader


def reference_assertions(ids, r, shards, padding_size):
    """What unique_test.cpp asserts on the enhanced outputs."""
    ids = np.asarray(ids, dtype=np.int64)
    np.testing.assert_array_equal(r["unique_id"][r["index"]], ids)                       # restoreIds == inputId
    first_seen = list(dict.fromkeys(ids.tolist()))
    expect_cnt = np.bincount(np.array(first_seen, dtype=np.uint64) % np.uint64(shards), minlength=shards)
    np.testing.assert_array_equal(r["cnt_in_bucket"], expect_cnt)                        # uniqueIdCntInBucket
    mult = {k: int(c) for k, c in zip(*np.unique(ids, return_counts=True))}
    if padding_size:
        assert r["unique_id_cnt"] == shards * padding_size
        want = [0 if k == -1 else mult[k] for k in r["unique_id"].tolist()]
        np.testing.assert_array_equal(r["id_cnt_fill"], want)                            # idCntFill
    else:
        assert r["unique_id_cnt"] == len(first_seen)
        np.testing.assert_array_equal(r["id_cnt"], [mult[k] for k in r["unique_id"].tolist()])
    np.testing.assert_array_equal(r["id_cnt"], [mult[k] for k in r["unique_id_in_bucket"].tolist()])


def test_padding_known_answer():
    # unique_test.cpp:716-797: ids {4,4,5,6,4,0}, 2 shards, paddingSize 4, paddingVal -1
    ids = [4, 4, 5, 6, 4, 0]
    r = oracle.unique_sharded(ids, 2, padding_size=4, padding_val=-1)
    reference_assertions(ids, r, 2, 4)
    # layout fixed by the definition: even ids in first-occurrence order, then odd ids, each padded to 4
    np.testing.assert_array_equal(r["unique_id"], [4, 6, 0, -1, 5, -1, -1, -1])
    np.testing.assert_array_equal(r["index"], [0, 0, 4, 1, 0, 2])
    np.testing.assert_array_equal(r["unique_id_in_bucket"], [4, 6, 0, 5])


def test_padding_too_small():
    # unique_test.cpp:36-47: paddingSize 1 with two even ids -> H_PADDING_SMALL
    with pytest.raises(RuntimeError):
        oracle.unique_sharded([0, 2, 1], 2, padding_size=1)


@pytest.mark.parametrize("shards,padding,use_mask", [(1, 0, False), (2, 0, False), (7, 0, False), (8, 0, True),
                                                    (4, 300, False), (16, 80, True)])
def test_random_against_bruteforce(shards, padding, use_mask):
    rng = np.random.default_rng(shards * 100 + padding)
    ids = rng.integers(0, 700, 1000).astype(np.int64)
    r = oracle.unique_sharded(ids, shards, padding_size=padding, padding_val=-1, use_mask=use_mask)
    reference_assertions(ids, r, shards, padding)
    # brute force of the compact layout: shard-major, first occurrence inside a shard
    first_seen = np.array(list(dict.fromkeys(ids.tolist())), dtype=np.int64)
    shard = first_seen % shards
    want = np.concatenate([first_seen[shard == s] for s in range(shards)])
    np.testing.assert_array_equal(r["unique_id_in_bucket"], want)


def test_sorted_matches_numpy():
    rng = np.random.default_rng(5)
    for n in (0, 1, 17, 5000):
        ids = rng.integers(-50, 50, n).astype(np.int64) * (1 << 40)
        u, inv = oracle.unique_sorted(ids)
        wu, winv = np.unique(ids, return_inverse=True)
        np.testing.assert_array_equal(u, wu)
        np.testing.assert_array_equal(inv, winv)


@pytest.mark.skipif(not ref_loader.available(), reason="oracle/_ref/libref_torch.so not built")
def test_sorted_matches_reference_build():
    rng = np.random.default_rng(6)
    for n in (1, 100, 20000):
        ids = rng.integers(-(1 << 62), 1 << 62, n).astype(np.int64)
        ids[rng.integers(0, n, n // 2)] = ids[0]
        u, inv = oracle.unique_sorted(ids)
        wu, winv = ref_loader.ref_unique_parallel(ids)
        np.testing.assert_array_equal(u, wu)
        np.testing.assert_array_equal(inv, winv)
