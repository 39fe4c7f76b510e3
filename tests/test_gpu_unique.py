"""GPU parity: multi-table first-occurrence dedup through the C ABI vs the CPU oracle (bit-exact)."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host
from tests.util import zipf_keys

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run_unique(uq, tables, in_counts=None, skip_key=None):
    keys = np.concatenate(tables + [np.zeros(0, np.int64)]).astype(np.int64)
    offs = np.concatenate([[0], np.cumsum([len(t) for t in tables])]).astype(np.int64)
    dk = torch.from_numpy(keys).to(DEV)
    do = torch.from_numpy(offs).to(DEV)
    dc = torch.from_numpy(in_counts.astype(np.int32)).to(DEV) if in_counts is not None else None
    uk, uo, inv, cnt = uq.run(dk, do, in_counts=dc, skip_key=skip_key).fetch()
    return uk.cpu().numpy(), uo.cpu().numpy(), inv.cpu().numpy(), cnt.cpu().numpy().astype(np.uint32), offs


def check_against_oracle(tables, got):
    uk, uo, inv, cnt, offs = got
    for t, keys in enumerate(tables):
        split, _, restore, counts = oracle.hash_split(keys, rank_size=1)
        assert uo[t + 1] - uo[t] == split.size
        np.testing.assert_array_equal(uk[uo[t]:uo[t + 1]], split)
        np.testing.assert_array_equal(inv[offs[t]:offs[t + 1]], restore)
        np.testing.assert_array_equal(cnt[uo[t]:uo[t + 1]], counts)


def test_hash_split_kat_on_gpu():
    kp = host.KeyProcess(1024)
    keys = torch.tensor([1, 4, 23, 14, 16, 7, 2, 21, 21, 29], dtype=torch.int64, device=DEV)
    uk, restore, cnt, _ = kp.hash_split(keys)
    # rankSize 1: one bucket, first-occurrence order (key_process_test.cpp:744-787 with a single rank)
    assert uk.tolist() == [1, 4, 23, 14, 16, 7, 2, 21, 29]
    assert restore.tolist() == [0, 1, 2, 3, 4, 5, 6, 7, 7, 8]
    assert cnt.tolist() == [1, 1, 1, 1, 1, 1, 1, 2, 1]


@pytest.mark.parametrize("seed", [0, 1])
def test_multi_table_ragged_and_empty(seed):
    rng = np.random.default_rng(seed)
    sizes = [0, 1, 5000, 0, 1023, 1024, 1025, 70000, 3, 0]
    tables = []
    for t, n in enumerate(sizes):
        hi = [3, 50, 10**6, 2**62][t % 4]
        tables.append(rng.integers(-hi, hi, n))
    uq = host.Unique(sum(sizes) + 10, len(sizes))
    check_against_oracle(tables, run_unique(uq, tables))
    # the handle is reusable: second run with other data
    tables2 = [rng.integers(0, 100, n) for n in sizes[::-1]]
    check_against_oracle(tables2, run_unique(uq, tables2))


def test_empty_batch():
    uq = host.Unique(16, 2)
    uk, uo, inv, cnt, _ = run_unique(uq, [np.zeros(0, np.int64), np.zeros(0, np.int64)])
    assert uk.size == 0 and uo.tolist() == [0, 0, 0] and inv.size == 0


def test_all_equal_all_distinct_and_sentinel_keys():
    n = 65536
    int_min = -2**63
    tables = [np.full(n, 42), np.arange(n)[::-1].copy(), np.full(777, -1),
              np.array([-1, int_min, -1, 5, int_min, 2**63 - 1, 0, -1] * 50)]
    uq = host.Unique(3 * n, len(tables))
    check_against_oracle(tables, run_unique(uq, tables))


def test_zipf_26_tables_batch_4096():
    rng = np.random.default_rng(3)
    tables = [zipf_keys(rng, 1.05, 1000 * (t + 1), 4096, table=t) for t in range(26)]
    uq = host.Unique(26 * 4096, 26)
    got = run_unique(uq, tables)
    check_against_oracle(tables, got)
    # size-independent invariant: unique[inverse] reproduces the input
    uk, uo, inv, cnt, offs = got
    for t, keys in enumerate(tables):
        np.testing.assert_array_equal(uk[uo[t]:uo[t + 1]][inv[offs[t]:offs[t + 1]]], keys)
        assert cnt[uo[t]:uo[t + 1]].sum() == len(keys)


def test_input_counts_are_summed():
    rng = np.random.default_rng(4)
    keys = rng.integers(0, 300, 5000)
    w = rng.integers(0, 7, 5000)
    uq = host.Unique(5000, 1)
    uk, uo, inv, cnt, _ = run_unique(uq, [keys], in_counts=w)
    split, _, restore, _ = oracle.hash_split(keys, 1)
    np.testing.assert_array_equal(uk, split)
    np.testing.assert_array_equal(inv, restore)
    np.testing.assert_array_equal(cnt, np.bincount(restore, weights=w, minlength=split.size).astype(np.uint32))


@pytest.mark.parametrize("dyn", [False, True])
def test_global_unique_static_padding(dyn):
    rng = np.random.default_rng(5)
    keys = rng.integers(-1, 40, 3000)
    kp = host.KeyProcess(4096)
    uk, rvs = kp.global_unique(torch.from_numpy(keys).to(DEV), use_static=True, use_dynamic_expansion=dyn)
    wu, wr, _ = oracle.global_unique(keys, True, dyn)
    np.testing.assert_array_equal(uk.cpu().numpy(), wu)
    np.testing.assert_array_equal(rvs.cpu().numpy(), wr)
    uk, rvs = kp.global_unique(torch.from_numpy(keys).to(DEV))
    wu, wr, _ = oracle.global_unique(keys, False, False)
    np.testing.assert_array_equal(uk.cpu().numpy(), wu)
    np.testing.assert_array_equal(rvs.cpu().numpy(), wr)


def test_capacity_errors():
    from recsdk_amd.capi import RecsdkError, ECAPACITY
    uq = host.Unique(100, 1)
    with pytest.raises(RecsdkError) as e:
        run_unique(uq, [np.arange(101)])
    assert e.value.code == ECAPACITY
    with pytest.raises(RecsdkError):
        run_unique(uq, [np.arange(5), np.arange(5)])


@pytest.mark.parametrize("seed", [0, 1])
def test_counts_delivered_with_the_lists(seed):
    """early_counts=False: the hashing pass collects no multiplicities; they come from the sorted position lists
    (list lengths) and fetch() orders itself after the list kernels.  Same results, skipped keys included."""
    rng = np.random.default_rng(100 + seed)
    sizes = [0, 1, 5000, 0, 1023, 1024, 1025, 70000, 3, 0]
    tables = [rng.integers(-[3, 50, 10**6, 2**62][t % 4], [3, 50, 10**6, 2**62][t % 4], n) for t, n in enumerate(sizes)]
    uq = host.Unique(sum(sizes) + 10, len(sizes), early_counts=False)
    check_against_oracle(tables, run_unique(uq, tables))
    tables2 = [zipf_keys(rng, 1.05, 2000, n, table=t) for t, n in enumerate(sizes[::-1])]
    check_against_oracle(tables2, run_unique(uq, tables2))
    # a skipped key: inverse -1, not counted, and its positions sit behind every list
    keys = [np.array([5, -1, 5, 9, -1, 7, 9, 5, -1])]
    uk, uo, inv, cnt, _ = run_unique(uq, keys, skip_key=-1)
    assert uk.tolist() == [5, 9, 7] and cnt.tolist() == [3, 2, 1]
    assert inv.tolist() == [0, -1, 0, 1, -1, 2, 1, 0, -1]


def test_promised_bound_of_keys_per_table():
    """set_max_table_keys sizes the sort behind the position lists.  Kept: same results with fewer radix passes.
    Broken: unique keys, inverse and counts are still right, the lists are empty and total() says so."""
    rng = np.random.default_rng(7)
    tables = [rng.integers(0, 3000, 4096) for _ in range(5)] + [np.array([-1, 4, -1, 4, 9])]
    uq = host.Unique(6 * 4096, 6, max_table_keys=4096)
    check_against_oracle(tables, run_unique(uq, tables))
    late = host.Unique(6 * 4096, 6, early_counts=False, max_table_keys=4096)
    check_against_oracle(tables, run_unique(late, tables))
    small = host.Unique(6 * 4096, 6, max_table_keys=1000)
    keys = np.concatenate(tables).astype(np.int64)
    offs = np.concatenate([[0], np.cumsum([len(t) for t in tables])]).astype(np.int64)
    small.run(torch.from_numpy(keys).to(DEV), torch.from_numpy(offs).to(DEV))
    with pytest.raises(capi.RecsdkError) as e:
        small.total()
    assert e.value.code == capi.ECAPACITY
