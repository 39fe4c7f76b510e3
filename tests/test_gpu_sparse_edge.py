"""GPU parity, edge shapes of the gradient reduce: position lists of every length class (1, 2..64, 65..1024, > 1024)
in one table and across many small tables whose 1024-key tiles straddle table borders; runs without position lists."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run_case(tables, dim, optim, steps=2, seed=0):
    """tables: list of int64 key arrays (one per table).  Gather + update on the device and in the oracle, exact."""
    rng = np.random.default_rng(seed)
    T = len(tables)
    batch = [int(t.size) for t in tables]
    n = sum(batch)
    offs = np.concatenate([[0], np.cumsum(batch)]).astype(np.int64)
    rows = [max(int(np.unique(t).size), 1) + 3 for t in tables]
    store = []
    for t in range(T):
        w = rng.normal(0, 0.01, (rows[t], dim)).astype(np.float32)
        store.append((w, np.full_like(w, 0.1 if optim == capi.OPT_ADAGRAD else 0.0), np.zeros_like(w)))
    dstore = [tuple(torch.from_numpy(a).to(DEV) for a in trip) for trip in store]
    rows_h = host.Rows(dim, [d[0] for d in dstore], [d[1] for d in dstore], [d[2] for d in dstore])
    uq = host.Unique(max(n, 1), T)
    tg = host.EmbeddingTables(rows, max(n, 1))
    orc_tab = [oracle.Table(r) for r in rows]
    d_off = torch.from_numpy(offs).to(DEV)
    keys = np.concatenate(tables).astype(np.int64) if n else np.zeros(0, np.int64)
    for step in range(1, steps + 1):
        grad = rng.normal(0, 1e-3, (n, dim)).astype(np.float32)
        uq.run(torch.from_numpy(keys).to(DEV), d_off)
        uk, uo, inv, cnt = uq.fetch()
        slots = uk.clone()
        tg.key2offset(slots, uo, capi.CHANNEL_TRAIN)
        out = host.gather_unique(rows_h, uq, slots)
        lr_t = 0.01 * np.sqrt(1 - 0.999 ** step) / (1 - 0.9 ** step) if optim == capi.OPT_ADAM else 0.01
        host.sparse_apply(rows_h, uq, slots, torch.from_numpy(grad).to(DEV), optim, float(lr_t))
        torch.cuda.synchronize()
        got_out = out.cpu().numpy()
        for t in range(T):
            kt = keys[offs[t]:offs[t + 1]]
            split, _, restore, _ = oracle.hash_split(kt, 1)
            so, rc = orc_tab[t].key2offset(split, 0)
            assert rc == 0
            wv, s1v, s2v = store[t]
            np.testing.assert_array_equal(got_out[offs[t]:offs[t + 1]], oracle.gather_rows(wv, dim, so[restore], dim))
            g = oracle.segment_sum(grad[offs[t]:offs[t + 1]], restore, split.size)
            oracle.byaddr_apply(optim, g, so, wv, s1v, s2v, dim, float(lr_t), delta_form=False)
        for t in range(T):
            for a, b in zip(dstore[t], store[t]):
                np.testing.assert_array_equal(a.cpu().numpy(), b)


def mixed_counts(rng, counts, base=0):
    """keys base, base+1, ... with the given multiplicities, shuffled"""
    keys = np.repeat(np.arange(len(counts), dtype=np.int64) + base, counts)
    rng.shuffle(keys)
    return keys


def test_one_table_every_list_length_class():
    rng = np.random.default_rng(1)
    counts = [70000, 5000, 1025, 1024, 1023, 700, 65, 64, 63, 2, 1, 1] + [3] * 500 + [1] * 3000
    run_case([mixed_counts(rng, counts)], 64, capi.OPT_ADAM)


def test_many_small_tables_with_long_keys_across_tile_borders():
    rng = np.random.default_rng(2)
    tables = []
    for t in range(40):
        counts = [int(rng.integers(65, 600)), int(rng.integers(1, 64)), 1, 1, 2] + [1] * int(rng.integers(0, 200))
        tables.append(mixed_counts(rng, counts, base=1000 * t))
    tables[7] = np.zeros(0, np.int64)                      # an empty table in the middle
    run_case(tables, 32, capi.OPT_ADAGRAD)


@pytest.mark.parametrize("n", [1, 64, 65, 66, 130])
def test_single_key_repeated(n):
    run_case([np.full(n, 12345, dtype=np.int64)], 16, capi.OPT_SGD, steps=1)


def test_wide_rows_long_lists():
    rng = np.random.default_rng(3)
    run_case([mixed_counts(rng, [3000, 200, 66, 5, 1, 1])], 256, capi.OPT_ADAM, steps=1)


@pytest.mark.parametrize("dim", [4, 8, 36, 68, 132, 200, 256, 512, 1000, 1024, 1536, 2048])
def test_narrow_and_very_wide_rows(dim):
    rng = np.random.default_rng(dim)
    run_case([mixed_counts(rng, [1500, 300, 70, 64, 9, 2, 1, 1, 1]), mixed_counts(rng, [5, 1, 1], base=50)], dim,
             capi.OPT_ADAM, steps=1)


def test_update_without_position_lists_is_refused():
    dim, n = 16, 100
    w = torch.zeros((8, dim), device=DEV)
    rows_h = host.Rows(dim, [w])
    uq = host.Unique(n, 1, position_lists=False)
    keys = torch.arange(n, device=DEV, dtype=torch.int64) % 5
    uq.run(keys, torch.tensor([0, n], dtype=torch.int64, device=DEV))
    uk, uo, inv, cnt = uq.fetch()
    np.testing.assert_array_equal(uk.cpu().numpy(), np.arange(5))
    np.testing.assert_array_equal(cnt.cpu().numpy(), np.full(5, 20))
    with pytest.raises(capi.RecsdkError) as e:
        host.sparse_apply(rows_h, uq, uk, torch.zeros((n, dim), device=DEV), capi.OPT_SGD, 0.1)
    assert e.value.code == capi.EINVAL


@pytest.mark.parametrize("dim,optim", [(16, capi.OPT_ADAGRAD), (128, capi.OPT_ADAM), (40, capi.OPT_SGD)])
def test_two_level_order_of_the_longest_lists(dim, optim):
    """Keys seen more than 1024 times are summed chunk by chunk (256 positions each, then the chunk sums in order);
    the oracle restates exactly that, so the results stay equal bit for bit on both sides of the threshold and for
    lists that end inside a chunk, on a chunk border, and one past it."""
    rng = np.random.default_rng(dim)
    counts = [1024, 1025, 1280, 1281, 4096, 4097, 5000, 8192, 8193, 20000, 256 * 5 + 1, 3000, 70, 2, 1] + [1] * 500
    run_case([mixed_counts(rng, counts), mixed_counts(rng, [6000, 4100, 10], base=10 ** 6)], dim, optim, steps=2)


def test_two_level_sum_is_within_the_stated_tolerance_of_a_double_sum():
    """What the fixed order costs in accuracy: |G - sum in double| <= 1e-6 * sum |g| (the path's stated tolerance)."""
    rng = np.random.default_rng(77)
    n, dim = 150_000, 32
    seg = np.zeros(n, np.int32)
    seg[rng.random(n) < 0.1] = 1
    grad = rng.normal(0, 1e-3, (n, dim)).astype(np.float32)
    got = oracle.segment_sum(grad, seg, 2)
    for s in (0, 1):
        exact = grad[seg == s].astype(np.float64).sum(axis=0)
        bound = 1e-6 * np.abs(grad[seg == s]).astype(np.float64).sum(axis=0)
        assert (np.abs(got[s] - exact) <= bound).all()
    # and the device forms the same sum as the oracle
    w = torch.zeros((4, dim), device=DEV)
    rows_h = host.Rows(dim, [w])
    uq = host.Unique(n, 1)
    keys = torch.from_numpy(seg.astype(np.int64) * 5 + 3).to(DEV)
    uq.run(keys, torch.tensor([0, n], dtype=torch.int64, device=DEV))
    uk, uo, inv, cnt = uq.fetch()
    slots = torch.arange(uk.numel(), device=DEV, dtype=torch.int64)
    host.sparse_apply(rows_h, uq, slots, torch.from_numpy(grad).to(DEV), capi.OPT_SGD, 1.0)   # w = -G
    first = int(seg[0])                                         # rank 0 is the key seen first
    np.testing.assert_array_equal(w[0].cpu().numpy(), -got[first])
    np.testing.assert_array_equal(w[1].cpu().numpy(), -got[1 - first])


def test_more_tables_than_the_staged_lookups_hold():
    """1100 tables: past the table counts up to which the gather (64) and the list bounds (1023) keep the tables'
    offsets in LDS."""
    rng = np.random.default_rng(9)
    tables = [mixed_counts(rng, [int(rng.integers(1, 70)), 2, 1, 1], base=10 * t) for t in range(1100)]
    tables[500] = np.zeros(0, np.int64)
    run_case(tables, 16, capi.OPT_ADAGRAD, steps=2)


@pytest.mark.parametrize("sizes", [(200_000,), (300_000,), (600_000,), (150_000, 190_000), (1_100_000,)],
                         ids=["18 bits", "19 bits", "20 bits", "two tables 18 bits", "21 bits"])
def test_position_sort_at_every_digit_width(sizes):
    """Above 180000 positions the lists come from a radix sort whose digit width follows the number of rank bits
    (8, 9 or 10 bits, whichever needs the fewest passes): one case per width and pass count, each a full step whose
    sums depend on the order inside every list."""
    rng = np.random.default_rng(sum(sizes))
    tables = []
    for n in sizes:
        # a heavy head (lists of thousands of positions), a middle of short lists and a tail of single keys
        k = np.where(rng.random(n) < 0.5, rng.zipf(1.2, n) % 5000, rng.integers(0, n, n) + 10_000)
        tables.append(k.astype(np.int64))
    run_case(tables, 8, capi.OPT_ADAGRAD, steps=1)
