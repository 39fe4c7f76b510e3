"""GPU parity over random shapes: table counts on both sides of every path switch (1, 64 | 65 tables, batches around 4096
keys), table sizes around the tile and wave borders, key distributions from all-distinct to a few keys with thousands of
occurrences, the skip key and the empty-marker key among them, with and without position lists, early multiplicities
and a promised bound of the keys per table; then the full step (slots, gather, fused update) against the oracle."""
import numpy as np
import pytest

import oracle
from recsdk_amd import capi, host
from tests.test_gpu_sparse_edge import mixed_counts, run_case
from tests.test_gpu_unique import check_against_oracle, run_unique

pytestmark = pytest.mark.gpu
SIZES = [0, 1, 2, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 3000, 5000, 20000]


def random_tables(rng):
    T = int(rng.choice([1, 1, 2, 3, 7, 26, 40, 64, 65, 100]))
    kind = int(rng.integers(0, 5))
    tables = []
    for _ in range(T):
        n = int(rng.choice(SIZES))
        if T >= 26:
            n = min(n, 3000)
        if kind == 0:          # a third as many keys as positions
            k = rng.integers(0, max(n // 3, 1) + 1, n)
        elif kind == 1:        # practically all distinct, the whole 64-bit range
            k = rng.integers(-2 ** 62, 2 ** 62, n)
        elif kind == 2:        # heavy head
            k = rng.zipf(1.3, n) % 1000
        elif kind == 3:        # a few keys with up to thousands of occurrences
            counts = list(rng.integers(1, 3000, int(rng.integers(1, 6)))) + [1] * int(rng.integers(0, 300))
            k = mixed_counts(rng, counts, base=int(rng.integers(0, 10 ** 9)))
        else:                  # the empty-marker key and the smallest key among few others
            k = np.where(rng.random(n) < 0.1, -1, rng.integers(0, 50, n))
            if n > 3:
                k[int(rng.integers(0, n))] = -2 ** 63
        tables.append(np.asarray(k, dtype=np.int64))
    return tables


@pytest.mark.parametrize("seed", range(48))
def test_random_shape(seed):
    rng = np.random.default_rng(7000 + seed)
    tables = random_tables(rng)
    n = sum(len(t) for t in tables)
    early_counts = bool(rng.integers(0, 2))
    lists = bool(rng.integers(0, 2))
    bound = int(max((len(t) for t in tables), default=1)) if rng.integers(0, 2) else 0
    uq = host.Unique(max(n, 1) + int(rng.integers(0, 100)), len(tables), position_lists=lists,
                     early_counts=early_counts, max_table_keys=bound)
    in_counts = rng.integers(0, 5, n) if early_counts and rng.integers(0, 3) == 0 else None
    uk, uo, inv, cnt, offs = got = run_unique(uq, tables, in_counts=in_counts)
    if in_counts is None:
        check_against_oracle(tables, got)
        # the handle once more, with the same keys in another order
        again = [rng.permutation(t) for t in tables]
        check_against_oracle(again, run_unique(uq, again))
    else:
        for t, keys in enumerate(tables):
            split, _, restore, _ = oracle.hash_split(keys, rank_size=1)
            np.testing.assert_array_equal(uk[uo[t]:uo[t + 1]], split)
            np.testing.assert_array_equal(inv[offs[t]:offs[t + 1]], restore)
            want = np.zeros(split.size, np.int64)
            np.add.at(want, restore, in_counts[offs[t]:offs[t + 1]])
            np.testing.assert_array_equal(cnt[uo[t]:uo[t + 1]].astype(np.int64), want)
    if n > 0:
        dim = int(rng.choice([4, 8, 16, 32, 64, 128, 260, 1028]))
        if n * dim > 40_000_000:
            dim = 16
        optim = int(rng.choice([capi.OPT_SGD, capi.OPT_ADAGRAD, capi.OPT_ADAM]))
        run_case(tables, dim, optim, steps=2)
