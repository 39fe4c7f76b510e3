"""GPU parity of the one-launch paths for small batches (at most 4096 keys per call): dedup, key -> slot, gather and
the scan-based gradient reduce give what the general path gives, bit for bit, and what the CPU oracle gives."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host
from tests.util import zipf_keys

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture
def general_path():
    """Switch the small-batch paths off for the duration of a block of code."""
    class Ctx:
        def __enter__(self):
            capi.check(capi.lib().recsdk_set_small_batch_keys(0))

        def __exit__(self, *a):
            capi.check(capi.lib().recsdk_set_small_batch_keys(4096))
    return Ctx()


def run_steps(tables_keys, rows, dim, optim, steps, layout_ext=False):
    """A few whole steps on fresh state; returns everything a caller can observe."""
    T = len(rows)
    rng = np.random.default_rng(5)
    w0 = [rng.normal(0, 0.01, (r, dim)).astype(np.float32) for r in rows]
    w = [torch.from_numpy(x.copy()).to(DEV) for x in w0]
    s1 = [torch.full((r, dim), 0.1, device=DEV) for r in rows]
    s2 = [torch.zeros((r, dim), device=DEV) for r in rows]
    rows_h = host.Rows(dim, w, s1, s2)
    n = sum(len(k) for k in tables_keys[0])
    uq = host.Unique(max(n, 1), T)
    tg = host.EmbeddingTables(rows, max(n, 1))
    seen = []
    for step in range(steps):
        tk = tables_keys[step]
        keys = np.concatenate(tk + [np.zeros(0, np.int64)]).astype(np.int64)
        offs = np.concatenate([[0], np.cumsum([len(t) for t in tk])]).astype(np.int64)
        grad = np.random.default_rng(100 + step).normal(0, 1e-2, (keys.size, dim)).astype(np.float32)
        uq.run(torch.from_numpy(keys).to(DEV), torch.from_numpy(offs).to(DEV), skip_key=-1)
        uk, uo, inv, cnt = uq.fetch()
        slots = uk.clone()
        tg.key2offset(slots, uo, capi.CHANNEL_TRAIN)
        out = host.gather_unique(rows_h, uq, slots)
        host.sparse_apply(rows_h, uq, slots, torch.from_numpy(grad).to(DEV), optim, 0.01, 0.9, 0.999, 1e-8,
                          0.001 if optim == capi.OPT_SGD else 0.0)
        seen.append([x.cpu().numpy() for x in (uk, uo, inv, cnt, slots, out)])
    state = [x.cpu().numpy() for x in w + s1 + s2]
    return seen, state, tg.stats()


def key_stream(kind, T, n_per_table, steps, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(steps):
        if kind == "uniform":
            out.append([rng.integers(0, 10 ** 6, n_per_table) for _ in range(T)])
        elif kind == "zipf":
            out.append([zipf_keys(rng, 1.2, 500, n_per_table, table=t) for t in range(T)])
        elif kind == "one_hot_key":      # one key almost everywhere: a queue that drains many times
            out.append([np.where(rng.random(n_per_table) < 0.9, 7, rng.integers(0, 50, n_per_table)) for _ in range(T)])
        elif kind == "chunk_borders":    # lists at the two-level threshold, one past it and on a chunk border
            out.append([rng.permutation(np.concatenate([np.full(c, 7), rng.integers(100, 200, 60)]))
                        for c in (1024, 1025, 1280)[:T]])
        else:                            # skipped keys, the empty-marker key and ragged tables
            out.append([np.array([5, -1, 5, -2 ** 63, -1, 2 ** 63 - 1, 0, -1], dtype=np.int64)[: (t * 3) % 9] for t in range(T)])
    return out


@pytest.mark.parametrize("kind,T,n_per,dim,optim", [
    ("uniform", 1, 4096, 16, capi.OPT_ADAGRAD),     # configuration 1's shape
    ("zipf", 3, 1365, 128, capi.OPT_ADAM),
    ("one_hot_key", 2, 2048, 32, capi.OPT_SGD),
    ("zipf", 64, 64, 8, capi.OPT_ADAM),
    ("ragged", 5, 0, 64, capi.OPT_ADAGRAD),
    ("zipf", 1, 300, 512, capi.OPT_ADAM),
    ("chunk_borders", 3, 0, 32, capi.OPT_ADAM),
])
def test_small_paths_equal_the_general_path(general_path, kind, T, n_per, dim, optim):
    steps = 3
    stream = key_stream(kind, T, n_per, steps, seed=T * 1000 + n_per)
    rows = [20000] * T if kind == "uniform" else [800] * T
    small = run_steps(stream, rows, dim, optim, steps)
    with general_path:
        big = run_steps(stream, rows, dim, optim, steps)
    for a, b in zip(small[0], big[0]):
        for x, y in zip(a, b):
            np.testing.assert_array_equal(x, y)
    for x, y in zip(small[1], big[1]):
        np.testing.assert_array_equal(x, y)
    assert small[2] == big[2]


def test_small_dedup_against_the_oracle():
    rng = np.random.default_rng(3)
    tables = [rng.integers(-40, 40, 1000), np.zeros(0, np.int64), zipf_keys(rng, 1.05, 3000, 3000, table=2),
              np.array([-1, -2 ** 63, -1, 5, -2 ** 63])]
    keys = np.concatenate(tables).astype(np.int64)
    offs = np.concatenate([[0], np.cumsum([len(t) for t in tables])]).astype(np.int64)
    uq = host.Unique(keys.size, len(tables))
    uk, uo, inv, cnt = (x.cpu().numpy() for x in uq.run(torch.from_numpy(keys).to(DEV),
                                                        torch.from_numpy(offs).to(DEV)).fetch())
    for t, kt in enumerate(tables):
        split, _, restore, counts = oracle.hash_split(kt, rank_size=1)
        np.testing.assert_array_equal(uk[uo[t]:uo[t + 1]], split)
        np.testing.assert_array_equal(inv[offs[t]:offs[t + 1]], restore)
        np.testing.assert_array_equal(cnt[uo[t]:uo[t + 1]].astype(np.uint32), counts)


def test_limit_is_validated():
    L = capi.lib()
    assert L.recsdk_set_small_batch_keys(4097) == capi.EINVAL
    assert L.recsdk_set_small_batch_keys(-1) == capi.EINVAL
    assert L.recsdk_set_small_batch_keys(4096) == capi.OK


@pytest.mark.parametrize("dynamic", [False, True])
def test_one_table_spread_over_blocks_equals_the_oracle_and_the_general_path(general_path, dynamic):
    """A small batch of ONE table is resolved by several blocks that agree on the new keys' ranks through words in the
    handle: batches around the block size, a caller's n above the number of keys the offsets name, the two marker
    keys, evicted slots handed out again, an evaluation batch, a table that overflows; the same calls on a twin table
    through the three-kernel path and on the oracle's table.  The words must be back at zero after every call, so the
    sequence is long enough for a stale word to show."""
    rng = np.random.default_rng(17)
    vocab = 7900
    row_bytes, base = 64, 1 << 20
    kw = dict(dynamic=[1], arena_bases=[base], row_bytes=[row_bytes]) if dynamic else {}
    spread = host.EmbeddingTables([vocab], 4096, **kw)
    with general_path:
        plain = host.EmbeddingTables([vocab], 4096, **kw)
    orc = oracle.Table(vocab, dynamic=dynamic, arena_base=base, row_bytes=row_bytes)
    pool = rng.permutation(40000).astype(np.int64)

    def call(keys, channel, n_arg=None):
        keys = np.asarray(keys, dtype=np.int64)
        off = torch.tensor([0, keys.size], dtype=torch.int64, device=DEV)
        pad = np.concatenate([keys, np.full((n_arg or keys.size) - keys.size, 12345, np.int64)])   # beyond the offsets
        a = spread.key2offset(torch.from_numpy(pad.copy()).to(DEV), off, channel, n=n_arg).cpu().numpy()
        with general_path:
            b = plain.key2offset(torch.from_numpy(pad.copy()).to(DEV), off, channel, n=n_arg).cpu().numpy()
        want, _ = orc.key2offset(keys, channel)
        np.testing.assert_array_equal(a[:keys.size], want)
        np.testing.assert_array_equal(a, b)
        np.testing.assert_array_equal(a[keys.size:], 12345)          # keys the offsets do not name stay untouched

    sizes = [257, 256 * 3, 1000, 4096, 300, 2049, 511]
    start = 0
    known = np.zeros(0, np.int64)          # keys the table holds
    for k, m in enumerate(sizes):
        n_old = min(known.size, m // 2)
        old = rng.choice(known, n_old, replace=False)
        fresh = pool[start:start + m - n_old]
        start += fresh.size
        keys = rng.permutation(np.concatenate([fresh, old]))
        known = np.concatenate([known, fresh])
        if k == 2:
            keys = np.insert(keys, [5, 700], [-1, -2 ** 63])           # the empty marker and the erased marker
        call(keys, capi.CHANNEL_TRAIN, n_arg=4096 if k % 2 else None)
        if k == 3 and not dynamic:
            ev = np.sort(rng.choice(known, 700, replace=False))
            known = np.setdiff1d(known, ev)
            off = torch.tensor([0, ev.size], dtype=torch.int64, device=DEV)
            spread.evict_keys(torch.from_numpy(ev).to(DEV), off)
            with general_path:
                plain.evict_keys(torch.from_numpy(ev).to(DEV), off)
            orc.evict(ev)
        if k == 4:
            call(rng.permutation(np.concatenate([known[:200], pool[30000:30300]])), capi.CHANNEL_EVAL)
    assert spread.stats() == plain.stats()
    # more new keys than the table has room for: the surplus is refused the same way
    keys = pool[start:start + 4096]
    off = torch.tensor([0, keys.size], dtype=torch.int64, device=DEV)
    a = spread.key2offset(torch.from_numpy(keys.copy()).to(DEV), off).cpu().numpy()
    with general_path:
        b = plain.key2offset(torch.from_numpy(keys.copy()).to(DEV), off).cpu().numpy()
    np.testing.assert_array_equal(a, b)
    for tg in (spread, plain):
        with pytest.raises(capi.RecsdkError):
            tg.stats()
