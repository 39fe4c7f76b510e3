"""GPU: the host-backed cache at the configuration's batch (65536 x 26 keys, Zipf(1.05)) over a 100 M-row pinned
host table, with an HBM cache small enough that rows are swapped out and back in all the time.

Property checked (no CPU run of the same size needed): rows start at zero (constant initializer), the gradient is
all ones and the optimizer is SGD with lr = 2^-10, so after any history of updates, swap-outs and swap-ins the row
of a key holds exactly -(number of times the key was looked up so far) / 1024 in every column.  The forward gather
of every step must therefore return -(earlier lookups of that key) / 1024, whichever tier the row came from.
Run with the swaps one after the other on one stream, and on the two- and three-stage schedules of the benchmark
(rows of batch i beside the move of batch i + 1 beside the dedup and plan of batch i + 2) with the call that moves
both directions at the same time, and on the benchmark's default schedule, in which the rows stage of batch i starts
when the link kernel of batch i + 1 starts (the event handed to the row store).
"""
import numpy as np
import pytest
import torch

from recsdk_amd import capi, host
from recsdk_amd.synth import splitmix64, zipf_ranks

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("stages", [1, 2, 3, 4])
def test_rows_keep_their_update_count_across_swaps(stages):
    T, batch, dim = 26, 65536, 64
    host_rows, cache_rows, steps = 100_000_000, 1_500_000, 10
    n = T * batch
    rng = np.random.default_rng(5)
    ranks = [zipf_ranks(rng, 1.05, host_rows, n) for _ in range(steps)]
    keys = [torch.from_numpy(splitmix64(r.astype(np.uint64)).astype(np.int64)).to(DEV) for r in ranks]
    off = torch.tensor([0, n], dtype=torch.int64, device=DEV)
    cache = torch.full((cache_rows, dim), 7.0, device=DEV)        # stale contents must never show
    rows_h = host.Rows(dim, [cache])
    grad = torch.ones((n, dim), device=DEV)
    outs = [torch.empty((n, dim), device=DEV) for _ in range(3)]
    store = host.EmbLocalTable(host_rows, dim, [(capi.INIT_CONSTANT, 0, dim, 0.0, 0.0, 0, 1.0)])
    uqs = [host.Unique(n, 1) for _ in range(3)]                    # batch i uses set i % 3
    om = host.OffsetMapper(cache_rows, max_keys=n)
    slots = [None] * 3
    lists = [None] * 3
    swapped = [0, 0]
    lr = 2.0 ** -10

    def index(i):
        b = i % 3
        slots[b], _, _, _ = uqs[b].run(keys[i], off).fetch()
        lists[b] = om.get_swap_pairs_and_key2offset(slots[b])
        swapped[0] += int(lists[b][0].numel())
        swapped[1] += int(lists[b][2].numel())

    def move(i):
        in_keys, in_pos, out_keys, out_pos = lists[i % 3]
        if stages > 1:
            store.swap(out_keys, out_pos, in_keys, in_pos, cache)        # both directions in one call
        else:
            if out_keys.numel():
                store.swap_out(out_keys, out_pos, cache)
            if in_keys.numel():
                store.swap_in(in_keys, in_pos, cache)

    def rows(i):
        b = i % 3
        host.gather_unique(rows_h, uqs[b], slots[b], outs[b])
        host.sparse_apply(rows_h, uqs[b], slots[b], grad, capi.OPT_SGD, lr)

    seen = np.zeros(host_rows, dtype=np.int32)

    def check(i):
        got = outs[i % 3]
        want = torch.from_numpy(seen[ranks[i]].astype(np.float32) * np.float32(-lr)).to(DEV)
        for col in (0, 37, 63):
            assert torch.equal(got[:, col], want), f"step {i}, column {col}"
        np.add.at(seen, ranks[i], 1)

    if stages == 1:
        for i in range(steps):
            index(i)
            move(i)
            rows(i)
            torch.cuda.synchronize()
            check(i)
    else:
        # stages == 2: dedup, plan and move of batch i + 1 on one stream beside the rows of batch i;
        # stages == 3: the move of batch i + 1 and the dedup and plan of batch i + 2 on a stream each
        s_index = torch.cuda.Stream()
        # stages == 4: as 3, and the rows of batch i wait for the link kernel of batch i + 1 to start
        s_move = s_index if stages == 2 else torch.cuda.Stream()
        s_rows = torch.cuda.Stream()
        ev_index = [torch.cuda.Event() for _ in range(3)]
        ev_move = [torch.cuda.Event() for _ in range(3)]
        ev_rows = [torch.cuda.Event() for _ in range(3)]
        ev_link = None
        if stages == 4:
            ev_link = torch.cuda.Event()
            ev_link.record(s_move)
            store.on_link_start(ev_link)
        torch.cuda.synchronize()

        def do_index(i):
            with torch.cuda.stream(s_index):
                if i >= 3:
                    s_index.wait_event(ev_rows[i % 3])
                index(i)
                ev_index[i % 3].record(s_index)

        def do_move(i):
            with torch.cuda.stream(s_move):
                s_move.wait_event(ev_index[i % 3])
                if i >= 2:
                    s_move.wait_event(ev_rows[(i - 2) % 3])
                move(i)
                ev_move[i % 3].record(s_move)

        def do_rows(i):
            with torch.cuda.stream(s_rows):
                s_rows.wait_event(ev_move[i % 3])
                if ev_link is not None:
                    s_rows.wait_event(ev_link)
                rows(i)
                ev_rows[i % 3].record(s_rows)

        do_index(0)
        do_move(0)
        if stages >= 3 and steps > 1:
            do_index(1)
        for i in range(steps):
            if stages == 2:
                do_rows(i)
                if i + 1 < steps:
                    do_index(i + 1)
                    do_move(i + 1)
            else:
                if stages == 3:
                    do_rows(i)
                if i + 1 < steps:
                    do_move(i + 1)
                if stages == 4:
                    do_rows(i)
                if i + 2 < steps:
                    do_index(i + 2)
            ev_rows[i % 3].synchronize()
            check(i)
        torch.cuda.synchronize()
        store.on_link_start(None)
    assert swapped[1] > 1_000_000        # rows did leave the cache and come back
    # every row still in the cache holds -(lookups) / 1024; slots never written keep the fill value
    col = cache[:, 11]
    assert bool(((col <= 0) | (col == 7.0)).all())


def test_adagrad_rows_follow_the_closed_form_behind_the_20m_row_cache():
    """The configuration's own cache size (20 M rows of [w | accumulator]) and optimizer (Adagrad, lr 0.01, accumulator
    0.1), warmed until the cache is full and rows are swapped out every step.  With a constant gradient g0 = 2^-10 per
    lookup the summed gradient of a key seen c times in a step is exactly c * g0, so the row of every key follows
        acc <- acc + (c g0)^2 ;  w <- w + (-lr * c g0) / sqrt(acc + eps)
    (adagrad_by_addr.py:101-125), which the host replays in float32 for the keys of each step alone: no CPU run of the
    whole pipeline is needed.  The forward gather of every step must return the replayed weights bit for bit, whether
    the row sat in the cache, came back from the host table or is new; after the last step the host table's rows of
    swapped-out keys hold the replayed values as well."""
    from recsdk_amd.synth import ZipfSampler
    T, batch, dim = 26, 65536, 64
    ext = 2 * dim
    host_rows, cache_rows, steps = 100_000_000, 20_000_000, 126   # the cache is full after some 108 batches
    n = T * batch
    lr, eps, g0 = np.float32(0.01), np.float32(1e-7), np.float32(2.0 ** -10)
    rng = np.random.default_rng(9)
    sampler = ZipfSampler(1.05, host_rows)
    off = torch.tensor([0, n], dtype=torch.int64, device=DEV)
    cache = torch.full((cache_rows, ext), 7.0, device=DEV)        # stale contents must never show
    flat = cache.view(-1)
    rows_h = host.Rows(dim, [cache], [flat[dim:]], None, [ext])
    grad = torch.full((n, dim), float(g0), device=DEV)
    out = torch.empty((n, dim), device=DEV)
    store = host.EmbLocalTable(host_rows, ext, [(capi.INIT_CONSTANT, 0, dim, 0.01, 0.0, 0, 1.0),
                                                (capi.INIT_CONSTANT, dim, dim, 0.1, 0.0, 0, 1.0)])
    uq = host.Unique(n, 1)
    om = host.OffsetMapper(cache_rows, max_keys=n)
    w_h = np.full(host_rows, 0.01, dtype=np.float32)              # one column stands for all: they start equal
    a_h = np.full(host_rows, 0.1, dtype=np.float32)
    swapped_out = 0
    last_out = None
    for i in range(steps):
        ranks = sampler.ranks(rng, n)
        keys_h = splitmix64(ranks.astype(np.uint64)).astype(np.int64)
        keys = torch.from_numpy(keys_h).to(DEV)
        slots, _, _, _ = uq.run(keys, off).fetch()
        in_keys, in_pos, out_keys, out_pos = om.get_swap_pairs_and_key2offset(slots)
        if out_keys.numel():
            store.swap_out(out_keys, out_pos, cache)
        if in_keys.numel():
            store.swap_in(in_keys, in_pos, cache)
        host.gather_unique(rows_h, uq, slots, out)
        host.sparse_apply(rows_h, uq, slots, grad, capi.OPT_ADAGRAD, float(lr), eps=float(eps))
        torch.cuda.synchronize()
        want = torch.from_numpy(w_h[ranks]).to(DEV)
        for col in (0, 21, 63):
            assert torch.equal(out[:, col], want), f"step {i}, column {col}"
        # replay of this step's updates on the host, float32 operation by operation (opt_update's order)
        u, c = np.unique(ranks, return_counts=True)
        g = c.astype(np.float32) * g0
        st = a_h[u] + g * g
        den = np.sqrt(st + eps)
        w_h[u] = w_h[u] + (-lr * g) / den
        a_h[u] = st
        if out_keys.numel():
            swapped_out += int(out_keys.numel())
            last_out = out_keys.cpu().numpy()
    assert swapped_out > 1_000_000, "the cache never filled: no row was swapped out"
    # the rows that left the cache in the last step sit in the host table with the replayed values (every column)
    probe = last_out[:: max(1, last_out.size // 4000)]
    got = store.gather(probe).reshape(probe.size, ext)
    r = _unsplitmix64(probe)
    assert np.array_equal(splitmix64(r).astype(np.int64), probe)
    assert np.array_equal(got[:, :dim], np.repeat(w_h[r][:, None], dim, axis=1))
    assert np.array_equal(got[:, dim:], np.repeat(a_h[r][:, None], dim, axis=1))
    assert np.any(a_h[r] > np.float32(0.1))


def _unsplitmix64(keys):
    """ranks whose splitmix64 finaliser gives `keys` (every step of the finaliser is a bijection on 64 bits)"""
    z = np.asarray(keys).view(np.uint64).copy()
    with np.errstate(over="ignore"):
        z = z ^ (z >> np.uint64(31)) ^ (z >> np.uint64(62))
        z = z * np.uint64(pow(0x94D049BB133111EB, -1, 1 << 64))
        z = z ^ (z >> np.uint64(27)) ^ (z >> np.uint64(54))
        z = z * np.uint64(pow(0xBF58476D1CE4E5B9, -1, 1 << 64))
        z = z ^ (z >> np.uint64(30)) ^ (z >> np.uint64(60))
        z = z - np.uint64(0x9E3779B97F4A7C15)
    return z
