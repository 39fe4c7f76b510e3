"""GPU parity: host-DRAM row store (AccCTR EmbLocalTable), its swap kernels, and the host-backed HBM cache step
(config 5 at small scale): unique -> cache planner -> swap-out / swap-in of rows -> gather -> Adagrad update, all
compared exactly with the CPU oracle's pipeline."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host
from recsdk_amd.synth import zipf_ranks

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
C, N, TN = capi.INIT_CONSTANT, capi.INIT_RANDOM_NORMAL, capi.INIT_TRUNCATED_NORMAL


def test_gather_scatter_remove_match_oracle():
    ext = 24
    descs = [(N, 0, 8, 0.0, 0.05, 1, 1.0), (C, 8, 8, 0.1, 0.0, 0, 1.0), (TN, 16, 8, 0.0, 0.05, 2, 1.0)]
    tab, orc = host.EmbLocalTable(400, ext, descs), oracle.HostRows(400, ext, descs)
    rng = np.random.default_rng(0)
    for step in range(12):
        keys = rng.choice(300, size=30, replace=False)
        np.testing.assert_array_equal(tab.gather(keys, threads=1 + step % 3), orc.gather(keys))
        upd = rng.normal(0, 1, (10, ext)).astype(np.float32)
        k2 = rng.choice(300, size=10, replace=False)
        tab.scatter(k2, upd)
        orc.scatter(k2, upd)
        if step % 3 == 2:
            k3 = rng.choice(300, size=40, replace=False)
            np.testing.assert_array_equal(tab.gather_and_remove(k3), orc.gather_and_remove(k3))
            k4 = rng.choice(300, size=15, replace=False)
            tab.remove(k4)
            orc.remove(k4)
        assert tab.size() == len(orc.rows)
    gk, gr = tab.export()
    wk, wr = orc.export()
    np.testing.assert_array_equal(gk, wk)
    np.testing.assert_array_equal(gr, wr)


def test_vocab_overflow_is_reported():
    tab = host.EmbLocalTable(4, 8, [(C, 0, 8, 1.0, 0.0, 0, 1.0)])
    tab.gather(np.arange(4))
    with pytest.raises(capi.RecsdkError) as e:
        tab.gather(np.array([10]))
    assert e.value.code == capi.ECAPACITY


def test_swap_kernels_move_rows():
    ext, cache_rows = 32, 64
    descs = [(N, 0, 16, 0.0, 0.01, 5, 1.0), (C, 16, 16, 0.1, 0.0, 0, 1.0)]
    tab, orc = host.EmbLocalTable(500, ext, descs), oracle.HostRows(500, ext, descs)
    cache = torch.zeros((cache_rows, ext), dtype=torch.float32, device=DEV)
    keys = np.array([7, 3, 100, 42])
    slots = torch.tensor([5, 0, 63, 17], dtype=torch.int64, device=DEV)
    tab.swap_in(keys, slots, cache)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(cache[slots].cpu().numpy(), orc.gather(keys))
    cache[slots] += 1.0
    tab.swap_out(keys[:2], slots[:2], cache)
    torch.cuda.synchronize()
    orc.scatter(keys[:2], orc.gather(keys[:2]) + 1.0)
    np.testing.assert_array_equal(tab.gather(keys), orc.gather(keys))


def test_device_key_swaps_create_rows_in_array_order():
    """Swaps with the keys on the device: rows are created in array order and take the next rows of the initializer
    stream, interleaved with calls that take host keys, exactly as the host-key calls do."""
    ext, cache_rows = 32, 4096
    descs = [(N, 0, 16, 0.0, 0.01, 5, 1.0), (TN, 16, 8, 0.0, 0.05, 9, 1.0), (C, 24, 8, 0.1, 0.0, 0, 1.0)]
    tab, orc = host.EmbLocalTable(20000, ext, descs), oracle.HostRows(20000, ext, descs)
    cache = torch.zeros((cache_rows, ext), dtype=torch.float32, device=DEV)
    rng = np.random.default_rng(7)
    for step in range(10):
        m = int(rng.integers(1, 3000))
        keys = rng.choice(15000, m, replace=False).astype(np.int64)
        slots = rng.choice(cache_rows, m, replace=False).astype(np.int64)
        d_slots = torch.from_numpy(slots).to(DEV)
        tab.swap_in(torch.from_numpy(keys).to(DEV), d_slots, cache)
        want = orc.gather(keys)
        np.testing.assert_array_equal(cache[d_slots].cpu().numpy(), want, err_msg=f"step {step}")
        cache[d_slots] += 1.0
        half = m // 2
        tab.swap_out(torch.from_numpy(keys[:half]).to(DEV), d_slots[:half], cache)
        orc.scatter(keys[:half], want[:half] + 1.0)
        # a swap-out of keys the store has never seen creates their rows (and uses up their initial values)
        fresh = (20000 + step * 100 + np.arange(50)).astype(np.int64)
        tab.swap_out(torch.from_numpy(fresh).to(DEV), d_slots[:50], cache)
        orc.scatter(fresh, cache[d_slots[:50]].cpu().numpy())
        # host-key calls in between draw from the same stream
        probe = rng.choice(40000, 40, replace=False).astype(np.int64)
        np.testing.assert_array_equal(tab.gather(probe), orc.gather(probe))
        if step % 3 == 2:
            gone = rng.choice(15000, 500, replace=False).astype(np.int64)
            tab.remove(gone)
            orc.remove(gone)
        assert tab.size() == len(orc.rows)
    for a, b in zip(tab.export(), orc.export()):
        np.testing.assert_array_equal(a, b)


def test_constant_rows_created_on_the_device_hold_their_initial_values_on_the_host():
    """Constant initializers: the store fills every host row once at creation and a device-key swap-in of a key that
    takes a never-used row writes the cache row only.  The host copy of such a row must still read as the initial
    values, and a row that comes back from the freed list (holding another key's old values) must be written again."""
    ext, cache_rows = 16, 512
    descs = [(C, 0, 8, 0.25, 0.0, 0, 2.0), (C, 8, 8, 0.1, 0.0, 0, 1.0)]
    tab, orc = host.EmbLocalTable(1000, ext, descs), oracle.HostRows(1000, ext, descs)
    cache = torch.zeros((cache_rows, ext), dtype=torch.float32, device=DEV)
    rng = np.random.default_rng(3)
    first = np.arange(100, 400, dtype=np.int64)
    slots = torch.arange(300, dtype=torch.int64, device=DEV)
    tab.swap_in(torch.from_numpy(first).to(DEV), slots, cache)
    np.testing.assert_array_equal(cache[:300].cpu().numpy(), orc.gather(first))
    np.testing.assert_array_equal(tab.gather(first), orc.gather(first))          # the host rows, read on the host
    # other values into the host rows, then free most of them
    upd = rng.normal(0, 1, (300, ext)).astype(np.float32)
    tab.scatter(first, upd)
    orc.scatter(first, upd)
    tab.remove(first[:250])
    orc.remove(first[:250])
    # 400 new keys: 250 take freed rows (stale values there), 150 take never-used rows
    second = np.arange(5000, 5400, dtype=np.int64)
    slots2 = torch.arange(400, dtype=torch.int64, device=DEV)
    tab.swap_in(torch.from_numpy(second).to(DEV), slots2, cache)
    want = orc.gather(second)
    np.testing.assert_array_equal(cache[:400].cpu().numpy(), want)
    np.testing.assert_array_equal(tab.gather(second), want)
    np.testing.assert_array_equal(tab.gather(first[250:]), orc.gather(first[250:]))
    assert tab.size() == len(orc.rows)
    for a, b in zip(tab.export(), orc.export()):
        np.testing.assert_array_equal(a, b)


@pytest.mark.parametrize("descs", [
    [(C, 0, 16, 0.25, 0.0, 0, 2.0), (C, 16, 16, 0.1, 0.0, 0, 1.0)],
    [(N, 0, 16, 0.0, 0.01, 5, 1.0), (TN, 16, 8, 0.0, 0.05, 9, 1.0), (C, 24, 8, 0.1, 0.0, 0, 1.0)],
], ids=["constant", "random"])
def test_combined_swap_equals_swap_out_then_swap_in(descs):
    """One call that sends rows out and brings rows in at the same time against the two calls one after the other
    (on the oracle): the rows that come in take the very slots of the rows that go out, some keys that go out are
    new to the store, some that come in were removed before, and the list lengths differ from step to step."""
    ext, cache_rows = 32, 4096
    tab, orc = host.EmbLocalTable(30000, ext, descs), oracle.HostRows(30000, ext, descs)
    cache = torch.zeros((cache_rows, ext), dtype=torch.float32, device=DEV)
    rng = np.random.default_rng(11)
    resident = {}                                   # key -> slot
    free = list(range(cache_rows))
    for step in range(12):
        n_in = int(rng.integers(1, 1500))
        out_keys = rng.permutation(np.array(list(resident), dtype=np.int64))[: int(rng.integers(0, 1 + len(resident)))]
        if step % 4 == 3:
            out_keys = out_keys[:0]                 # nothing goes out: the call falls back to one direction
        out_slots = np.array([resident.pop(int(k)) for k in out_keys], dtype=np.int64)
        free.extend(int(x) for x in out_slots)
        pool = np.setdiff1d(np.arange(20000, dtype=np.int64), np.array(list(resident) + list(out_keys), dtype=np.int64))
        in_keys = rng.choice(pool, min(n_in, len(free)), replace=False)
        in_slots = np.array([free.pop() for _ in in_keys], dtype=np.int64)     # last freed first: the victims' slots
        for k, p in zip(in_keys, in_slots):
            resident[int(k)] = int(p)
        before = cache.cpu().numpy()
        tab.swap(torch.from_numpy(out_keys).to(DEV), torch.from_numpy(out_slots).to(DEV),
                 torch.from_numpy(in_keys).to(DEV), torch.from_numpy(in_slots).to(DEV), cache)
        if len(out_keys):
            orc.scatter(out_keys, before[out_slots])
        want = orc.gather(in_keys)
        torch.cuda.synchronize()
        got = cache.cpu().numpy()
        np.testing.assert_array_equal(got[in_slots], want, err_msg=f"step {step}")
        untouched = np.setdiff1d(np.arange(cache_rows), in_slots)
        np.testing.assert_array_equal(got[untouched], before[untouched])
        # the cached rows change before they go out again; a few keys leave the store altogether
        cache[torch.from_numpy(in_slots).to(DEV)] += float(step + 1)
        if step % 3 == 1:
            gone = rng.choice(20000, 300, replace=False).astype(np.int64)
            gone = np.setdiff1d(gone, np.array(list(resident), dtype=np.int64))
            tab.remove(gone)
            orc.remove(gone)
        if step % 4 == 1:
            # rows filled on the device under keys the store has never seen: their swap-out creates their host rows
            for j in range(20):
                resident[25000 + step * 100 + j] = free.pop()
        assert tab.size() == len(orc.rows), f"step {step}"
    for a, b in zip(tab.export(), orc.export()):
        np.testing.assert_array_equal(a, b)


def test_combined_swap_with_lists_longer_than_one_device_call():
    """Lists above 2^20 keys go in pieces, one direction after the other; the rows still make the round trip."""
    ext, n = 4, 1_200_000
    tab = host.EmbLocalTable(3_000_000, ext, [(C, 0, ext, 0.5, 0.0, 0, 1.0)])
    cache = torch.zeros((n, ext), dtype=torch.float32, device=DEV)
    slots = torch.arange(n, dtype=torch.int64, device=DEV)
    a = torch.arange(n, dtype=torch.int64, device=DEV)
    b = a + n
    none = torch.empty(0, dtype=torch.int64, device=DEV)
    tab.swap(none, none, a, slots, cache)
    assert bool((cache == 0.5).all())
    cache[:, 0] = a.to(torch.float32)                    # exact below 2^24
    cache[:, 3] = -1.0
    tab.swap(a, slots, b, slots, cache)                  # a's rows out, b's rows into the same slots
    assert bool((cache == 0.5).all())
    cache[:, 1] = 7.0
    tab.swap(b[:1000], slots[:1000], a[5000:6000], slots[:1000], cache)
    torch.cuda.synchronize()
    got = cache[:1000].cpu().numpy()
    np.testing.assert_array_equal(got[:, 0], np.arange(5000, 6000, dtype=np.float32))
    np.testing.assert_array_equal(got[:, 1], np.full(1000, 0.5, np.float32))
    np.testing.assert_array_equal(got[:, 3], np.full(1000, -1.0, np.float32))
    assert tab.size() == 2 * n
    np.testing.assert_array_equal(tab.gather(np.arange(n, n + 3))[:, 1], np.full(3, 7.0, np.float32))


def test_device_key_swap_into_full_store_is_reported():
    tab = host.EmbLocalTable(8, 8, [(C, 0, 8, 1.0, 0.0, 0, 1.0)])
    cache = torch.zeros((64, 8), dtype=torch.float32, device=DEV)
    keys = torch.arange(100, 112, dtype=torch.int64, device=DEV)
    slots = torch.arange(12, dtype=torch.int64, device=DEV)
    tab.swap_in(keys, slots, cache)
    torch.cuda.synchronize()
    got = cache.cpu().numpy()
    assert (got[:8] == 1.0).all() and (got[8:12] == 0.0).all()     # the keys past the eighth found no row
    with pytest.raises(capi.RecsdkError) as e:
        tab.size()
    assert e.value.code == capi.ECAPACITY


@pytest.mark.parametrize("device_keys", [False, True])
@pytest.mark.parametrize("dim,cache_rows,universe,batch", [(16, 1024, 2000, 120), (64, 8192, 60000, 1500)])
def test_host_backed_cache_steps_match_oracle(dim, cache_rows, universe, batch, device_keys):
    """Adagrad rows [w | accum] in the host store, a device cache in front of it."""
    ext = 2 * dim
    descs = [(N, 0, dim, 0.0, 0.01, 0, 1.0), (C, dim, dim, 0.1, 0.0, 0, 1.0)]
    rng = np.random.default_rng(dim)
    tab, orc_tab = host.EmbLocalTable(universe, ext, descs), oracle.HostRows(universe, ext, descs)
    om, orc_om = host.OffsetMapper(cache_rows, max_keys=batch * 4), oracle.OffsetMapper(cache_rows)
    cache = torch.zeros((cache_rows, ext), dtype=torch.float32, device=DEV)
    orc_cache = np.zeros((cache_rows, ext), dtype=np.float32)
    rows_h = host.Rows(dim, [cache], [cache.view(-1)[dim:]], None, [ext])
    uq = host.Unique(batch * 4, 1)
    lr = 0.01
    for step in range(25):
        n = batch * 3
        keys = zipf_ranks(rng, 1.05, universe, n).astype(np.int64)
        grad = rng.normal(0, 1e-3, (n, dim)).astype(np.float32)
        dk = torch.from_numpy(keys).to(DEV)
        d_off = torch.tensor([0, n], dtype=torch.int64, device=DEV)
        # ---- device
        uq.run(dk, d_off)
        uk, uo, inv, cnt = uq.fetch()
        slots = uk.clone()
        sik, sip, sok, sop = om.get_swap_pairs_and_key2offset(slots)
        tab.swap_out(sok if device_keys else sok.cpu().numpy(), sop, cache)
        tab.swap_in(sik if device_keys else sik.cpu().numpy(), sip, cache)
        out = host.gather_unique(rows_h, uq, slots)
        host.sparse_apply(rows_h, uq, slots, torch.from_numpy(grad).to(DEV), capi.OPT_ADAGRAD, lr)
        torch.cuda.synchronize()
        # ---- oracle
        split, _, restore, _ = oracle.hash_split(keys, 1)
        off, w_sik, w_sip, w_sok, w_sop = orc_om.get_swap_pairs_and_key2offset(split)
        orc_tab.scatter(w_sok, orc_cache[w_sop])
        orc_cache[w_sip] = orc_tab.gather(w_sik)
        want_out = oracle.gather_rows(orc_cache, ext, off[restore], dim)
        g = oracle.segment_sum(grad, restore, split.size)
        oracle.byaddr_apply(capi.OPT_ADAGRAD, g, off, orc_cache, orc_cache.reshape(-1)[dim:], None, ext, lr,
                            delta_form=False)
        np.testing.assert_array_equal(slots.cpu().numpy(), off)
        np.testing.assert_array_equal(sok.cpu().numpy(), w_sok)
        np.testing.assert_array_equal(out.cpu().numpy(), want_out)
    np.testing.assert_array_equal(cache.cpu().numpy(), orc_cache)
    # flush the cache and compare the stores
    ck, cs = om.export_sorted_kv_pairs()
    tab.swap_out(ck if device_keys else ck.cpu().numpy(), cs, cache)
    torch.cuda.synchronize()
    st = orc_om.state()
    orc_tab.scatter(st["keys"], orc_cache[st["slots"]])
    gk, gr = tab.export()
    wk, wr = orc_tab.export()
    np.testing.assert_array_equal(gk, wk)
    np.testing.assert_array_equal(gr, wr)


def test_swaps_of_the_next_batch_may_run_beside_the_current_batch():
    """The planner reuses a slot only when its key was last needed two calls ago, so the swaps of batch i + 1 can run on
    a second stream while batch i is gathered and updated.  Same results as the one-stream order (oracle)."""
    dim, cache_rows, universe, batch = 32, 6000, 40000, 1200
    ext = 2 * dim
    descs = [(N, 0, dim, 0.0, 0.01, 0, 1.0), (C, dim, dim, 0.1, 0.0, 0, 1.0)]
    rng = np.random.default_rng(3)
    steps = 20
    tab, orc_tab = host.EmbLocalTable(universe, ext, descs), oracle.HostRows(universe, ext, descs)
    om, orc_om = host.OffsetMapper(cache_rows, max_keys=batch), oracle.OffsetMapper(cache_rows)
    cache = torch.zeros((cache_rows, ext), dtype=torch.float32, device=DEV)
    orc_cache = np.zeros((cache_rows, ext), dtype=np.float32)
    rows_h = host.Rows(dim, [cache], [cache.view(-1)[dim:]], None, [ext])
    uqs = [host.Unique(batch, 1), host.Unique(batch, 1)]
    keys = [zipf_ranks(rng, 1.05, universe, batch).astype(np.int64) for _ in range(steps)]
    grads = [rng.normal(0, 1e-3, (batch, dim)).astype(np.float32) for _ in range(steps)]
    d_keys = [torch.from_numpy(k).to(DEV) for k in keys]
    d_grads = [torch.from_numpy(g).to(DEV) for g in grads]
    d_off = torch.tensor([0, batch], dtype=torch.int64, device=DEV)
    outs = [torch.empty((batch, dim), device=DEV) for _ in range(steps)]
    slots = [None, None]
    s_plan, s_rows = torch.cuda.Stream(), torch.cuda.Stream()
    ev_plan = [torch.cuda.Event(), torch.cuda.Event()]
    ev_rows = [torch.cuda.Event(), torch.cuda.Event()]
    torch.cuda.synchronize()

    def plan(i):
        b = i % 2
        with torch.cuda.stream(s_plan):
            if i >= 2:
                s_plan.wait_event(ev_rows[b])
            slots[b] = uqs[b].run(d_keys[i], d_off).fetch()[0]
            sik, sip, sok, sop = om.get_swap_pairs_and_key2offset(slots[b])
            tab.swap_out(sok, sop, cache)
            tab.swap_in(sik, sip, cache)
            ev_plan[b].record(s_plan)

    plan(0)
    for i in range(steps):
        b = i % 2
        with torch.cuda.stream(s_rows):
            s_rows.wait_event(ev_plan[b])
            host.gather_unique(rows_h, uqs[b], slots[b], outs[i])
            host.sparse_apply(rows_h, uqs[b], slots[b], d_grads[i], capi.OPT_ADAGRAD, 0.01)
            ev_rows[b].record(s_rows)
        if i + 1 < steps:
            plan(i + 1)
    torch.cuda.synchronize()
    for i in range(steps):
        split, _, restore, _ = oracle.hash_split(keys[i], 1)
        off, w_sik, w_sip, w_sok, w_sop = orc_om.get_swap_pairs_and_key2offset(split)
        orc_tab.scatter(w_sok, orc_cache[w_sop])
        orc_cache[w_sip] = orc_tab.gather(w_sik)
        want_out = oracle.gather_rows(orc_cache, ext, off[restore], dim)
        g = oracle.segment_sum(grads[i], restore, split.size)
        oracle.byaddr_apply(capi.OPT_ADAGRAD, g, off, orc_cache, orc_cache.reshape(-1)[dim:], None, ext, 0.01,
                            delta_form=False)
        np.testing.assert_array_equal(outs[i].cpu().numpy(), want_out, err_msg=f"step {i}")
    np.testing.assert_array_equal(cache.cpu().numpy(), orc_cache)
