"""GPU: the dynamic-expansion step with nothing returning to the host.  Admission takes its timestamp from device memory
(recsdk_faae_admit_distinct_dev), eviction leaves its keys and their count on the device (recsdk_faae_evict_dev) and
recsdk_tables_evict consumes them there.  Checked (1) against the CPU oracle step by step: distinct keys, admission
mask, addresses, and the evicted keys as SETS (the device-side eviction fixes no order; a dynamic table never reuses an
address, so the order has no effect on later steps); (2) as a HIP graph: every replay of the captured step equals the
same step issued eagerly on a twin state."""
import ctypes
from ctypes import c_void_p

import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host
from recsdk_amd.synth import ZipfSampler, splitmix64

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DIM, EXT = 32, 96


class Loop:
    """One table of dynamic addresses over an arena of [w | m | v] rows, admission >= 2, eviction idle > `idle`."""

    def __init__(self, slots, batch, idle, history, evict_beside=False):
        self.L = capi.lib()
        # the eviction on a stream of its own beside the step's gather and update (what the benchmark does)
        self.s_evict = torch.cuda.Stream() if evict_beside else None
        self.ev_fork, self.ev_join = torch.cuda.Event(), torch.cuda.Event()
        self.batch = batch
        self.arena = torch.zeros((slots, EXT), device=DEV)
        flat = self.arena.view(-1)
        self.rows_h = host.Rows(DIM, [self.arena], [flat[DIM:]], [flat[2 * DIM:]], [EXT])
        self.uq = host.Unique(batch, 1)
        self.tg = host.EmbeddingTables([slots], 1 << 18, dynamic=[1], arena_bases=[self.arena.data_ptr()],
                                       row_bytes=[EXT * 4])
        self.f = host.FeatureAdmitAndEvict([history], [2], [idle], max_keys=batch)
        self.keys = torch.zeros(batch, dtype=torch.int64, device=DEV)
        self.grad = torch.zeros((batch, DIM), device=DEV)
        self.out = torch.zeros((batch, DIM), device=DEV)
        self.addr = torch.zeros(batch, dtype=torch.int64, device=DEV)    # per distinct key: address, 0 = not admitted
        self.slots = torch.zeros(batch, dtype=torch.int64, device=DEV)   # the same as row numbers of the arena
        self.ts = torch.zeros(1, dtype=torch.int64, device=DEV)
        self.off = torch.tensor([0, batch], dtype=torch.int64, device=DEV)
        self.ev_cap = 1 << 18
        self.ev_keys = torch.zeros(self.ev_cap, dtype=torch.int64, device=DEV)
        self.ev_off = torch.zeros(2, dtype=torch.int64, device=DEV)
        self.p_uk, self.p_uo, self.p_cnt = c_void_p(), c_void_p(), c_void_p()
        capi.check(self.L.recsdk_unique_results(self.uq.h, ctypes.byref(self.p_uk), ctypes.byref(self.p_uo), None,
                                                ctypes.byref(self.p_cnt)))

    def evict(self, sp):
        L = self.L
        capi.check(L.recsdk_faae_evict_dev(self.f.h, 0, c_void_p(self.ev_keys.data_ptr()), self.ev_cap,
                                           c_void_p(self.ev_off.data_ptr()), sp))
        capi.check(L.recsdk_tables_evict(self.tg.h, c_void_p(self.ev_keys.data_ptr()), c_void_p(self.ev_off.data_ptr()),
                                         1, self.ev_cap, sp))

    def step(self):
        cur = torch.cuda.current_stream()
        L, sp = self.L, c_void_p(cur.cuda_stream)
        self.uq.run(self.keys, self.off)
        capi.check(L.recsdk_faae_admit_distinct_dev(self.f.h, capi.CHANNEL_TRAIN, self.p_uk, self.p_cnt, self.p_uo, 1,
                                                    self.batch, c_void_p(self.ts.data_ptr()), sp))
        capi.check(L.recsdk_tables_key2offset(self.tg.h, self.p_uk, self.p_uo, 1, self.batch, capi.CHANNEL_TRAIN, sp))
        # addresses -> row numbers of the arena for the row kernels (-1: the key was not admitted)
        capi.check(L.recsdk_unique_fetch(self.uq.h, c_void_p(self.addr.data_ptr()), None, None, None, sp))
        if self.s_evict is not None:
            # history and key -> slot table are final for this step; the rows are not the eviction's business
            self.ev_fork.record(cur)
            self.s_evict.wait_event(self.ev_fork)
            self.evict(c_void_p(self.s_evict.cuda_stream))
            self.ev_join.record(self.s_evict)
        torch.sub(self.addr, self.arena.data_ptr(), out=self.slots)
        self.slots.div_(EXT * 4, rounding_mode="floor")
        self.slots.masked_fill_(self.addr == 0, -1)
        capi.check(L.recsdk_gather_unique(self.rows_h.h, self.uq.h, c_void_p(self.slots.data_ptr()),
                                          c_void_p(self.out.data_ptr()), sp))
        capi.check(L.recsdk_sparse_apply(self.rows_h.h, self.uq.h, c_void_p(self.slots.data_ptr()),
                                         c_void_p(self.grad.data_ptr()), capi.OPT_ADAM, 1e-3, 0.9, 0.999, 1e-8, 0.0, sp))
        if self.s_evict is not None:
            cur.wait_event(self.ev_join)
        else:
            self.evict(sp)

    def distinct_keys_and_addresses(self):
        return self.addr[:self.uq.total()].cpu().numpy()


def make_batches(n_batches, batch, hot, seed):
    rng = np.random.default_rng(seed)
    sampler = ZipfSampler(1.2, hot)
    fresh = 1 << 40
    out = []
    for _ in range(n_batches):
        is_hot = rng.random(batch) < 0.7
        keys = np.where(is_hot, splitmix64(sampler.ranks(rng, batch).astype(np.uint64)),
                        splitmix64(np.arange(fresh, fresh + batch, dtype=np.uint64))).astype(np.int64)
        fresh += batch
        out.append((keys, rng.normal(0, 1e-3, (batch, DIM)).astype(np.float32)))
    return out


@pytest.mark.parametrize("evict_beside", [False, True])
def test_device_only_loop_matches_the_oracle_and_replays_as_a_graph(evict_beside):
    slots, batch, hot, idle, steps = 2_000_000, 32768, 200_000, 5, 40
    batches = make_batches(steps, batch, hot, seed=9)
    eager = Loop(slots, batch, idle, 1 << 20, evict_beside)
    graph = Loop(slots, batch, idle, 1 << 20, evict_beside)
    orc_f = oracle.Faae(2, idle)
    orc_t = oracle.Table(slots, dynamic=True, arena_base=eager.arena.data_ptr(), row_bytes=EXT * 4)
    g = None
    evicted_total = 0
    for step, (keys, grad) in enumerate(batches):
        for s in (eager, graph):
            s.keys.copy_(torch.from_numpy(keys))
            s.grad.copy_(torch.from_numpy(grad))
            s.ts.fill_(step)
        eager.step()
        if step < 8:
            graph.step()                       # workspaces reach their steady size, evictions have begun
        elif g is None:
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph(keep_graph=True)
            with torch.cuda.graph(g):
                graph.step()
            kinds = host.graph_node_kinds(g.raw_cuda_graph())
            assert "kernel" in kinds and "memset" not in kinds, sorted(set(kinds))   # workspaces are cleared by kernels
            g.instantiate()
            g.replay()
        else:
            g.replay()
        torch.cuda.synchronize()
        # (1) the eager device loop against the oracle
        split, _, restore, counts = oracle.hash_split(keys, 1, with_counts=True)
        want_adm = orc_f.admit(split, counts, step, capi.CHANNEL_TRAIN)
        want_addr, rc = orc_t.key2offset(want_adm, capi.CHANNEL_TRAIN)
        assert rc == 0
        got_addr = eager.distinct_keys_and_addresses()
        np.testing.assert_array_equal(got_addr, want_addr, err_msg=f"addresses, step {step}")
        want_ev = orc_f.evict()
        orc_t.evict(want_ev)
        m = int(eager.ev_off.cpu()[1])
        assert m == want_ev.size, f"evicted count, step {step}"
        np.testing.assert_array_equal(np.sort(eager.ev_keys[:m].cpu().numpy()), np.sort(want_ev))
        evicted_total += m
        # (2) the twin state driven by the graph
        # addresses differ between the twins by their arenas' bases: compare what they hold and read
        assert torch.equal(eager.out, graph.out), f"gathered rows differ at step {step}"
        assert torch.equal(eager.ev_off, graph.ev_off)
        gm = int(graph.ev_off.cpu()[1])
        assert torch.equal(torch.sort(eager.ev_keys[:m]).values, torch.sort(graph.ev_keys[:gm]).values)
    assert evicted_total > 50_000
    assert torch.equal(eager.arena, graph.arena)
    for s in (eager, graph):
        live, latest = s.f.stats()
        assert live[0] == orc_f.dump()[0].size and latest[0] == steps - 1
        mo, lv, _ = s.tg.stats()
        assert mo[0] == orc_t.size and lv[0] == orc_t.live
