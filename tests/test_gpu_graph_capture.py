"""GPU: one whole step (dedup, key -> slot, gather, segment-reduce + update) recorded into a HIP graph.

The step's entry points take a stream, never synchronise, clear their workspaces with kernels and allocate
nothing once their handles have seen the batch size, and the dedup's side stream forks from and joins the
caller's stream through events: a caller may therefore capture the step once and replay it on new keys.  Every
replay is compared exactly with the same step issued eagerly on a twin state; eager work and synchronisations sit
between the replays.
"""
import ctypes
from ctypes import c_void_p

import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host
from tests.test_gpu_tbe import dev, make_problem
from tests.util import zipf_keys

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def assert_no_memset_nodes(g):
    """The nodes of a graph captured with keep_graph=True: kernels and the event / empty nodes of the library's side
    streams, never a memset (workspaces are cleared by kernels; memset nodes have misbehaved on replays)."""
    kinds = host.graph_node_kinds(g.raw_cuda_graph())
    assert "kernel" in kinds
    assert "memset" not in kinds and "memcpy" not in kinds, sorted(set(kinds))
    g.instantiate()


class StepState:
    def __init__(self, dim, rows, batch, w0, optim):
        self.L = capi.lib()
        self.T = len(rows)
        self.n = int(sum(batch))
        self.optim = optim
        self.w = [w.clone() for w in w0]
        self.acc = [torch.full_like(w, 0.1) for w in w0]
        self.out = torch.empty((self.n, dim), device=DEV)
        self.keys = torch.zeros(self.n, dtype=torch.int64, device=DEV)
        self.grad = torch.zeros((self.n, dim), device=DEV)
        offs = np.concatenate([[0], np.cumsum(batch)]).astype(np.int64)
        self.off = torch.from_numpy(offs).to(DEV)
        self.rows_h = host.Rows(dim, self.w, self.acc, None)
        self.uq = host.Unique(self.n, self.T)
        self.tg = host.EmbeddingTables(rows, self.n)
        self.p_uk, self.p_uo = c_void_p(), c_void_p()
        capi.check(self.L.recsdk_unique_results(self.uq.h, ctypes.byref(self.p_uk), ctypes.byref(self.p_uo), None,
                                                None))

    def step(self, lr=0.01, lr_dev=None):
        """lr_dev: a one-element device tensor the update reads its rate from (instead of the launch argument lr)"""
        sp = c_void_p(torch.cuda.current_stream().cuda_stream)
        L = self.L
        self.uq.run(self.keys, self.off)
        capi.check(L.recsdk_tables_key2offset(self.tg.h, self.p_uk, self.p_uo, self.T, self.n, capi.CHANNEL_TRAIN, sp))
        capi.check(L.recsdk_gather_unique(self.rows_h.h, self.uq.h, self.p_uk, c_void_p(self.out.data_ptr()), sp))
        if lr_dev is not None:
            capi.check(L.recsdk_sparse_apply_lr_dev(self.rows_h.h, self.uq.h, self.p_uk,
                                                    c_void_p(self.grad.data_ptr()), self.optim,
                                                    c_void_p(lr_dev.data_ptr()), 0.9, 0.999, 1e-8, 0.0, sp))
        else:
            capi.check(L.recsdk_sparse_apply(self.rows_h.h, self.uq.h, self.p_uk, c_void_p(self.grad.data_ptr()),
                                             self.optim, float(lr), 0.9, 0.999, 1e-8, 0.0, sp))


@pytest.mark.parametrize("optim", [capi.OPT_ADAGRAD, capi.OPT_SGD])
@pytest.mark.parametrize("rows,batch", [([30000, 500, 9000], [6000, 2500, 4000]),
                                        ([200000], [4000])])   # one table, a small batch: the one-launch kernels
def test_replays_of_a_captured_step_equal_the_eager_step(optim, rows, batch):
    dim = 32
    rng = np.random.default_rng(11)
    w0 = [torch.from_numpy(rng.normal(0, 0.01, (r, dim)).astype(np.float32)).to(DEV) for r in rows]
    eager = StepState(dim, rows, batch, w0, optim)
    graph = StepState(dim, rows, batch, w0, optim)
    n = eager.n

    def batch_no(i):
        keys = np.concatenate([zipf_keys(rng, 1.05, rows[t], batch[t], table=t) for t in range(len(rows))])
        if i % 3 == 1:
            keys[:3000:2] = keys[1]      # one key seen more than 1024 times
        if i % 4 == 2 and n > 8200:
            keys[7000:8200] = keys[7000]  # a long list in the second table
        grad = rng.normal(0, 1e-3, (n, dim)).astype(np.float32)
        return torch.from_numpy(keys.astype(np.int64)).to(DEV), torch.from_numpy(grad).to(DEV)

    def load(state, kg):
        state.keys.copy_(kg[0])
        state.grad.copy_(kg[1])

    # both states see the same first batches eagerly: workspaces reach their steady size before the capture
    for i in range(2):
        kg = batch_no(i)
        for s in (eager, graph):
            load(s, kg)
            s.step()
    torch.cuda.synchronize()
    kg = batch_no(2)
    load(eager, kg)
    load(graph, kg)
    eager.step()
    g = torch.cuda.CUDAGraph(keep_graph=True)
    with torch.cuda.graph(g):
        graph.step()
    assert_no_memset_nodes(g)
    g.replay()   # the capture itself runs nothing
    torch.cuda.synchronize()
    assert torch.equal(eager.out, graph.out)
    for i in range(3, 12):
        kg = batch_no(i)
        load(eager, kg)
        load(graph, kg)
        eager.step()
        g.replay()
        if i % 2 == 0:
            # eager work of the program itself and a synchronisation between replays
            torch.cuda.synchronize()
            assert torch.isfinite((graph.w[0] * 2.0).sum()).item()
        torch.cuda.synchronize()
        assert torch.equal(eager.out, graph.out), f"gather output differs on replay {i}"
        for t in range(len(rows)):
            assert torch.equal(eager.w[t], graph.w[t]), f"weights of table {t} differ on replay {i}"
            assert torch.equal(eager.acc[t], graph.acc[t]), f"accumulators of table {t} differ on replay {i}"
        assert eager.uq.total() == graph.uq.total()


@pytest.mark.parametrize("optim", [capi.OPT_ADAM, capi.OPT_ADAGRAD, capi.OPT_SGD])
def test_a_captured_step_takes_the_rate_of_every_replay_from_device_memory(optim):
    """Adam's bias-corrected rate changes every step and a graph's launch arguments are fixed at capture: the update
    reads the rate from a device word instead, which the caller rewrites before each replay.  Every replay equals the
    eager step that was handed the same rate as a launch argument, bit for bit."""
    dim = 16
    rows = [20000, 3000]
    batch = [5000, 3000]
    rng = np.random.default_rng(23)
    w0 = [torch.from_numpy(rng.normal(0, 0.01, (r, dim)).astype(np.float32)).to(DEV) for r in rows]

    def state():
        s = StepState(dim, rows, batch, w0, optim)
        if optim == capi.OPT_ADAM:           # a second moment beside the first
            s.acc2 = [torch.zeros_like(w) for w in w0]
            for a in s.acc:
                a.zero_()
            s.rows_h = host.Rows(dim, s.w, s.acc, s.acc2)
        return s

    eager, graph = state(), state()
    n = eager.n
    lr_dev = torch.zeros(1, dtype=torch.float32, device=DEV)

    def rate(i):
        return np.float32(0.01 * np.sqrt(1 - 0.999 ** (i + 1)) / (1 - 0.9 ** (i + 1)))

    def batch_no(i):
        keys = np.concatenate([zipf_keys(rng, 1.1, rows[t], batch[t], table=t) for t in range(len(rows))])
        if i % 2 == 1:
            keys[:2600:2] = keys[1]          # one key seen more than 1024 times
        grad = rng.normal(0, 1e-3, (n, dim)).astype(np.float32)
        return torch.from_numpy(keys.astype(np.int64)).to(DEV), torch.from_numpy(grad).to(DEV)

    def load(s, kg):
        s.keys.copy_(kg[0])
        s.grad.copy_(kg[1])

    for i in range(2):
        kg = batch_no(i)
        load(eager, kg)
        load(graph, kg)
        lr_dev.fill_(float(rate(i)))
        eager.step(lr=rate(i))
        graph.step(lr_dev=lr_dev)            # the device-rate entry point issued eagerly
    torch.cuda.synchronize()
    for t in range(len(rows)):
        assert torch.equal(eager.w[t], graph.w[t])
    kg = batch_no(2)
    load(eager, kg)
    load(graph, kg)
    eager.step(lr=rate(2))
    lr_dev.fill_(float(rate(2)))
    g = torch.cuda.CUDAGraph(keep_graph=True)
    with torch.cuda.graph(g):
        graph.step(lr_dev=lr_dev)
    assert_no_memset_nodes(g)
    g.replay()
    torch.cuda.synchronize()
    for i in range(3, 10):
        kg = batch_no(i)
        load(eager, kg)
        load(graph, kg)
        eager.step(lr=rate(i))
        lr_dev.fill_(float(rate(i)))          # a fill kernel on the stream, before the replay
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(eager.out, graph.out), f"gather output differs on replay {i}"
        for t in range(len(rows)):
            assert torch.equal(eager.w[t], graph.w[t]), f"weights of table {t} differ on replay {i}"
            assert torch.equal(eager.acc[t], graph.acc[t]), f"first state of table {t} differs on replay {i}"


@pytest.mark.parametrize("optim", [capi.OPT_SGD, capi.OPT_ADAGRAD])
def test_replays_of_a_captured_pooled_backward_equal_the_oracle(optim):
    """The backward forks onto the dedup handle's stream (classes of the long lists) and onto the update's side stream
    (chunk sums): both must join the capturing stream again, and every replay must give the eager result."""
    T, B, dims, rows = 4, 2500, [64, 64, 16, 128], [3000, 20, 100000, 500]
    d_off, w_off, hcs, offsets, indices, weights = make_problem(5, T, B, dims, rows, 30, alpha=1.1, min_len=1)
    total_d, max_d = int(d_off[-1]), max(dims)
    w_host = weights.copy()
    w_dev = dev(weights)
    m1 = np.full_like(weights, 0.1) if optim == capi.OPT_ADAGRAD else np.zeros_like(weights)
    m2 = np.zeros_like(weights)
    d_m1, d_m2 = dev(m1), dev(m2)
    bw = host.SplitEmbeddingBackward(T, indices.size)
    d_args = (dev(w_off), dev(d_off), total_d, max_d, dev(hcs), dev(indices), dev(offsets))
    rng = np.random.default_rng(6)
    gbuf = torch.zeros((B, total_d), device="cuda:0")

    def check(gout):
        oracle.tbe_backward(optim, gout, w_host, w_off, d_off, total_d, hcs, indices, offsets, T, B, capi.POOL_SUM, m1, m2,
                            0.05, 1e-8, 0.9, 0.999, 1, bf16=False)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(w_dev.cpu().numpy(), w_host)
        np.testing.assert_array_equal(d_m1.cpu().numpy(), m1)

    def step():
        bw(optim, gbuf, w_dev, *d_args, capi.POOL_SUM, d_m1, d_m2, 0.05, 1e-8, 0.9, 0.999, 1)

    gout = rng.normal(0, 1e-2, (B, total_d)).astype(np.float32)
    gbuf.copy_(dev(gout))
    step()                                  # eager: every buffer that grows on demand has its size
    check(gout)
    g = torch.cuda.CUDAGraph(keep_graph=True)
    cs = torch.cuda.Stream()
    cs.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(cs):
        with torch.cuda.graph(g, stream=cs):
            step()
    torch.cuda.current_stream().wait_stream(cs)
    assert_no_memset_nodes(g)
    for _ in range(3):
        gout = rng.normal(0, 1e-2, (B, total_d)).astype(np.float32)
        gbuf.copy_(dev(gout))
        torch.cuda.synchronize()
        g.replay()
        check(gout)
        _ = (w_dev * 1.0).sum().item()      # eager work and a synchronisation between replays
