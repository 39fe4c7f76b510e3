"""The library's own radix sort through the C ABI (recsdk_sort_pairs) against numpy's stable sort: bit-exact keys and,
because the sort is stable, bit-exact values.  Sizes cover every tile shape (2048 / 4096 / 8192 pairs, the last as
1024 x 8 and as 512 x 16), every digit width (8, 9, 10 bits), partial last tiles, one pair, and keys with a heavy head
(what the row grouping of a Zipf batch sorts)."""
import numpy as np
import pytest
import torch

from recsdk_amd import capi, host

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _keys(rng, n, bits, dist, dtype):
    top = (1 << bits) - 1
    if dist == "uniform":
        k = rng.integers(0, top + 1, n, dtype=np.uint64)
    elif dist == "head":          # a few values hold most of the mass, the high digits barely vary
        k = np.minimum((rng.pareto(1.1, n) * 3).astype(np.uint64), np.uint64(top))
    elif dist == "three":
        k = rng.integers(0, 3, n, dtype=np.uint64) & np.uint64(top)
    else:                         # all equal: the sort must return the input order
        k = np.full(n, top // 2, dtype=np.uint64)
    return k.astype(dtype)


def _check(n, bits, dist, key_bytes=4, descending=False, seed=0):
    rng = np.random.default_rng(seed + n + bits)
    np_dtype = np.uint32 if key_bytes == 4 else np.uint64
    t_dtype = torch.int32 if key_bytes == 4 else torch.int64
    keys = _keys(rng, n, bits, dist, np_dtype)
    vals = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
    order = np.argsort(keys if not descending else ~keys, kind="stable")
    sorter = host.Sorter(n, key_bytes)
    d_keys = torch.from_numpy(keys.view(np.int32 if key_bytes == 4 else np.int64)).to(DEV)
    d_vals = torch.from_numpy(vals.view(np.int32)).to(DEV)
    assert d_keys.dtype == t_dtype
    out_k, out_v = sorter.sort_pairs(d_keys, d_vals, bits, descending)
    torch.cuda.synchronize()
    got_k = out_k.cpu().numpy().view(np_dtype)
    got_v = out_v.cpu().numpy().view(np.uint32)
    assert np.array_equal(got_k, keys[order])
    assert np.array_equal(got_v, vals[order])
    # the inputs are untouched
    assert np.array_equal(d_keys.cpu().numpy().view(np_dtype), keys)
    sorter.close()


@pytest.mark.parametrize("n,bits", [(1, 1), (63, 5), (64, 32), (2048, 8), (2049, 9), (5000, 13), (40000, 16),
                                    (99999, 18), (100000, 17), (131072, 17), (300000, 19), (1048575, 20),
                                    (1048576, 27), (1703936, 16), (2200000, 21), (4194304, 26), (4200001, 32)])
@pytest.mark.parametrize("dist", ["uniform", "head", "three", "equal"])
def test_sort_pairs_u32_matches_numpy_stable_sort(n, bits, dist):
    _check(n, bits, dist)


@pytest.mark.parametrize("n,bits,desc", [(100000, 20, True), (777, 9, True), (2500000, 30, True), (1200000, 10, True)])
def test_sort_pairs_u32_descending_is_stable(n, bits, desc):
    _check(n, bits, "head", descending=desc)


@pytest.mark.parametrize("n,bits,desc", [(1, 64, False), (100000, 40, False), (50000, 64, True), (2500000, 64, True),
                                         (300000, 30, False), (1100000, 57, True), (4300000, 33, False)])
@pytest.mark.parametrize("dist", ["uniform", "head"])
def test_sort_pairs_u64_matches_numpy_stable_sort(n, bits, desc, dist):
    _check(n, bits, dist, key_bytes=8, descending=desc)


def test_one_sorter_serves_sorts_of_different_sizes_back_to_back():
    """no state survives a call: a small sort after a large one (other tile shape, other digit width) is exact"""
    rng = np.random.default_rng(5)
    sorter = host.Sorter(5_000_000)
    for n, bits in [(5_000_000, 26), (1000, 10), (1_500_000, 19), (70_000, 32), (5_000_000, 8)]:
        keys = rng.integers(0, 1 << bits, n, dtype=np.uint64).astype(np.uint32)
        vals = np.arange(n, dtype=np.uint32)
        out_k, out_v = sorter.sort_pairs(torch.from_numpy(keys.view(np.int32)).to(DEV),
                                         torch.from_numpy(vals.view(np.int32)).to(DEV), bits)
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(out_k.cpu().numpy().view(np.uint32), keys[order])
        assert np.array_equal(out_v.cpu().numpy().view(np.uint32), vals[order])
    sorter.close()


def test_argument_errors():
    sorter = host.Sorter(1000)
    k = torch.zeros(2000, dtype=torch.int32, device=DEV)
    v = torch.zeros(2000, dtype=torch.int32, device=DEV)
    with pytest.raises(capi.RecsdkError) as e:
        sorter.sort_pairs(k, v, 8)
    assert e.value.code == capi.ECAPACITY
    with pytest.raises(capi.RecsdkError) as e:
        sorter.sort_pairs(k[:10], v[:10], 33)
    assert e.value.code == capi.EINVAL
    L = capi.lib()
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    import ctypes
    assert L.recsdk_sort_pairs(sorter.h, p(k), p(k), p(v), p(v), 10, 8, 0, None) == capi.EINVAL   # outputs alias inputs
    sorter.close()
    h = ctypes.c_void_p()
    assert L.recsdk_sorter_create(10, 3, ctypes.byref(h)) == capi.EINVAL
    assert L.recsdk_sorter_create(0, 4, ctypes.byref(h)) == capi.EINVAL


def test_a_captured_sort_records_kernel_nodes_only_and_replays_exactly():
    """The sort inside a HIP graph: no memset node among the graph's nodes (the look-back words are cleared by a
    kernel), and every replay on new keys equals the eager result."""
    rng = np.random.default_rng(11)
    n, bits = 300_000, 19
    sorter = host.Sorter(n)
    kbuf = torch.zeros(n, dtype=torch.int32, device=DEV)
    vbuf = torch.arange(n, dtype=torch.int32, device=DEV)
    out = {}
    g = torch.cuda.CUDAGraph(keep_graph=True)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        sorter.sort_pairs(kbuf, vbuf, bits)   # warm
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=s):
            out["k"], out["v"] = sorter.sort_pairs(kbuf, vbuf, bits)
    torch.cuda.current_stream().wait_stream(s)
    kinds = host.graph_node_kinds(g.raw_cuda_graph())
    assert kinds, "the captured graph is empty"
    assert set(kinds) == {"kernel"}, kinds
    g.instantiate()
    for rep in range(4):
        keys = rng.integers(0, 1 << bits, n, dtype=np.uint64).astype(np.uint32)
        kbuf.copy_(torch.from_numpy(keys.view(np.int32)).to(DEV))
        torch.cuda.synchronize()          # the program's own work between replays
        g.replay()
        torch.cuda.synchronize()
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(out["k"].cpu().numpy().view(np.uint32), keys[order]), rep
        assert np.array_equal(out["v"].cpu().numpy().view(np.uint32), order.astype(np.uint32)), rep
    sorter.close()
