"""GPU: the reference's torch operator names (fbgemm::split_embedding_*, registered by recsdk_amd/torch_ops for ROCm
tensors) called the way the reference's python layer calls them, against the CPU oracle: forward, the three exact
backward operators, and the lookup functions whose autograd backward runs the fused update."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, torch_ops
from tests.test_gpu_tbe import dev, make_problem

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    torch_ops.load()
    return torch.ops.fbgemm


def problem(seed=9):
    T, B, dims, rows = 4, 300, [64, 32, 16, 128], [3000, 20, 50000, 500]
    d_off, w_off, hcs, offsets, indices, weights = make_problem(seed, T, B, dims, rows, 20, alpha=1.1, min_len=1)
    return T, B, int(d_off[-1]), max(dims), d_off, w_off, hcs, offsets, indices, weights


def test_forward_operator(ops):
    T, B, total_d, max_d, d_off, w_off, hcs, offsets, indices, weights = problem()
    none = torch.empty(0, device=DEV)
    for mode in (capi.POOL_SUM, capi.POOL_MEAN):
        out = ops.split_embedding_codegen_forward_unweighted_cuda(
            dev(weights), none, none, none, dev(w_off), dev(d_off), total_d, max_d, dev(indices), dev(offsets), mode,
            none, none, 0, False, none, none)
        want = oracle.tbe_forward(weights, w_off, d_off, total_d, indices, offsets, T, B, mode)
        np.testing.assert_array_equal(out.cpu().numpy(), want)
    # int32 index tensors, as torchrec hands them over, are accepted
    out = ops.split_embedding_codegen_forward_unweighted_cuda(
        dev(weights), none, none, none, dev(w_off), dev(d_off), total_d, max_d, dev(indices).int(), dev(offsets).int(),
        capi.POOL_SUM, none, none, 0, False, none, none)
    np.testing.assert_array_equal(out.cpu().numpy(),
                                  oracle.tbe_forward(weights, w_off, d_off, total_d, indices, offsets, T, B, 0))


@pytest.mark.parametrize("optim", ["sgd", "adagrad", "adam"])
def test_backward_operators(ops, optim):
    T, B, total_d, max_d, d_off, w_off, hcs, offsets, indices, weights = problem(10)
    none = torch.empty(0, device=DEV)
    w_host, m1, m2 = weights.copy(), np.zeros_like(weights), np.zeros_like(weights)
    w_dev, d_m1, d_m2 = dev(weights), dev(m1), dev(m2)
    head = lambda g: (g, w_dev, none, none, none, dev(w_off), dev(d_off), max_d, dev(hcs), 0, dev(indices), dev(offsets),
                      capi.POOL_SUM, none, 0, 0, False, 0, 0, False, False)
    mom1 = (d_m1, none, none, none)
    mom2 = (d_m2, none, none, none)
    tail = (none, none, none, none, none)   # hash_indices, unique_ids, unique_offsets, unique_inverse, offset_per_key:
    #                                         declared `Tensor x = None`, so a caller hands over tensors, as the reference's do
    code = {"sgd": capi.OPT_SGD, "adagrad": capi.OPT_ADAGRAD, "adam": capi.OPT_ADAM}[optim]
    rng = np.random.default_rng(12)
    for it in range(1, 4):
        gout = rng.normal(0, 1e-2, (B, total_d)).astype(np.float32)
        if optim == "sgd":
            ops.split_embedding_backward_codegen_sgd_unweighted_exact_cuda(*head(dev(gout)), *tail, learning_rate=0.05)
        elif optim == "adagrad":
            ops.split_embedding_backward_codegen_adagrad_unweighted_exact_cuda(*head(dev(gout)), *mom1, *tail, eps=1e-8,
                                                                               learning_rate=0.05)
        else:
            ops.split_embedding_backward_codegen_adam_unweighted_exact_cuda(
                *head(dev(gout)), *mom1, *mom2, *tail, eps=1e-8, learning_rate=0.05, beta1=0.9, beta2=0.999, iter=it)
        oracle.tbe_backward(code, gout, w_host, w_off, d_off, total_d, hcs, indices, offsets, T, B, capi.POOL_SUM, m1, m2,
                            0.05, 1e-8, 0.9, 0.999, it)
        np.testing.assert_array_equal(w_dev.cpu().numpy(), w_host)
        np.testing.assert_array_equal(d_m1.cpu().numpy(), m1)
        np.testing.assert_array_equal(d_m2.cpu().numpy(), m2)


def test_lookup_function_trains_through_autograd(ops):
    """split_embedding_codegen_lookup_adam_function: the output feeds a loss, loss.backward() runs the fused
    segment-reduce + Adam on the tables in place (the reference's test_split_embedding_codegen_lookup_function.py
    drives the operator the same way)."""
    T, B, total_d, max_d, d_off, w_off, hcs, offsets, indices, weights = problem(11)
    none = torch.empty(0, device=DEV)
    w_host, m1, m2 = weights.copy(), np.zeros_like(weights), np.zeros_like(weights)
    w_dev, d_m1, d_m2 = dev(weights), dev(m1), dev(m2)
    rng = np.random.default_rng(13)
    for it in range(1, 4):
        placeholder = torch.zeros(1, device=DEV, requires_grad=True)
        out = ops.split_embedding_codegen_lookup_adam_function(
            placeholder, w_dev, none, none, none, dev(w_off), dev(d_off), total_d, max_d, dev(hcs), 0, dev(indices),
            dev(offsets), capi.POOL_SUM, None, None, none, False, 0.0, False, d_m1, none, none, none, d_m2, none, none,
            none, eps=1e-8, learning_rate=0.01, beta1=0.9, beta2=0.999, iter=it)
        assert out.requires_grad
        want_out = oracle.tbe_forward(w_host, w_off, d_off, total_d, indices, offsets, T, B, capi.POOL_SUM)
        np.testing.assert_array_equal(out.detach().cpu().numpy(), want_out)
        coef = rng.normal(0, 1e-2, (B, total_d)).astype(np.float32)
        (out * dev(coef)).sum().backward()           # d loss / d out = coef
        oracle.tbe_backward(capi.OPT_ADAM, coef, w_host, w_off, d_off, total_d, hcs, indices, offsets, T, B,
                            capi.POOL_SUM, m1, m2, 0.01, 1e-8, 0.9, 0.999, it)
        np.testing.assert_array_equal(w_dev.cpu().numpy(), w_host)
        np.testing.assert_array_equal(d_m1.cpu().numpy(), m1)
        np.testing.assert_array_equal(d_m2.cpu().numpy(), m2)
    # without a gradient requirement the function is a plain lookup
    with torch.no_grad():
        out = ops.split_embedding_codegen_lookup_sgd_function(
            torch.zeros(1, device=DEV), w_dev, none, none, none, dev(w_off), dev(d_off), total_d, max_d, dev(hcs), 0,
            dev(indices), dev(offsets), capi.POOL_SUM, None, None, none, False, 0.0, False, learning_rate=0.1)
    np.testing.assert_array_equal(out.cpu().numpy(),
                                  oracle.tbe_forward(w_host, w_off, d_off, total_d, indices, offsets, T, B, 0))


def test_ids_mapper_torch_class_matches_reference_vectors(ops):
    """torch.classes.hybrid.IdsMapper, one mapper per table as hybrid_torchrec creates them, against the vectors
    recorded from the reference's own IdsMapper::ParallelUniqueHashOut (tests/golden/ref_vectors.npz)."""
    import os

    G = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_vectors.npz"))
    T, steps = (int(x) for x in G["ids_a_cfg"])
    mappers = [torch.classes.hybrid.IdsMapper(10 ** 6, True) for _ in range(T)]
    for s in range(steps):
        offs, ids = G[f"ids_a_{s}_offs"], G[f"ids_a_{s}_ids"]
        n = ids.size
        d_ids = dev(ids)
        hash_idx = torch.full((n,), -7, dtype=torch.int64, device=DEV)
        uniq = torch.full((n,), -7, dtype=torch.int64, device=DEV)
        uniq_ids = torch.full((n,), -7, dtype=torch.int64, device=DEV)
        inv = torch.full((n,), -7, dtype=torch.int64, device=DEV)
        uoff = torch.zeros(T + 1, dtype=torch.int64)
        torch.classes.hybrid.IdsMapper.parallel_ids2indices_unique_out(mappers, d_ids, hash_idx, torch.from_numpy(offs),
                                                                       uniq, uniq_ids, inv, uoff)
        want_uoff = G[f"ids_a_{s}_uoff"]
        u = int(want_uoff[-1])
        np.testing.assert_array_equal(uoff.numpy(), want_uoff)
        np.testing.assert_array_equal(uniq_ids.cpu().numpy()[:u], G[f"ids_a_{s}_uniq_ids"])
        np.testing.assert_array_equal(uniq.cpu().numpy()[:u], G[f"ids_a_{s}_uniq"])
        np.testing.assert_array_equal(inv.cpu().numpy(), G[f"ids_a_{s}_inv"])
        np.testing.assert_array_equal(hash_idx.cpu().numpy(), G[f"ids_a_{s}_hash_idx"])
    # the single-table call: indices continue the mapper's state; unique is the sorted distinct indices
    ids = np.array([5, 900, 5, 17, 900, 5], dtype=np.int64)
    fresh = torch.classes.hybrid.IdsMapper(100, True)
    hash_idx, uniq, inv = fresh.ids2indices_unique(dev(ids))
    np.testing.assert_array_equal(hash_idx.cpu().numpy(), [0, 1, 0, 2, 1, 0])
    np.testing.assert_array_equal(uniq.cpu().numpy(), [0, 1, 2])
    np.testing.assert_array_equal(inv.cpu().numpy(), [0, 1, 0, 2, 1, 0])
    hash_idx, uniq, inv = fresh.ids2indices_unique(dev(np.array([17, 3, 5], dtype=np.int64)))
    np.testing.assert_array_equal(hash_idx.cpu().numpy(), [2, 3, 0])
    np.testing.assert_array_equal(uniq.cpu().numpy(), [0, 2, 3])
    np.testing.assert_array_equal(inv.cpu().numpy(), [1, 2, 0])
    small = torch.classes.hybrid.IdsMapper(2, True)
    with pytest.raises(RuntimeError, match="Ids map reached maxIndex"):
        small.ids2indices_unique(dev(np.array([1, 2, 3], dtype=np.int64)))
    with pytest.raises(RuntimeError, match="Invalid key value"):
        fresh.ids2indices_unique(dev(np.array([1, -4], dtype=np.int64)))
