"""GPU parity of the pooled-lookup operators in the cases of the reference's operator test beyond one feature per
table (test_split_embedding_codegen_lookup_function.py:320-350): features that share a table, no pooling in the
backward, hash_indices in place of indices, and the unique variant fed with inputs built as the reference's
generate_unique builds them (:268-287).  Through the C ABI and through torch.ops.fbgemm, bit-exact against the CPU oracle
run on the hashed indices."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host, torch_ops
from tests.tbe_cases import TbeProblem

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
LR, EPS, B1, B2 = 0.05, 1e-8, 0.9, 0.999
CODES = {"sgd": capi.OPT_SGD, "adagrad": capi.OPT_ADAGRAD, "adam": capi.OPT_ADAM}


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def total_d_of(p, mode):
    return p.max_d * p.F if mode == capi.POOL_NONE else p.total_d


CASES = [
    ([(20000, 32), (40000, 32)], [0, 0, 1], 16, [8, 16, 100]),      # the reference test's two-table shapes
    ([(40000, 128), (80000, 128)], [0, 1, 1], 8, [2, 64, 200]),
    ([(1234, 64)], [0], 301, [11]),
    ([(500, 8), (3, 8), (70000, 8), (900, 8)], [0, 1, 1, 3], 64, [3, 70, 5, 1]),   # table 2 unused by any feature
]


@pytest.mark.parametrize("unique", [False, True])
@pytest.mark.parametrize("optim", ["sgd", "adagrad", "adam"])
@pytest.mark.parametrize("mode", [capi.POOL_SUM, capi.POOL_MEAN, capi.POOL_NONE])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_backward_c_abi(case, mode, optim, unique):
    tables, fmap, batch, hots = CASES[case]
    p = TbeProblem(100 + case, tables, fmap, batch, max_len=0, fixed_len=hots)
    total_d = total_d_of(p, mode)
    bwd = host.SplitEmbeddingBackward(p.F, p.nnz)
    w, m1, m2 = p.weights.copy(), np.zeros_like(p.weights), np.zeros_like(p.weights)
    d_w, d_m1, d_m2 = dev(w), dev(m1), dev(m2)
    uid, uoff, uinv = p.unique_inputs()
    kw = dict(unique_ids=dev(uid), unique_offsets=dev(uoff), unique_inverse=dev(uinv)) if unique else {}
    for it in range(1, 4):
        gout = p.rng.normal(0, 1e-2, p.grad_shape(mode)).astype(np.float32)
        out = host.split_embedding_codegen_forward_unweighted(d_w, dev(p.weights_offsets), dev(p.d_offsets), total_d,
                                                              p.max_d, dev(p.indices), dev(p.offsets), mode)
        np.testing.assert_array_equal(out.cpu().numpy(),
                                      oracle.tbe_forward(w, p.weights_offsets, p.d_offsets, total_d, p.indices,
                                                         p.offsets, p.F, p.B, mode))
        bwd(CODES[optim], dev(gout), d_w, dev(p.weights_offsets), dev(p.d_offsets), total_d, p.max_d,
            dev(p.hash_size_cumsum), dev(p.indices), dev(p.offsets), mode, d_m1, d_m2, LR, EPS, B1, B2, it, **kw)
        oracle.tbe_backward(CODES[optim], gout, w, p.weights_offsets, p.d_offsets, total_d, p.hash_size_cumsum,
                            p.indices, p.offsets, p.F, p.B, mode, m1, m2, LR, EPS, B1, B2, it)
        np.testing.assert_array_equal(d_w.cpu().numpy(), w)
        np.testing.assert_array_equal(d_m1.cpu().numpy(), m1)
        np.testing.assert_array_equal(d_m2.cpu().numpy(), m2)


def test_unique_variant_leaves_out_what_lies_outside_its_table():
    p = TbeProblem(7, [(50, 8), (60, 8)], [0, 1], 33, max_len=6)
    uid, uoff, uinv = p.unique_inputs()
    uid2, uinv2 = uid.copy(), uinv.copy()
    bad_row = int(uoff[1]) - 1           # last distinct row of table 0 -> outside the table
    uid2[bad_row] = 50
    uinv2[3] = 10 ** 6                   # a position whose inverse lies outside its table's slice
    gout = p.rng.normal(0, 1, (p.B, p.total_d)).astype(np.float32)
    d_w = dev(p.weights)
    bwd = host.SplitEmbeddingBackward(p.F, p.nnz)
    bwd(capi.OPT_SGD, dev(gout), d_w, dev(p.weights_offsets), dev(p.d_offsets), p.total_d, p.max_d,
        dev(p.hash_size_cumsum), dev(p.indices), dev(p.offsets), capi.POOL_SUM, learning_rate=LR,
        unique_ids=dev(uid2), unique_offsets=dev(uoff), unique_inverse=dev(uinv2))
    # the same on the CPU with position 3 and the bad row's positions dropped: zero their gradient contribution by
    # running the oracle on a copy of the problem in which those positions sit in an empty slot of a bag
    keep = np.ones(p.nnz, bool)
    keep[3] = False
    keep[:p.offsets[p.B]] &= uinv[:p.offsets[p.B]] != (bad_row - uoff[0])
    w = p.weights.copy()
    G = {}
    for f in range(p.F):
        for b in range(p.B):
            for k in range(p.offsets[f * p.B + b], p.offsets[f * p.B + b + 1]):
                if keep[k]:
                    key = (f, int(p.indices[k]))
                    g = gout[b, p.d_offsets[f]:p.d_offsets[f + 1]]
                    G[key] = G[key] + g if key in G else g.copy()
    for (f, row), g in G.items():
        base = p.weights_offsets[f] + row * 8
        w[base:base + 8] += g * np.float32(-LR)
    np.testing.assert_array_equal(d_w.cpu().numpy(), w)


@pytest.fixture(scope="module")
def ops():
    torch_ops.load()
    return torch.ops.fbgemm


@pytest.mark.parametrize("optim", ["sgd", "adagrad", "adam"])
@pytest.mark.parametrize("unique", [False, True])
def test_torch_operators_read_rows_by_hash_indices_and_group_by_the_unique_inputs(ops, optim, unique):
    """hash_indices differs from indices (the raw ids a hybrid_torchrec caller keeps in `indices`); the operators must
    read and update the rows hash_indices names.  With the unique tensors the backward groups by unique_inverse."""
    p = TbeProblem(41, [(3000, 64), (20, 32), (50000, 16)], [0, 1, 1, 2], 200, max_len=12)
    raw = p.indices * 7919 + 123456789           # raw ids: useless as row numbers
    none = torch.empty(0, device=DEV)
    w, m1, m2 = p.weights.copy(), np.zeros_like(p.weights), np.zeros_like(p.weights)
    d_w, d_m1, d_m2 = dev(w), dev(m1), dev(m2)
    uid, uoff, uinv = p.unique_inputs()
    u3 = (dev(uid), dev(uoff), dev(uinv)) if unique else (none, none, none)
    tail = (dev(p.indices), *u3, none)           # hash_indices, unique_ids, unique_offsets, unique_inverse, offset_per_key
    head = lambda g: (g, d_w, none, none, none, dev(p.weights_offsets), dev(p.d_offsets), p.max_d,
                      dev(p.hash_size_cumsum), 0, dev(raw), dev(p.offsets), capi.POOL_SUM, none, 0, 0, False, 0, 0,
                      False, False)
    for it in range(1, 4):
        out = ops.split_embedding_codegen_forward_unweighted_cuda(
            d_w, none, none, none, dev(p.weights_offsets), dev(p.d_offsets), p.total_d, p.max_d, dev(raw),
            dev(p.offsets), capi.POOL_SUM, none, none, 0, False, dev(p.indices), none)
        np.testing.assert_array_equal(out.cpu().numpy(),
                                      oracle.tbe_forward(w, p.weights_offsets, p.d_offsets, p.total_d, p.indices,
                                                         p.offsets, p.F, p.B, capi.POOL_SUM))
        gout = p.rng.normal(0, 1e-2, (p.B, p.total_d)).astype(np.float32)
        if optim == "sgd":
            ops.split_embedding_backward_codegen_sgd_unweighted_exact_cuda(*head(dev(gout)), *tail, learning_rate=LR)
        elif optim == "adagrad":
            ops.split_embedding_backward_codegen_adagrad_unweighted_exact_cuda(
                *head(dev(gout)), d_m1, none, none, none, *tail, eps=EPS, learning_rate=LR)
        else:
            ops.split_embedding_backward_codegen_adam_unweighted_exact_cuda(
                *head(dev(gout)), d_m1, none, none, none, d_m2, none, none, none, *tail, eps=EPS, learning_rate=LR,
                beta1=B1, beta2=B2, iter=it)
        oracle.tbe_backward(CODES[optim], gout, w, p.weights_offsets, p.d_offsets, p.total_d, p.hash_size_cumsum,
                            p.indices, p.offsets, p.F, p.B, capi.POOL_SUM, m1, m2, LR, EPS, B1, B2, it)
        np.testing.assert_array_equal(d_w.cpu().numpy(), w)
        np.testing.assert_array_equal(d_m1.cpu().numpy(), m1)
        np.testing.assert_array_equal(d_m2.cpu().numpy(), m2)


@pytest.mark.parametrize("unique", [False, True])
def test_lookup_function_with_hash_indices_and_unique_inputs(ops, unique):
    """The autograd function the reference's HybridSplitTableBatchedEmbeddingBagsCodegen calls: forward by hash_indices,
    loss = sum(out^2 / 2) as in the reference test, backward fused into the tables."""
    p = TbeProblem(43, [(2000, 32), (700, 32)], [0, 0, 1], 64, max_len=0, fixed_len=[8, 16, 100])
    raw = p.indices + 10 ** 12
    none = torch.empty(0, device=DEV)
    w, m1 = p.weights.copy(), np.zeros_like(p.weights)
    m2 = np.zeros_like(w)
    d_w, d_m1 = dev(w), dev(m1)
    uid, uoff, uinv = p.unique_inputs()
    kw = dict(hash_indices=dev(p.indices))
    if unique:
        kw.update(unique_ids=dev(uid), unique_offsets=dev(uoff), unique_inverse=dev(uinv))
    for it in range(1, 4):
        placeholder = torch.zeros(1, device=DEV, requires_grad=True)
        out = ops.split_embedding_codegen_lookup_adagrad_function(
            placeholder, d_w, none, none, none, dev(p.weights_offsets), dev(p.d_offsets), p.total_d, p.max_d,
            dev(p.hash_size_cumsum), 0, dev(raw), dev(p.offsets), capi.POOL_MEAN, None, None, none, False, 0.0, False,
            d_m1, none, none, none, eps=EPS, learning_rate=LR, **kw)
        want = oracle.tbe_forward(w, p.weights_offsets, p.d_offsets, p.total_d, p.indices, p.offsets, p.F, p.B,
                                  capi.POOL_MEAN)
        np.testing.assert_array_equal(out.detach().cpu().numpy(), want)
        (out ** 2 / 2).sum().backward()
        oracle.tbe_backward(capi.OPT_ADAGRAD, want, w, p.weights_offsets, p.d_offsets, p.total_d, p.hash_size_cumsum,
                            p.indices, p.offsets, p.F, p.B, capi.POOL_MEAN, m1, m2, LR, EPS, B1, B2, it)
        np.testing.assert_array_equal(d_w.cpu().numpy(), w)
        np.testing.assert_array_equal(d_m1.cpu().numpy(), m1)


@pytest.mark.parametrize("unique", [False, True])
def test_rows_named_thousands_of_times_take_the_two_level_order(unique):
    """A row named more than 4096 times by the bags of a batch: chunk sums of 1024 positions, then the chunk sums in
    order, on the device as in the oracle (both forms of the backward)."""
    p = TbeProblem(61, [(30, 16), (5000, 16)], [0, 1], 400, max_len=0, fixed_len=[40, 3])   # 16000 positions on 30 rows
    p.indices[:9000] = 7                                                                    # one row 9000+ times
    p.per_feature[0][:9000] = 7
    bwd = host.SplitEmbeddingBackward(p.F, p.nnz)
    w, m1, m2 = p.weights.copy(), np.zeros_like(p.weights), np.zeros_like(p.weights)
    d_w, d_m1, d_m2 = dev(w), dev(m1), dev(m2)
    uid, uoff, uinv = p.unique_inputs()
    kw = dict(unique_ids=dev(uid), unique_offsets=dev(uoff), unique_inverse=dev(uinv)) if unique else {}
    for mode in (capi.POOL_SUM, capi.POOL_MEAN):
        gout = p.rng.normal(0, 1e-2, (p.B, p.total_d)).astype(np.float32)
        bwd(capi.OPT_ADAM, dev(gout), d_w, dev(p.weights_offsets), dev(p.d_offsets), p.total_d, p.max_d,
            dev(p.hash_size_cumsum), dev(p.indices), dev(p.offsets), mode, d_m1, d_m2, LR, EPS, B1, B2, 2, **kw)
        oracle.tbe_backward(capi.OPT_ADAM, gout, w, p.weights_offsets, p.d_offsets, p.total_d, p.hash_size_cumsum,
                            p.indices, p.offsets, p.F, p.B, mode, m1, m2, LR, EPS, B1, B2, 2)
        np.testing.assert_array_equal(d_w.cpu().numpy(), w)
        np.testing.assert_array_equal(d_m1.cpu().numpy(), m1)
        np.testing.assert_array_equal(d_m2.cpu().numpy(), m2)
