"""Pins the oracle's pooled-lookup backward in the cases the reference's operator test covers beyond one feature per
table (test_split_embedding_codegen_lookup_function.py:320-350): features that share a table (feature_map [0,0,1] and
[0,1,1]), no pooling, and the unique variant.  The check is the reference test's own golden model: torch.nn.Embedding /
EmbeddingBag per table, loss = sum(out^2 / 2), torch.optim.{SGD, Adagrad, SparseAdam} over several steps."""
import numpy as np
import pytest
import torch

import oracle
from tests.tbe_cases import TbeProblem

B1, B2 = 0.9, 0.999
LR, EPS = 0.05, 1e-8


def torch_model(p, mode, optim):
    mods = []
    for t, (rows, dim) in enumerate(p.tables):
        if mode == 2:
            m = torch.nn.Embedding(rows, dim, sparse=optim != 0)
        else:
            m = torch.nn.EmbeddingBag(rows, dim, mode="sum" if mode == 0 else "mean", sparse=optim != 0,
                                      include_last_offset=True)
        m.weight.data.copy_(torch.from_numpy(p.table_view(p.weights, t)))
        mods.append(m)
    params = [m.weight for m in mods]
    if optim == 0:
        opt = torch.optim.SGD(params, lr=LR)
    elif optim == 1:
        opt = torch.optim.Adagrad(params, lr=LR, eps=EPS)
    else:
        opt = torch.optim.SparseAdam(params, lr=LR, betas=(B1, B2), eps=EPS)
    return mods, opt


def torch_forward(p, mods, mode):
    outs = []
    for f, t in enumerate(p.feature_map):
        idx = torch.from_numpy(p.per_feature[f])
        if mode == 2:
            outs.append(mods[t](idx))
        else:
            o = torch.from_numpy(p.offsets[f * p.B:(f + 1) * p.B + 1] - p.offsets[f * p.B])
            outs.append(mods[t](idx, o))
    return torch.cat(outs, dim=0 if mode == 2 else 1)


CASES = [([(40, 8), (25, 8)], [0, 0, 1]), ([(40, 8), (25, 8)], [0, 1, 1]), ([(30, 16)], [0]),
         ([(20, 8), (50, 8), (7, 8)], [0, 1, 2])]


@pytest.mark.parametrize("unique", [False, True])
@pytest.mark.parametrize("optim", [0, 1, 2])
@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("tables,feature_map", CASES)
def test_backward_matches_the_reference_tests_torch_model(tables, feature_map, mode, optim, unique):
    p = TbeProblem(31 + optim, tables, feature_map, batch=9, max_len=5)
    mods, opt = torch_model(p, mode, optim)
    w = p.weights.copy()
    m1 = np.zeros_like(w)
    m2 = np.zeros_like(w)
    uid, uoff, uinv = p.unique_inputs()
    for it in range(1, 5):
        opt.zero_grad()
        out = torch_forward(p, mods, mode)
        got = oracle.tbe_forward(w, p.weights_offsets, p.d_offsets, p.total_d if mode != 2 else p.max_d * p.F,
                                 p.indices, p.offsets, p.F, p.B, mode)
        np.testing.assert_allclose(got, out.detach().numpy(), rtol=2e-6, atol=1e-7)
        (out ** 2 / 2).sum().backward()
        opt.step()
        gout = got   # d loss / d out = out
        total_d = p.total_d if mode != 2 else p.max_d * p.F
        if unique:
            oracle.tbe_backward_unique(optim, gout, w, p.weights_offsets, p.d_offsets, total_d, p.offsets, p.F, p.B,
                                       mode, uid, uoff, uinv, m1, m2, LR, EPS, B1, B2, it)
        else:
            oracle.tbe_backward(optim, gout, w, p.weights_offsets, p.d_offsets, total_d, p.hash_size_cumsum,
                                p.indices, p.offsets, p.F, p.B, mode, m1, m2, LR, EPS, B1, B2, it)
    for t in range(len(tables)):
        np.testing.assert_allclose(p.table_view(w, t), mods[t].weight.detach().numpy(), rtol=3e-5, atol=3e-6)


def test_unique_variant_equals_the_plain_one_up_to_summation_order():
    """Both group the same gradient rows per table row; the plain form adds them in position order, the unique form
    too (one accumulator per distinct row), so the results are equal bit for bit."""
    p = TbeProblem(5, [(60, 8), (35, 16)], [0, 0, 1], batch=21, max_len=7)
    uid, uoff, uinv = p.unique_inputs()
    for mode in (0, 1):
        for optim in (0, 1, 2):
            gout = p.rng.normal(0, 1, p.grad_shape(mode)).astype(np.float32)
            res = []
            for unique in (False, True):
                w, m1, m2 = p.weights.copy(), np.zeros_like(p.weights), np.zeros_like(p.weights)
                if unique:
                    oracle.tbe_backward_unique(optim, gout, w, p.weights_offsets, p.d_offsets, p.total_d, p.offsets,
                                               p.F, p.B, mode, uid, uoff, uinv, m1, m2, LR, EPS, B1, B2, 3)
                else:
                    oracle.tbe_backward(optim, gout, w, p.weights_offsets, p.d_offsets, p.total_d,
                                        p.hash_size_cumsum, p.indices, p.offsets, p.F, p.B, mode, m1, m2, LR, EPS, B1,
                                        B2, 3)
                res.append((w, m1, m2))
            for a, b in zip(*res):
                np.testing.assert_array_equal(a, b)
