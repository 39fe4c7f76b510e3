"""Pins the CPU oracle's floating-point half against closed forms and third-party routines.

  lookup / update by address : numpy gather and `+=` as in the reference's golden generators
      cust_op/test/aclnn_cust_op_by_addr_test/tf/scripts/gen_lookup_data.py:22-38, gen_update_data.py:22-38
  lazy_adam : the numpy golden of cust_op/test/aclnn_lazy_adam_test/tf/scripts/gen_data.py:90-127, and
      torch.optim.Adam (eps -> 0, where the two epsilon placements coincide)
  sgd / by-address SGD, Adagrad : torch.optim.SGD(weight_decay), torch.optim.Adagrad(eps=0)
  tbe_forward : torch.nn.functional.embedding_bag (sum / mean)
  tbe_backward : torch.optim.{SGD, Adagrad, SparseAdam} on sparse EmbeddingBag gradients over several steps,
      the scheme of cust_op/test/split_embedding_codegen_lookup_adagrad_function_test/torch/
      test_split_embedding_codegen_lookup_function.py:149-172
Tolerance where an independent implementation orders its fp32 operations differently: 1e-6 relative
(+1e-9 absolute); identical-order checks are exact.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle

RTOL, ATOL = 1e-6, 1e-9


def addr_of(arr, rows):
    """Host addresses of rows of a C-contiguous 2-D array."""
    return arr.ctypes.data + np.asarray(rows, dtype=np.int64) * arr.strides[0]


def test_lookup_by_addr_closed_form():
    rng = np.random.default_rng(0)
    emb_size, addr_num, dim = 100000, 21632, 8
    offset = rng.integers(0, emb_size, addr_num)
    emb = (np.arange(emb_size * dim) * 0.01).astype(np.float32).reshape(emb_size, dim)
    addr = addr_of(emb, offset)
    addr[::97] = 0
    got = oracle.lookup_by_addr(addr, dim)
    want = emb[offset].copy()
    want[::97] = 0
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("update_type", [0, 1])
def test_update_by_addr_closed_form(update_type):
    rng = np.random.default_rng(1)
    emb_size, addr_num, dim = 5000, 21632, 8  # duplicates on purpose
    offset = rng.integers(0, emb_size, addr_num)
    emb = (np.arange(emb_size * dim) * 0.01).astype(np.float32).reshape(emb_size, dim)
    grad = rng.uniform(1, 10, (addr_num, dim)).astype(np.float32)
    want = emb.copy()
    for i in range(addr_num):  # the reference generator's sequential `+=`
        if update_type == 0:
            want[offset[i]] += grad[i]
        else:
            want[offset[i]] = grad[i]
    oracle.update_by_addr(addr_of(emb, offset), grad, update_type)
    np.testing.assert_array_equal(emb, want)


def test_lazy_adam_matches_reference_numpy_golden():
    rng = np.random.default_rng(2)
    rows, n, dim = 20000, 5641, 32
    var = rng.uniform(1, 2, (rows, dim)).astype(np.float32)
    m = rng.uniform(1, 2, (rows, dim)).astype(np.float32)
    v = rng.uniform(1, 2, (rows, dim)).astype(np.float32)
    idx = rng.permutation(rows)[:n].astype(np.int32)
    idx[::50] = -1
    grad = rng.uniform(1, 2, (n, dim)).astype(np.float32)
    beta1, beta2, lr, eps = np.float32(0.9), np.float32(0.999), np.float32(0.001), np.float32(1e-7)
    ok = idx >= 0
    um = beta1 * m[idx[ok]] + (1 - beta1) * grad[ok]
    uv = beta2 * v[idx[ok]] + (1 - beta2) * np.square(grad[ok])
    wm, wv, wvar = m.copy(), v.copy(), var.copy()
    wm[idx[ok]] = um
    wv[idx[ok]] = uv
    wvar[idx[ok]] = var[idx[ok]] + np.divide(-lr * um, np.sqrt(np.abs(uv)) + eps)
    oracle.lazy_adam(grad, idx, m, v, var, float(lr), float(beta1), float(beta2), float(eps))
    np.testing.assert_allclose(m, wm, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(v, wv, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(var, wvar, rtol=RTOL, atol=ATOL)


# beta values exactly representable in fp32: the reference forms (1 - beta) in fp32 (lazy_adam.cpp:170,175,
# gen_data.py:96-99) while torch forms it in double, which differ by 1e-5 relative for 0.999.
B1, B2 = 0.875, 1.0 - 2.0 ** -9


def test_lazy_adam_three_steps_match_torch_adam():
    rng = np.random.default_rng(3)
    rows, dim = 64, 16
    w0 = rng.normal(0, 0.01, (rows, dim)).astype(np.float32)
    p = torch.nn.Parameter(torch.from_numpy(w0.copy()))
    opt = torch.optim.Adam([p], lr=1e-3, betas=(B1, B2), eps=1e-30)
    m = np.zeros_like(w0)
    v = np.zeros_like(w0)
    w = w0.copy()
    idx = np.arange(rows, dtype=np.int32)
    for t in range(1, 4):
        g = rng.normal(0, 1e-3, (rows, dim)).astype(np.float32)
        p.grad = torch.from_numpy(g.copy())
        opt.step()
        lr_t = 1e-3 * np.sqrt(1 - B2 ** t) / (1 - B1 ** t)
        oracle.lazy_adam(g, idx, m, v, w, float(lr_t), B1, B2, 0.0)
    np.testing.assert_allclose(w, p.detach().numpy(), rtol=RTOL, atol=1e-9)


@pytest.mark.parametrize("wd", [0.0, 0.01])
def test_sgd_matches_torch(wd):
    rng = np.random.default_rng(4)
    rows, dim = 300, 24
    w0 = rng.normal(0, 1, (rows, dim)).astype(np.float32)
    idx = rng.permutation(rows)[:100].astype(np.int32)
    g = rng.normal(0, 1, (100, dim)).astype(np.float32)
    p = torch.nn.Parameter(torch.from_numpy(w0.copy()))
    dense = torch.zeros(rows, dim)
    dense[torch.from_numpy(idx.astype(np.int64))] = torch.from_numpy(g)
    # torch applies weight decay to every row; restrict the comparison to touched rows
    p.grad = dense
    torch.optim.SGD([p], lr=0.05, weight_decay=wd).step()
    w = w0.copy()
    oracle.sgd(g, idx, w, 0.05, wd)
    np.testing.assert_allclose(w[idx], p.detach().numpy()[idx], rtol=RTOL, atol=1e-7)
    untouched = np.setdiff1d(np.arange(rows), idx)
    np.testing.assert_array_equal(w[untouched], w0[untouched])
    # the by-address SGD algebra is the same update
    w2 = w0.copy()
    oracle.byaddr_apply(0, g, idx.astype(np.int64), w2, None, None, dim, 0.05, weight_decay=wd)
    np.testing.assert_allclose(w2, w, rtol=RTOL, atol=1e-7)


def test_byaddr_adagrad_matches_torch_adagrad():
    rng = np.random.default_rng(5)
    rows, dim = 128, 16
    w0 = rng.normal(0, 0.01, (rows, dim)).astype(np.float32)
    p = torch.nn.Parameter(torch.from_numpy(w0.copy()))
    opt = torch.optim.Adagrad([p], lr=0.01, initial_accumulator_value=0.1, eps=0.0)
    # extended rows [w | acc]
    ext = np.concatenate([w0, np.full_like(w0, 0.1)], axis=1).copy()
    slots = np.arange(rows, dtype=np.int64)
    for _ in range(3):
        g = rng.normal(0, 1e-3, (rows, dim)).astype(np.float32)
        p.grad = torch.from_numpy(g.copy())
        opt.step()
        w_view = ext[:, :dim]
        s_view = ext[:, dim:]
        oracle.lib().orc_byaddr_apply(1, g.ctypes.data_as(ctypes.c_void_p), slots.ctypes.data_as(ctypes.c_void_p),
                                      rows, dim, ctypes.c_void_p(w_view.ctypes.data),
                                      ctypes.c_void_p(s_view.ctypes.data), None, 2 * dim, 0.01, 0.9, 0.999, 0.0, 0.0,
                                      1)
    np.testing.assert_allclose(ext[:, :dim], p.detach().numpy(), rtol=RTOL, atol=1e-9)


def test_byaddr_adam_delta_and_direct_forms_agree_and_match_lazy_adam():
    rng = np.random.default_rng(6)
    rows, dim = 200, 8
    ext = rng.normal(0, 0.01, (rows, 3 * dim)).astype(np.float32)
    ext[:, 2 * dim:] = np.abs(ext[:, 2 * dim:])
    g = rng.normal(0, 1e-3, (rows, dim)).astype(np.float32)
    slots = rng.permutation(rows).astype(np.int64)
    slots[::9] = -1

    def run(delta):
        e = ext.copy()
        L = oracle.lib()
        vp = ctypes.c_void_p
        L.orc_byaddr_apply(2, g.ctypes.data_as(vp), slots.ctypes.data_as(vp), rows, dim, vp(e.ctypes.data),
                           vp(e.ctypes.data + 4 * dim), vp(e.ctypes.data + 8 * dim), 3 * dim, 1e-3, 0.9, 0.999, 1e-8,
                           0.0, delta)
        return e

    a, b = run(1), run(0)
    np.testing.assert_allclose(a, b, rtol=RTOL, atol=1e-12)
    # direct form == LazyAdam on split tables
    ok = slots >= 0
    w = np.ascontiguousarray(ext[:, :dim])
    m = np.ascontiguousarray(ext[:, dim:2 * dim])
    v = np.ascontiguousarray(ext[:, 2 * dim:])
    oracle.lazy_adam(g, np.where(ok, slots, -1).astype(np.int32), m, v, w, 1e-3, 0.9, 0.999, 1e-8)
    np.testing.assert_array_equal(b[:, :dim], w)
    np.testing.assert_array_equal(b[:, dim:2 * dim], m)
    np.testing.assert_array_equal(b[:, 2 * dim:], v)


def test_segment_sum_is_sequential_and_matches_float64_within_tolerance():
    rng = np.random.default_rng(7)
    n, dim, u = 4000, 8, 37
    g = rng.normal(0, 1e-3, (n, dim)).astype(np.float32)
    seg = rng.integers(-1, u, n).astype(np.int32)
    got = oracle.segment_sum(g, seg, u)
    want = np.zeros((u, dim), np.float32)
    for i in range(n):
        if seg[i] >= 0:
            want[seg[i]] += g[i]
    np.testing.assert_array_equal(got, want)
    ref64 = np.zeros((u, dim))
    np.add.at(ref64, seg[seg >= 0], g[seg >= 0].astype(np.float64))
    scale = np.zeros((u, dim))
    np.add.at(scale, seg[seg >= 0], np.abs(g[seg >= 0]).astype(np.float64))
    assert (np.abs(got - ref64) <= 1e-6 * scale + 1e-12).all()


def make_tbe_problem(seed, T, B, dims, rows, max_len, bf16=False):
    rng = np.random.default_rng(seed)
    d_offsets = np.concatenate([[0], np.cumsum(dims)]).astype(np.int32)
    w_sizes = [r * d for r, d in zip(rows, dims)]
    weights_offsets = np.concatenate([[0], np.cumsum(w_sizes)])[:-1].astype(np.int64)
    hash_size_cumsum = np.concatenate([[0], np.cumsum(rows)]).astype(np.int64)
    lengths = rng.integers(0, max_len + 1, T * B)
    offsets = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int64)
    indices = np.concatenate([rng.integers(0, rows[t], int(lengths[t * B:(t + 1) * B].sum())) for t in range(T)]
                             + [np.zeros(0, np.int64)]).astype(np.int64)
    weights = rng.normal(0, 0.1, int(sum(w_sizes))).astype(np.float32)
    return d_offsets, weights_offsets, hash_size_cumsum, offsets, indices, weights


@pytest.mark.parametrize("mode", [0, 1])
def test_tbe_forward_matches_torch_embedding_bag(mode):
    T, B, dims, rows = 3, 17, [8, 16, 8], [50, 30, 70]
    d_off, w_off, _, offsets, indices, weights = make_tbe_problem(8, T, B, dims, rows, 6)
    out = oracle.tbe_forward(weights, w_off, d_off, int(d_off[-1]), indices, offsets, T, B, mode)
    for t in range(T):
        W = torch.from_numpy(weights[w_off[t]:w_off[t] + rows[t] * dims[t]].reshape(rows[t], dims[t]))
        o = torch.from_numpy(offsets[t * B:(t + 1) * B + 1] - offsets[t * B])
        idx = torch.from_numpy(indices[offsets[t * B]:offsets[(t + 1) * B]])
        ref = torch.nn.functional.embedding_bag(idx, W, o, mode="sum" if mode == 0 else "mean",
                                                include_last_offset=True)
        np.testing.assert_allclose(out[:, d_off[t]:d_off[t + 1]], ref.numpy(), rtol=2e-6, atol=1e-7)


def test_tbe_forward_nobag_is_row_copy():
    T, B, dims, rows = 2, 9, [8, 8], [40, 60]
    d_off, w_off, _, offsets, indices, weights = make_tbe_problem(9, T, B, dims, rows, 4)
    out = oracle.tbe_forward(weights, w_off, d_off, 16, indices, offsets, T, B, 2)
    k = 0
    for t in range(T):
        W = weights[w_off[t]:w_off[t] + rows[t] * 8].reshape(rows[t], 8)
        for j in indices[offsets[t * B]:offsets[(t + 1) * B]]:
            np.testing.assert_array_equal(out[k], W[j])
            k += 1
    assert k == indices.size


@pytest.mark.parametrize("optim", [0, 1, 2])
@pytest.mark.parametrize("mode", [0, 1])
def test_tbe_backward_matches_torch_optim_over_steps(optim, mode):
    T, B, dims, rows = 2, 13, [8, 16], [40, 25]
    d_off, w_off, hcs, offsets, indices, weights = make_tbe_problem(10 + optim, T, B, dims, rows, 5)
    total_d = int(d_off[-1])
    bags = []
    params = []
    for t in range(T):
        W = weights[w_off[t]:w_off[t] + rows[t] * dims[t]].reshape(rows[t], dims[t]).copy()
        bag = torch.nn.EmbeddingBag(rows[t], dims[t], mode="sum" if mode == 0 else "mean", sparse=True,
                                    include_last_offset=True)
        bag.weight.data.copy_(torch.from_numpy(W))
        bags.append(bag)
        params.append(bag.weight)
    lr, eps = 0.05, 1e-8
    if optim == 0:
        opt = torch.optim.SGD(params, lr=lr)
    elif optim == 1:
        opt = torch.optim.Adagrad(params, lr=lr, eps=eps)
    else:
        opt = torch.optim.SparseAdam(params, lr=lr, betas=(B1, B2), eps=eps)
    w = weights.copy()
    m1 = np.zeros_like(w)
    m2 = np.zeros_like(w)
    rng = np.random.default_rng(99)
    for it in range(1, 5):
        gout = rng.normal(0, 1, (B, total_d)).astype(np.float32)
        opt.zero_grad()
        outs = []
        for t in range(T):
            o = torch.from_numpy(offsets[t * B:(t + 1) * B + 1] - offsets[t * B])
            idx = torch.from_numpy(indices[offsets[t * B]:offsets[(t + 1) * B]])
            outs.append(bags[t](idx, o))
        out = torch.cat(outs, dim=1)
        (out * torch.from_numpy(gout)).sum().backward()
        opt.step()
        oracle.tbe_backward(optim, gout, w, w_off, d_off, total_d, hcs, indices, offsets, T, B, mode, m1, m2, lr, eps,
                            B1, B2, it)
    for t in range(T):
        got = w[w_off[t]:w_off[t] + rows[t] * dims[t]].reshape(rows[t], dims[t])
        np.testing.assert_allclose(got, params[t].detach().numpy(), rtol=2e-6, atol=2e-7)


def test_tbe_bf16_weights_accumulate_in_fp32():
    T, B, dims, rows = 1, 5, [8], [20]
    d_off, w_off, _, offsets, indices, weights = make_tbe_problem(20, T, B, dims, rows, 4)
    wb = torch.from_numpy(weights).to(torch.bfloat16)
    out = oracle.tbe_forward(wb.view(torch.int16).numpy(), w_off, d_off, 8, indices, offsets, T, B, 0, bf16=True)
    ref = oracle.tbe_forward(wb.float().numpy(), w_off, d_off, 8, indices, offsets, T, B, 0)
    np.testing.assert_array_equal(out, ref)
