"""GPU: the pooled multi-hot configuration at its full size (26 bf16 tables of 2 M x 64, batch 16384, bag lengths
U[1,50], Zipf(1.1) indices, about 10.9 M indices per step) checked through properties that need no CPU run of the
same size:

* forward: weights are a closed-form function of (table, row, column) whose values and bag sums are exact in
  bf16 / fp32, so every pooled output must equal the sum of that function over the bag's indices;
* backward: with a gradient of ones the summed gradient of a row is its multiplicity, so SGD leaves
  bf16(-lr * count) in every touched row and Adam leaves count * (1 - beta1) and count^2 * (1 - beta2) in the
  moments; untouched rows keep their contents.
"""
import numpy as np
import pytest
import torch

from recsdk_amd import capi, host
from recsdk_amd.synth import zipf_ranks

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
T, D, B, ROWS = 26, 64, 16384, 2_000_000


def closed_form(t, rows, c):
    """Multiples of 1/64 in [-0.5, 0.5): exact in bf16, and sums of 50 of them are exact in fp32."""
    return (((rows * 31 + c * 7 + t * 3) % 64) - 32).astype(np.float32) / np.float32(64)


@pytest.fixture(scope="module")
def batch():
    rng = np.random.default_rng(33)
    lengths = rng.integers(1, 51, T * B)
    offsets = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int64)
    per_table = [int(lengths[t * B:(t + 1) * B].sum()) for t in range(T)]
    indices = np.concatenate([zipf_ranks(rng, 1.1, ROWS, n) for n in per_table]).astype(np.int64)
    table_of = np.repeat(np.arange(T), per_table)
    return offsets, indices, table_of


def device_args(offsets, indices):
    woff = torch.arange(T, device=DEV, dtype=torch.int64) * ROWS * D
    doff = torch.arange(T + 1, device=DEV, dtype=torch.int32) * D
    cumsum = torch.arange(T + 1, device=DEV, dtype=torch.int64) * ROWS
    return woff, doff, cumsum, torch.from_numpy(indices).to(DEV), torch.from_numpy(offsets).to(DEV)


def test_forward_sums_a_closed_form_table(batch):
    offsets, indices, table_of = batch
    w = torch.empty(T * ROWS * D, dtype=torch.bfloat16, device=DEV)
    r = torch.arange(ROWS, device=DEV, dtype=torch.int64).view(ROWS, 1)
    c = torch.arange(D, device=DEV, dtype=torch.int64).view(1, D)
    for t in range(T):
        vals = (((r * 31 + c * 7 + t * 3) % 64) - 32).to(torch.float32) / 64
        w[t * ROWS * D:(t + 1) * ROWS * D] = vals.to(torch.bfloat16).view(-1)
    woff, doff, _, d_idx, d_off = device_args(offsets, indices)
    out = host.split_embedding_codegen_forward_unweighted(w, woff, doff, T * D, D, d_idx, d_off, capi.POOL_SUM)
    torch.cuda.synchronize()
    assert out.shape == (B, T * D)
    for col in (0, 21, 63):
        vals = closed_form(table_of, indices, col)
        want = np.add.reduceat(vals, offsets[:-1]).reshape(T, B).T          # [B, T]
        got = out[:, col::D].cpu().numpy()
        np.testing.assert_array_equal(got, want, err_msg=f"column {col}")


def test_backward_leaves_each_row_its_multiplicity(batch):
    offsets, indices, table_of = batch
    count = np.bincount(table_of * ROWS + indices, minlength=T * ROWS)
    woff, doff, cumsum, d_idx, d_off = device_args(offsets, indices)
    gout = torch.ones((B, T * D), device=DEV)
    bwd = host.SplitEmbeddingBackward(T, int(indices.size))
    # SGD on bf16 rows of zeros
    w = torch.zeros(T * ROWS * D, dtype=torch.bfloat16, device=DEV)
    lr = 2.0 ** -10
    bwd(capi.OPT_SGD, gout, w, woff, doff, T * D, D, cumsum, d_idx, d_off, capi.POOL_SUM, learning_rate=lr)
    torch.cuda.synchronize()
    want = (torch.from_numpy(count.astype(np.float32)) * np.float32(-lr)).to(torch.bfloat16).float().numpy()
    wv = w.view(T * ROWS, D)
    for col in (0, 63):
        np.testing.assert_array_equal(wv[:, col].float().cpu().numpy(), want, err_msg=f"SGD, column {col}")
    # Adam: the moments of every row, from zero state
    w.zero_()
    m1 = torch.zeros(T * ROWS * D, device=DEV)
    m2 = torch.zeros(T * ROWS * D, device=DEV)
    b1, b2 = 0.9, 0.999
    bwd(capi.OPT_ADAM, gout, w, woff, doff, T * D, D, cumsum, d_idx, d_off, capi.POOL_SUM, m1, m2,
        learning_rate=1e-3, beta1=b1, beta2=b2, iter=1)
    torch.cuda.synchronize()
    g = count.astype(np.float32)
    want1 = g * (np.float32(1) - np.float32(b1))
    want2 = (g * g) * (np.float32(1) - np.float32(b2))
    for col in (0, 40):
        np.testing.assert_array_equal(m1.view(T * ROWS, D)[:, col].cpu().numpy(), want1, err_msg=f"m, column {col}")
        np.testing.assert_array_equal(m2.view(T * ROWS, D)[:, col].cpu().numpy(), want2, err_msg=f"v, column {col}")
    touched = torch.from_numpy(count > 0).to(DEV)
    wz = (w.view(T * ROWS, D)[:, 5] != 0)
    assert torch.equal(wz, touched)      # every touched row moved, no other row did
