"""GPU parity at the size of configuration 1: one fp32 table of 1,000,000 rows x dim 16 initialised N(0, 0.01) from
seed 0, Adagrad accumulators 0.1, 100 steps of batch 4096 one-hot int64 keys uniform in [0, 1e6), gradients N(0, 1e-3),
learning rate 0.01: dedup + key -> slot + gather + segment-reduce + Adagrad.  Every step's distinct keys, inverse index,
counts, slots and gathered rows, and the whole table and its accumulators after the last step, equal the CPU oracle's
bit for bit.  The Adagrad form is the by-address one (adagrad_by_addr.py:101-125); the stock-TensorFlow static form
differs only in where epsilon sits and is pinned to torch.optim.Adagrad in tests/test_oracle_ops.py."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROWS, DIM, BATCH, STEPS = 1_000_000, 16, 4096, 100
LR, ACC0, EPS = 0.01, 0.1, 1e-7


def test_hundred_steps_of_config1_match_the_oracle():
    rng = np.random.default_rng(0)
    hw = rng.normal(0, 0.01, (ROWS, DIM)).astype(np.float32)
    hs = np.full((ROWS, DIM), ACC0, np.float32)
    none = np.zeros((1, DIM), np.float32)
    w = torch.from_numpy(hw).to(DEV)
    acc = torch.from_numpy(hs).to(DEV)
    rows_h = host.Rows(DIM, [w], [acc], None)
    uq = host.Unique(BATCH, 1)
    tg = host.EmbeddingTables([ROWS], BATCH)
    tab = oracle.Table(ROWS)
    off = torch.tensor([0, BATCH], dtype=torch.int64, device=DEV)
    for step in range(STEPS):
        keys = rng.integers(0, ROWS, BATCH).astype(np.int64)
        grad = rng.normal(0, 1e-3, (BATCH, DIM)).astype(np.float32)
        uq.run(torch.from_numpy(keys).to(DEV), off)
        uk, uo, inv, cnt = uq.fetch()
        slots = uk.clone()
        tg.key2offset(slots, uo, capi.CHANNEL_TRAIN)
        out = host.gather_unique(rows_h, uq, slots)
        host.sparse_apply(rows_h, uq, slots, torch.from_numpy(grad).to(DEV), capi.OPT_ADAGRAD, LR, 0.9, 0.999, EPS, 0.0)
        split, _, restore, counts = oracle.hash_split(keys, 1)
        so, rc = tab.key2offset(split, 0)
        assert rc == 0
        np.testing.assert_array_equal(uk.cpu().numpy(), split, err_msg=f"distinct keys, step {step}")
        np.testing.assert_array_equal(inv.cpu().numpy(), restore, err_msg=f"inverse, step {step}")
        np.testing.assert_array_equal(cnt.cpu().numpy().astype(np.uint32), counts, err_msg=f"counts, step {step}")
        np.testing.assert_array_equal(slots.cpu().numpy(), so, err_msg=f"slots, step {step}")
        np.testing.assert_array_equal(out.cpu().numpy(), oracle.gather_rows(hw, DIM, so[restore], DIM),
                                      err_msg=f"gathered rows, step {step}")
        g = oracle.segment_sum(grad, restore, split.size)
        oracle.byaddr_apply(capi.OPT_ADAGRAD, g, so, hw, hs, none, DIM, LR, 0.9, 0.999, EPS, 0.0, delta_form=False)
    np.testing.assert_array_equal(w.cpu().numpy(), hw)
    np.testing.assert_array_equal(acc.cpu().numpy(), hs)
    mo, live, _ = tg.stats()
    assert mo[0] == live[0] == tab.size
    # rows no key ever took are as initialised
    assert np.all(hs[tab.size:] == np.float32(ACC0))
