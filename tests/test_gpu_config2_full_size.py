"""GPU parity at the full size of the DLRM-style configuration: 26 fp32 tables of dim 128 with 60 M rows in
total plus Adam moments (92 GB in HBM), batch 65536 with one key per field, Zipf(1.05) keys hashed to 64-bit ids
that the device hash table resolves; three steps of dedup + key -> slot + gather + segment-reduce + Adam.

Slots are handed out in first-seen order, so after three steps every touched row lies in the first 3 x 65536 rows of
its table: the CPU oracle works on that prefix of the same initial weights, and every step's distinct keys, inverse
index, slots and gathered rows and the final weights and moments of the prefix are compared exactly.
"""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host, synth

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
T, DIM, BATCH, STEPS = 26, 128, 65536, 3


def test_three_steps_of_the_full_configuration_match_the_oracle():
    rows = [int(r) for r in synth.dlrm_table_rows(T, 60_000_000)]
    rng = np.random.default_rng(22)
    samplers = [synth.ZipfSampler(1.05, r) for r in rows]
    n = T * BATCH
    offs = np.arange(T + 1, dtype=np.int64) * BATCH
    d_off = torch.from_numpy(offs).to(DEV)
    w = [torch.randn((r, DIM), device=DEV) * 0.01 for r in rows]
    m = [torch.zeros((r, DIM), device=DEV) for r in rows]
    v = [torch.zeros((r, DIM), device=DEV) for r in rows]
    prefix = [min(r, STEPS * BATCH) for r in rows]
    hw = [w[t][:prefix[t]].cpu().numpy() for t in range(T)]
    hm = [np.zeros((prefix[t], DIM), np.float32) for t in range(T)]
    hv = [np.zeros((prefix[t], DIM), np.float32) for t in range(T)]
    rows_h = host.Rows(DIM, w, m, v)
    uq = host.Unique(n, T, early_counts=False, max_table_keys=BATCH)   # as the benchmark runs it
    tg = host.EmbeddingTables(rows, n)
    orc_tab = [oracle.Table(r) for r in rows]
    lr, b1, b2, eps = 1e-3, 0.9, 0.999, 1e-8
    for step in range(1, STEPS + 1):
        keys = np.concatenate([synth.ranks_to_keys(samplers[t].ranks(rng, BATCH), t) for t in range(T)]).astype(np.int64)
        grad = rng.normal(0, 1e-3, (n, DIM)).astype(np.float32)
        dk = torch.from_numpy(keys).to(DEV)
        dg = torch.from_numpy(grad).to(DEV)
        uq.run(dk, d_off)
        uk, uo, inv, cnt = uq.fetch()
        slots = uk.clone()
        tg.key2offset(slots, uo, capi.CHANNEL_TRAIN)
        out = host.gather_unique(rows_h, uq, slots)
        lr_t = float(lr * np.sqrt(1 - b2 ** step) / (1 - b1 ** step))
        host.sparse_apply(rows_h, uq, slots, dg, capi.OPT_ADAM, lr_t, b1, b2, eps, 0.0)
        torch.cuda.synchronize()
        uk_h, uo_h, inv_h = uk.cpu().numpy(), uo.cpu().numpy(), inv.cpu().numpy()
        slots_h = slots.cpu().numpy()
        for t in range(T):
            kt = keys[offs[t]:offs[t + 1]]
            split, _, restore, _ = oracle.hash_split(kt, 1)
            np.testing.assert_array_equal(uk_h[uo_h[t]:uo_h[t + 1]], split, err_msg=f"distinct keys, table {t}")
            np.testing.assert_array_equal(inv_h[offs[t]:offs[t + 1]], restore, err_msg=f"inverse, table {t}")
            so, rc = orc_tab[t].key2offset(split, 0)
            assert rc == 0
            np.testing.assert_array_equal(slots_h[uo_h[t]:uo_h[t + 1]], so, err_msg=f"slots, table {t}")
            assert so.max() < prefix[t]
            want_out = oracle.gather_rows(hw[t], DIM, so[restore], DIM)
            np.testing.assert_array_equal(out[offs[t]:offs[t + 1]].cpu().numpy(), want_out,
                                          err_msg=f"gathered rows, step {step}, table {t}")
            g = oracle.segment_sum(grad[offs[t]:offs[t + 1]], restore, split.size)
            oracle.byaddr_apply(capi.OPT_ADAM, g, so, hw[t], hm[t], hv[t], DIM, lr_t, b1, b2, eps, 0.0,
                                delta_form=False)
    for t in range(T):
        p = prefix[t]
        np.testing.assert_array_equal(w[t][:p].cpu().numpy(), hw[t], err_msg=f"weights, table {t}")
        np.testing.assert_array_equal(m[t][:p].cpu().numpy(), hm[t], err_msg=f"first moments, table {t}")
        np.testing.assert_array_equal(v[t][:p].cpu().numpy(), hv[t], err_msg=f"second moments, table {t}")
        if rows[t] > p:   # rows past the prefix were never touched
            assert float(m[t][p:].abs().max()) == 0.0
