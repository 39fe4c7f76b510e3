"""GPU parity at the full size of the dynamic-expansion configuration: 100 steps of batch 131072 on a table of
200 M slots, keys 70 % Zipf(1.2) over a hot set of 10 M and 30 % fresh ids, admission at count >= 2, eviction of
keys idle for more than 20 steps every step.  Every step's distinct keys, counts, admission mask, slots and evicted
keys, and the final table state, are compared exactly with the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host
from recsdk_amd.synth import splitmix64, zipf_ranks

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_admit_slot_evict_sequence_of_100_steps_matches_oracle():
    slots, batch, hot, steps = 200_000_000, 131072, 10_000_000, 100
    rng = np.random.default_rng(4)
    uq = host.Unique(batch, 1)
    tg = host.EmbeddingTables([slots], batch)
    f = host.FeatureAdmitAndEvict([8_000_000], [2], [20], max_keys=batch)
    orc_f = oracle.Faae(2, 20)
    orc_t = oracle.Table(slots)
    off = torch.tensor([0, batch], dtype=torch.int64, device=DEV)
    fresh = 1 << 40
    evicted_total = 0
    admitted_total = 0
    for step in range(steps):
        is_hot = rng.random(batch) < 0.7
        keys = np.where(is_hot, splitmix64(zipf_ranks(rng, 1.2, hot, batch).astype(np.uint64)),
                        splitmix64(np.arange(fresh, fresh + batch, dtype=np.uint64))).astype(np.int64)
        fresh += batch
        uq.run(torch.from_numpy(keys).to(DEV), off)
        uk, uo, inv, cnt = uq.fetch()
        split, _, restore, counts = oracle.hash_split(keys, 1, with_counts=True)
        np.testing.assert_array_equal(uk.cpu().numpy(), split)
        np.testing.assert_array_equal(inv.cpu().numpy(), restore)
        np.testing.assert_array_equal(cnt.cpu().numpy().view(np.uint32), counts)
        adm = f.feature_admit(capi.CHANNEL_TRAIN, uk.clone(), cnt, uo, [step], distinct=True)
        want_adm = orc_f.admit(split, counts, step, capi.CHANNEL_TRAIN)
        np.testing.assert_array_equal(adm.cpu().numpy(), want_adm, err_msg=f"admission mask, step {step}")
        admitted_total += int((want_adm != -1).sum())
        tg.key2offset(adm, uo, capi.CHANNEL_TRAIN)
        want_slots, rc = orc_t.key2offset(want_adm, capi.CHANNEL_TRAIN)
        assert rc == 0
        np.testing.assert_array_equal(adm.cpu().numpy(), want_slots, err_msg=f"slots, step {step}")
        ev, eo = f.feature_evict(cap=1 << 22)
        want_ev = orc_f.evict()
        np.testing.assert_array_equal(ev.cpu().numpy(), want_ev, err_msg=f"evicted keys, step {step}")
        evicted_total += want_ev.size
        for first in range(0, want_ev.size, batch):      # the table handle takes `batch` keys per call
            m = min(batch, want_ev.size - first)
            tg.evict_keys(ev[first:first + m].contiguous(), torch.tensor([0, m], dtype=torch.int64, device=DEV))
        orc_t.evict(want_ev)
        if step % 10 == 9 or step == steps - 1:
            mo, lv, _ = tg.stats()
            assert mo[0] == orc_t.size and lv[0] == orc_t.live
            live, latest = f.stats()
            assert live[0] == orc_f.dump()[0].size and latest[0] == step
    assert evicted_total > 1_000_000 and admitted_total > 500_000   # the sequence exercised both paths
    np.testing.assert_array_equal(np.array(tg.evict_pos(0, 1 << 22), dtype=np.int64), orc_t.evict_pos)
    gk, gc, gt = f.dump(0, 1 << 22)
    k, c, ts = orc_f.dump()
    order = k.argsort(kind="stable")
    np.testing.assert_array_equal(gk, k[order])
    np.testing.assert_array_equal(gc, c[order])
    np.testing.assert_array_equal(gt, ts[order])
