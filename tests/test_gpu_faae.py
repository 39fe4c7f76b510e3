"""GPU parity: feature admission / eviction history through the C ABI vs the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import capi, host
from recsdk_amd.synth import splitmix64, zipf_ranks

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    return (t.to(dtype) if dtype is not None else t).to(DEV)


def offs(*lens):
    return torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int64, device=DEV)


def test_feature_admit_and_evict_kat():
    """feature_admit_and_evict_test.cpp:283-325,405-421 with explicit timestamps; tables AAA (2, 5) and BBB (3, 7)."""
    t0 = 1000
    f = host.FeatureAdmitAndEvict([64, 64], [2, 3], [5, 7], max_keys=64)

    def admit(table, keys, cnt, ts):
        k = dev(np.array(keys, dtype=np.int64))
        c = dev(np.array(cnt, dtype=np.int32))
        o = offs(len(keys), 0) if table == 0 else offs(0, len(keys))
        stamps = [ts, 0] if table == 0 else [0, ts]
        # the other table gets no keys; its time must not move backwards
        stamps[1 - table] = -2**40
        return f.feature_admit(capi.CHANNEL_TRAIN, k, c, o, stamps).cpu().tolist()

    assert admit(0, [11, 11, 33, 44, 11, 55, 88, 55], [1, 2, 1, 3, 1, 1, 4, 1], t0) == [11, 11, -1, 44, 11, 55, 88, 55]
    assert admit(0, [11, 12, 33, 21, 11, 12], [1, 2, 1, 1, 2, 3], t0 + 1) == [11, 12, 33, -1, 11, 12]
    ev, eo = f.feature_evict()
    assert eo == [0, 0, 0]
    assert admit(1, [123, 121, 121, 212, 211], [1, 2, 1, 1, 2], t0 + 3) == [-1, 121, 121, -1, -1]
    assert admit(0, [11, 11, 33, 44, 55, 88, 55], [1, 2, 3, 2, 1, 2, 1], t0 + 9) == [11, 11, 33, 44, 55, 88, 55]
    assert admit(1, [125, 121, 122, 212, 211], [1, 2, 1, 3, 1], t0 + 11) == [-1, 121, -1, 212, 211]
    ev, eo = f.feature_evict()
    ev = ev.cpu().tolist()
    assert ev[eo[0]:eo[1]] == [12, 21] and ev[eo[1]:eo[2]] == [123]
    k, c, _ = f.dump(0, 64)
    assert dict(zip(k.tolist(), c.tolist())) == {11: 10, 33: 5, 44: 5, 55: 4, 88: 6}
    k, c, _ = f.dump(1, 64)
    assert dict(zip(k.tolist(), c.tolist())) == {121: 5, 122: 1, 125: 1, 211: 3, 212: 4}
    assert f.stats()[0] == [5, 5]


@pytest.mark.parametrize("coef,enable_sum", [(1, True), (3, True), (1, False)])
def test_random_stream_matches_oracle(coef, enable_sum):
    """Dynamic-expansion shaped stream: hot Zipf keys plus fresh ids, admit at count >= 2, evict idle >= 4."""
    rng = np.random.default_rng(0)
    T, n = 2, 3000
    f = host.FeatureAdmitAndEvict([40000, 40000], [2, 2], [4, 4], [coef, coef], [enable_sum, enable_sum],
                                  max_keys=T * n)
    orc = [oracle.Faae(2, 4, coef, enable_sum) for _ in range(T)]
    hot = [splitmix64(np.arange(500, dtype=np.uint64) + np.uint64(t * 10**6)) for t in range(T)]
    fresh = 10**9
    o = offs(n, n)
    for step in range(14):
        tables = []
        for t in range(T):
            is_hot = rng.random(n) < 0.7
            k = np.where(is_hot, hot[t][zipf_ranks(rng, 1.2, 500, n)], splitmix64(np.arange(fresh, fresh + n, dtype=np.uint64)))
            fresh += n
            k = np.where(rng.random(n) < 0.02, -1, k)
            tables.append(k.astype(np.int64))
        channel = capi.CHANNEL_EVAL if step % 5 == 3 else capi.CHANNEL_TRAIN
        keys = np.concatenate(tables)
        cnt = rng.integers(1, 4, keys.size)
        got = f.feature_admit(channel, dev(keys), dev(cnt, torch.int32), o, [step, step]).cpu().numpy()
        for t in range(T):
            want = orc[t].admit(tables[t], cnt[t * n:(t + 1) * n], step, channel)
            np.testing.assert_array_equal(got[t * n:(t + 1) * n], want)
        if step % 2 == 1:
            ev, eo = f.feature_evict()
            ev = ev.cpu().numpy()
            for t in range(T):
                np.testing.assert_array_equal(ev[eo[t]:eo[t + 1]], orc[t].evict())
        live, latest = f.stats()
        for t in range(T):
            k, c, ts = orc[t].dump()
            assert live[t] == k.size
            gk, gc, gt = f.dump(t, 1 << 16)
            np.testing.assert_array_equal(gk, k)
            np.testing.assert_array_equal(gc, c)
            np.testing.assert_array_equal(gt, ts)


def test_torch_feature_filter_flow_matches_oracle():
    rng = np.random.default_rng(1)
    n = 2000
    f = host.FeatureAdmitAndEvict([20000], [3], [4], max_keys=n)
    orc = oracle.Filter(admit_threshold=3, evict_threshold=4, evict_step_interval=2)
    o = offs(n)
    for step in range(10):
        keys = np.where(rng.random(n) < 0.6, zipf_ranks(rng, 1.1, 300, n), rng.integers(10**6, 10**9, n)).astype(np.int64)
        counts = rng.integers(0, 3, n)
        f.statistics_key_count(dev(keys), dev(counts, torch.int32), o)
        orc.statistics_key_count(keys, counts)
        got = f.count_filter(dev(keys), o).cpu().numpy()
        np.testing.assert_array_equal(got, orc.count_filter(keys))
        stamps = step + rng.integers(0, 2, n)
        f.record_timestamp(dev(keys), dev(stamps.astype(np.int64)), o)
        want_ev = orc.record_timestamp(keys, stamps)
        if want_ev is not None:  # the host wrapper of the reference evicts every evictStepInterval batches
            ev, eo = f.feature_evict(strict=True)
            np.testing.assert_array_equal(ev.cpu().numpy(), want_ev)


def test_history_full_is_reported():
    f = host.FeatureAdmitAndEvict([16], [1], [5], max_keys=4096)
    keys = dev(np.arange(4096, dtype=np.int64))
    f.feature_admit(capi.CHANNEL_TRAIN, keys, dev(np.ones(4096, np.int32)), offs(4096), [1])
    with pytest.raises(capi.RecsdkError) as e:
        f.stats()
    assert e.value.code == capi.EOVERFLOW


def test_admit_of_distinct_keys_equals_the_merging_call():
    """recsdk_faae_admit_distinct on a unique run's output behaves like recsdk_faae_admit on the same arrays."""
    rng = np.random.default_rng(9)
    T, n = 3, 4000
    a = host.FeatureAdmitAndEvict([60000] * T, [2, 3, 1], [4, 4, 4], max_keys=T * n)
    b = host.FeatureAdmitAndEvict([60000] * T, [2, 3, 1], [4, 4, 4], max_keys=T * n)
    uq = host.Unique(T * n, T)
    o = offs(*([n] * T))
    for step in range(8):
        keys = np.concatenate([np.where(rng.random(n) < 0.6, zipf_ranks(rng, 1.2, 400, n) + t * 10**6,
                                        rng.integers(10**7, 10**9, n)) for t in range(T)]).astype(np.int64)
        uk, uo, inv, cnt = uq.run(dev(keys), o).fetch()
        ka, kb = uk.clone(), uk.clone()
        channel = capi.CHANNEL_EVAL if step == 5 else capi.CHANNEL_TRAIN
        a.feature_admit(channel, ka, cnt, uo, [step] * T)
        b.feature_admit(channel, kb, cnt, uo, [step] * T, distinct=True)
        np.testing.assert_array_equal(ka.cpu().numpy(), kb.cpu().numpy())
        if step % 3 == 2:
            ea, eb = a.feature_evict(cap=1 << 16), b.feature_evict(cap=1 << 16)
            np.testing.assert_array_equal(ea[0].cpu().numpy(), eb[0].cpu().numpy())
        assert a.stats() == b.stats()
    for t in range(T):
        for x, y in zip(a.dump(t, 1 << 16), b.dump(t, 1 << 16)):
            np.testing.assert_array_equal(x, y)
