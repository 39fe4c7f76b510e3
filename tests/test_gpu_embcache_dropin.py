"""GPU: Embcache::SwapManager and Embcache::FeatureFilter as HIP-backed drop-ins (recsdk_amd/embcache), compiled
against the reference's own headers and driven through the classes' methods by tests/embcache_dropin_shim.cpp, replay
the vectors recorded from the reference's implementation of the same classes (tests/golden/ref_vectors.npz), bit for
bit.  Building needs the reference checkout (python -m recsdk_amd.embcache.build); the built files travel with the tree.
"""
import ctypes
import os

import numpy as np
import pytest

import oracle
from recsdk_amd.embcache import build as embcache_build

pytestmark = pytest.mark.gpu
G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors.npz"), allow_pickle=False)
P = ctypes.c_void_p
I64 = ctypes.c_int64


def _p(a):
    return None if a is None else a.ctypes.data_as(P)


@pytest.fixture(scope="module")
def shim():
    if not os.path.isfile(embcache_build.SHIM):
        if not os.path.isdir(embcache_build.CSRC):
            pytest.skip("the drop-in classes are not built and no reference checkout is here to build them against")
        embcache_build.build(verbose=False)
    lib = ctypes.CDLL(embcache_build.SHIM)
    for name, res, args in [
        ("dropin_swap_create", P, [I64, I64]), ("dropin_swap_destroy", None, [P]),
        ("dropin_swap_compute", ctypes.c_int32, [P, P, I64]), ("dropin_swap_error", ctypes.c_char_p, [P]),
        ("dropin_swap_result", I64, [P, ctypes.c_int32, P, I64]), ("dropin_swap_remove", None, [P, P, I64]),
        ("dropin_swap_get_keys", None, [P, I64, I64, P]), ("dropin_swap_mem_start", I64, [P]),
        ("dropin_filter_create", P, [I64, ctypes.c_uint64, ctypes.c_uint64]), ("dropin_filter_destroy", None, [P]),
        ("dropin_filter_statistics", ctypes.c_int32, [P, P, P, I64, I64]),
        ("dropin_filter_count_filter", ctypes.c_int32, [P, P, I64, I64]),
        ("dropin_filter_record_timestamp", I64, [P, P, P, I64, I64, P, I64]),
        ("dropin_filter_counts", I64, [P, P, P, I64]), ("dropin_filter_timestamps", I64, [P, P, P, I64]),
        ("dropin_filter_load", ctypes.c_int32, [P, P, P, P, I64]),
    ]:
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


def swap_compute(lib, h, keys):
    keys = np.ascontiguousarray(keys, dtype=np.int64)
    if lib.dropin_swap_compute(h, _p(keys), keys.size) != 0:
        raise RuntimeError(lib.dropin_swap_error(h).decode())
    out = []
    for which in range(5):
        buf = np.empty(max(keys.size, 1), dtype=np.int64)
        m = lib.dropin_swap_result(h, which, _p(buf), buf.size)
        out.append(buf[:m].copy())
    return out


@pytest.mark.parametrize("tag", ["swap_a", "swap_b"])
def test_swap_manager_class_replays_reference_vectors(shim, tag):
    cache, mem_start, steps = (int(x) for x in G[f"{tag}_cfg"])
    h = shim.dropin_swap_create(cache, mem_start)
    assert shim.dropin_swap_mem_start(h) == mem_start
    try:
        for s in range(steps):
            keys = G[f"{tag}_{s}_keys"]
            got = swap_compute(shim, h, keys)
            for name, g in zip(("so_keys", "so_offs", "si_keys", "si_offs", "batch_offs"), got):
                np.testing.assert_array_equal(g, G[f"{tag}_{s}_{name}"], err_msg=f"{tag} step {s} {name}")
            # GetKey: every slot the batch was sent to holds that batch's key (swap_manager.cpp:161-165)
            offs = got[4][keys != -1]
            for k, off in zip(keys[keys != -1][:64], offs[:64]):
                one = np.empty(1, dtype=np.int64)
                shim.dropin_swap_get_keys(h, int(off), int(off) + 1, _p(one))
                assert one[0] == k
            rm = np.ascontiguousarray(G[f"{tag}_{s}_remove"], dtype=np.int64)
            if rm.size:
                shim.dropin_swap_remove(h, _p(rm), rm.size)
    finally:
        shim.dropin_swap_destroy(h)


def test_swap_manager_class_raises_the_reference_message_when_the_batch_does_not_fit(shim):
    h = shim.dropin_swap_create(8, 0)
    try:
        swap_compute(shim, h, np.arange(4))
        with pytest.raises(RuntimeError, match="cacheSize_ too small"):
            swap_compute(shim, h, np.arange(100, 109))
    finally:
        shim.dropin_swap_destroy(h)


def test_swap_manager_class_against_the_oracle_on_a_longer_run(shim):
    rng = np.random.default_rng(5)
    cache, mem_start = 4096, 16
    h = shim.dropin_swap_create(cache, mem_start)
    orc = oracle.Swap(cache, mem_start)
    try:
        for s in range(30):
            keys = rng.zipf(1.2, 1500).astype(np.int64) % 20000
            keys[rng.random(keys.size) < 0.02] = -1
            got = swap_compute(shim, h, keys)
            want = orc.compute_swap_info(keys)
            for g, w in zip(got, want):
                np.testing.assert_array_equal(g, w, err_msg=f"step {s}")
            if s % 5 == 4:
                rm = rng.integers(0, 20000, 200).astype(np.int64)
                shim.dropin_swap_remove(h, _p(rm), rm.size)
                orc.remove_keys(rm)
    finally:
        shim.dropin_swap_destroy(h)


def test_feature_filter_class_replays_reference_vectors(shim):
    admit, evict, interval, steps = (int(x) for x in G["filter_a_cfg"])
    h = shim.dropin_filter_create(admit, evict, interval)
    try:
        for s in range(steps):
            keys = np.ascontiguousarray(G[f"filter_a_{s}_keys"], dtype=np.int64)
            counts = np.ascontiguousarray(G[f"filter_a_{s}_counts"], dtype=np.int64)
            stamps = np.ascontiguousarray(G[f"filter_a_{s}_stamps"], dtype=np.int64)
            assert shim.dropin_filter_statistics(h, _p(keys), _p(counts), 0, keys.size) == 0
            filtered = keys.copy()
            assert shim.dropin_filter_count_filter(h, _p(filtered), 0, keys.size) == 0
            np.testing.assert_array_equal(filtered, G[f"filter_a_{s}_filtered"], err_msg=f"step {s}")
            out = np.empty(4096, dtype=np.int64)
            m = shim.dropin_filter_record_timestamp(h, _p(keys), _p(stamps), 0, keys.size, _p(out), out.size)
            assert m >= 0
            np.testing.assert_array_equal(np.sort(out[:m]), G[f"filter_a_{s}_evicted_sorted"], err_msg=f"step {s}")
    finally:
        shim.dropin_filter_destroy(h)


def test_feature_filter_class_slices_maps_and_loads(shim):
    """The [startIndex, endIndex) slices EmbcacheManager hands each table (embcache_manager.cpp:219-262), the two maps
    the checkpoint writer reads and the two loaders, against the CPU oracle's restatement of the class."""
    rng = np.random.default_rng(11)
    admit, evict, interval = 4, 3, 2
    h = shim.dropin_filter_create(admit, evict, interval)
    orc = oracle.Filter(admit, evict, interval)
    want_counts, want_times = {}, {}   # the two maps, kept as the reference keeps them (feature_filter.cpp:34-80,112-140)
    try:
        for s in range(12):
            whole = rng.integers(0, 300, 400).astype(np.int64)
            first, last = 100, 350
            keys = whole[first:last]
            stamps_whole = (s + rng.integers(0, 2, whole.size)).astype(np.int64)
            assert shim.dropin_filter_statistics(h, _p(whole), None, first, last) == 0
            orc.statistics_key_count(keys, None)
            filtered = whole.copy()
            assert shim.dropin_filter_count_filter(h, _p(filtered), first, last) == 0
            np.testing.assert_array_equal(filtered[:first], whole[:first])
            np.testing.assert_array_equal(filtered[last:], whole[last:])
            np.testing.assert_array_equal(filtered[first:last], orc.count_filter(keys))
            out = np.empty(4096, dtype=np.int64)
            m = shim.dropin_filter_record_timestamp(h, _p(whole), _p(stamps_whole), first, last, _p(out), out.size)
            ev = orc.record_timestamp(keys, stamps_whole[first:last])
            ev = np.zeros(0, np.int64) if ev is None else np.sort(ev)
            np.testing.assert_array_equal(np.sort(out[:m]), ev, err_msg=f"step {s}")
            for k, t in zip(keys.tolist(), stamps_whole[first:last].tolist()):
                want_counts[k] = want_counts.get(k, 0) + 1
                want_times[k] = t
            for k in ev.tolist():
                want_counts.pop(k, None)
                want_times.pop(k, None)
        # the maps
        ck, cc = np.empty(4096, np.int64), np.empty(4096, np.uint64)
        nc = shim.dropin_filter_counts(h, _p(ck), _p(cc), ck.size)
        tk, tt = np.empty(4096, np.int64), np.empty(4096, np.int64)
        nt = shim.dropin_filter_timestamps(h, _p(tk), _p(tt), tk.size)
        assert dict(zip(ck[:nc].tolist(), cc[:nc].tolist())) == want_counts
        assert dict(zip(tk[:nt].tolist(), tt[:nt].tolist())) == want_times
        # a second filter loaded from the maps filters and evicts like the first
        h2 = shim.dropin_filter_create(admit, evict, interval)
        try:
            lk = np.ascontiguousarray(ck[:nc]); lc = np.ascontiguousarray(cc[:nc])
            assert shim.dropin_filter_load(h2, _p(lk), _p(lc), None, lk.size) == 0
            lk2 = np.ascontiguousarray(tk[:nt]); lt = np.ascontiguousarray(tt[:nt])
            assert shim.dropin_filter_load(h2, _p(lk2), None, _p(lt), lk2.size) == 0
            probe = np.arange(0, 300, dtype=np.int64)
            a, b = probe.copy(), probe.copy()
            assert shim.dropin_filter_count_filter(h, _p(a), 0, a.size) == 0
            assert shim.dropin_filter_count_filter(h2, _p(b), 0, b.size) == 0
            np.testing.assert_array_equal(a, b)
            nc2 = shim.dropin_filter_counts(h2, _p(ck), _p(cc), ck.size)
            assert dict(zip(ck[:nc2].tolist(), cc[:nc2].tolist())) == want_counts
        finally:
            shim.dropin_filter_destroy(h2)
    finally:
        shim.dropin_filter_destroy(h)


def test_two_swap_managers_driven_from_two_threads(shim):
    """EmbcacheManager computes the swap info of its tables from worker threads (embcache_manager.cpp:89-185): two
    objects driven at once, each on its thread's own stream, give what the oracle gives one after the other."""
    import threading

    def drive(seed, result):
        rng = np.random.default_rng(seed)
        h = shim.dropin_swap_create(2048, 1)
        orc = oracle.Swap(2048, 1)
        try:
            for s in range(25):
                keys = rng.zipf(1.2, 800).astype(np.int64) % 9000
                got = swap_compute(shim, h, keys)
                want = orc.compute_swap_info(keys)
                for g, w in zip(got, want):
                    np.testing.assert_array_equal(g, w, err_msg=f"seed {seed} step {s}")
            result.append(seed)
        finally:
            shim.dropin_swap_destroy(h)

    done = []
    threads = [threading.Thread(target=drive, args=(seed, done)) for seed in (21, 22)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert sorted(done) == [21, 22]
