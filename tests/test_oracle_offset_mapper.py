"""CPU checks that pin the oracle's restatement of the AccCTR OffsetMapper (HBM-cache planner of the TF path).

The AccCTR sources need a header that is not in the image (securec.h), so no reference build exists for them.
Pins used instead:
  * the return-code cases of the reference's own test (AccCTR/tests/ut/src/emb_cache_test.cpp:925-1036, 1144-1301),
  * the invariants its DEVICE_COMBINE_TEST asserts over 50 random batches (emb_cache_test.cpp:1039-1142),
  * an independent model written from the sequential definition with a different data structure (a plain Python
    list for the reusable-slot order), which a wrong list direction, a wrong hit/miss order or a dropped
    "previous batch" rule would contradict,
  * a hand-derived sequence.
"""
import numpy as np
import pytest

import oracle


class ListModel:
    """OffsetMapper written with Python lists/dicts (offset_mapper.h:135-295): `valid` and `evicted` hold slots in
    iteration order (front = most recently inserted)."""

    def __init__(self, max_cache):
        self.max = max_cache
        self.use = 0
        self.map = {}
        self.pos2key = {}
        self.valid = []
        self.evicted = []
        self.last = []

    def compute(self, keys):
        keys = [int(k) for k in keys]
        swap_in = []
        ids = []
        for i, k in enumerate(keys):
            if k == -1:
                continue
            if k in self.map:
                keys[i] = self.map[k]
                if keys[i] in self.valid:
                    self.valid.remove(keys[i])
            else:
                swap_in.append(k)
                ids.append(i)
        free = self.max - self.use + len(self.evicted)
        out_num = max(0, len(swap_in) - free)
        pos = []
        out_keys, out_pos = [], []
        taken = 0
        for p in list(self.evicted):
            if len(pos) == len(swap_in):
                break
            pos.append(p)
            taken += 1
        for p in list(self.valid):
            if len(out_keys) == out_num:
                break
            pos.append(p)
            out_keys.append(self.pos2key[p])
            out_pos.append(p)
        if len(out_keys) < out_num:
            raise RuntimeError("too small")
        while len(pos) < len(swap_in):
            if self.use >= self.max:
                raise RuntimeError("too small")
            pos.append(self.use)
            self.use += 1
        for k in out_keys:
            del self.map[k]
        for k, p, i in zip(swap_in, pos, ids):
            self.map[k] = p
            self.pos2key[p] = k
            keys[i] = p
        for p in self.last:
            if p != -1 and p not in self.valid:
                self.valid.insert(0, p)
        for p in keys:
            if p != -1:
                if p in self.valid:
                    self.valid.remove(p)
                if p in self.evicted:
                    self.evicted.remove(p)
        self.last = list(keys)
        return np.array(keys), np.array(swap_in), np.array(pos), np.array(out_keys), np.array(out_pos)

    def remove(self, keys):
        for k in keys:
            k = int(k)
            if k not in self.map:
                continue
            p = self.map.pop(k)
            if p in self.valid:
                self.valid.remove(p)
            if p in self.last:
                self.last.remove(p)
            if p not in self.evicted:
                self.evicted.insert(0, p)


def same(a, b):
    for x, y in zip(a, b):
        np.testing.assert_array_equal(np.asarray(x, dtype=np.int64), np.asarray(y, dtype=np.int64))


def test_reference_return_code_cases():
    # emb_cache_test.cpp:948-984: 5 new keys, 3 cached keys, fill to exactly max, then one key too many
    om = oracle.OffsetMapper(10)
    off, sik, sip, sok, sop = om.get_swap_pairs_and_key2offset([0, 1, 2, 3, 4])
    np.testing.assert_array_equal(sik, [0, 1, 2, 3, 4])
    off, sik, *_ = om.get_swap_pairs_and_key2offset([1, 2, 3])
    assert sik.size == 0
    np.testing.assert_array_equal(off, [1, 2, 3])
    om.get_swap_pairs_and_key2offset(np.arange(10))
    with pytest.raises(RuntimeError):
        om.get_swap_pairs_and_key2offset(np.arange(11))
    # :987-992 a single batch larger than the cache
    with pytest.raises(RuntimeError):
        oracle.OffsetMapper(10).get_swap_pairs_and_key2offset(np.arange(15))
    # :1017-1035 invalid keys and empty input
    om = oracle.OffsetMapper(10)
    off, sik, sip, sok, sop = om.get_swap_pairs_and_key2offset([-1] * 5)
    assert sik.size == sip.size == sok.size == sop.size == 0
    np.testing.assert_array_equal(off, [-1] * 5)
    off, sik, sip, sok, sop = om.get_swap_pairs_and_key2offset([])
    assert off.size == sik.size == sok.size == 0


def test_three_batches_hand_derived():
    # emb_cache_test.cpp:1002-1014 asserts H_OK; the lists follow from the definition: batch 3 finds the cache full,
    # only batch 1's slots may be reused, and the list hands them out last-pushed first (slot 4 .. slot 0)
    om = oracle.OffsetMapper(10)
    om.get_swap_pairs_and_key2offset([0, 1, 2, 3, 4])
    om.get_swap_pairs_and_key2offset([5, 6, 7, 8, 9])
    off, sik, sip, sok, sop = om.get_swap_pairs_and_key2offset([10, 11, 12, 13, 14])
    np.testing.assert_array_equal(off, [4, 3, 2, 1, 0])
    np.testing.assert_array_equal(sip, [4, 3, 2, 1, 0])
    np.testing.assert_array_equal(sok, [4, 3, 2, 1, 0])
    np.testing.assert_array_equal(sop, [4, 3, 2, 1, 0])


def test_remove_then_reuse_like_reference_test():
    # emb_cache_test.cpp:1219-1298: fill, remove all, the next keys reuse freed slots (latest freed first)
    om = oracle.OffsetMapper(10)
    om.get_swap_pairs_and_key2offset(np.arange(10))
    om.remove(np.arange(10))
    st = om.state()
    assert st["keys"].size == 0 and st["evict_size"] == 10
    off, sik, sip, sok, sop = om.get_swap_pairs_and_key2offset([9, 10, 11, 12, 13])
    np.testing.assert_array_equal(sik, [9, 10, 11, 12, 13])
    np.testing.assert_array_equal(sip, [9, 8, 7, 6, 5])   # slot 9 was freed last
    assert sok.size == 0
    om.remove([9, 10, 11, 3])
    off, sik, sip, sok, sop = om.get_swap_pairs_and_key2offset(np.arange(8))
    np.testing.assert_array_equal(sik, np.arange(8))
    assert sok.size == 0 and sip.size == 8
    om.get_swap_pairs_and_key2offset([15])


@pytest.mark.parametrize("cache,universe,batch", [(10, 40, 4), (64, 200, 20), (500, 5000, 150)])
def test_matches_list_model(cache, universe, batch):
    rng = np.random.default_rng(cache)
    om = oracle.OffsetMapper(cache)
    model = ListModel(cache)
    for step in range(60):
        n = int(rng.integers(0, batch + 1))
        keys = rng.choice(universe, size=n, replace=False).astype(np.int64)
        keys = np.where(rng.random(n) < 0.05, -1, keys)
        try:
            want = model.compute(keys)
        except RuntimeError:
            with pytest.raises(RuntimeError):
                om.get_swap_pairs_and_key2offset(keys)
            break
        same(om.get_swap_pairs_and_key2offset(keys), want)
        if step % 5 == 4:
            rm = rng.choice(universe, size=min(10, universe), replace=False)
            model.remove(rm)
            om.remove(rm)
        st = om.state()
        assert st["use_length"] == model.use and st["evict_size"] == len(model.evicted)
        assert dict(zip(st["keys"].tolist(), st["slots"].tolist())) == model.map


def test_device_combine_invariants():
    # the properties emb_cache_test.cpp:1039-1142 asserts, on inputs of the same shape (about 9.5k distinct sorted
    # keys of [0, 100000] per batch, cache of 30000 slots, 50 batches)
    rng = np.random.default_rng(123)
    cache = 30000
    om = oracle.OffsetMapper(cache)
    cached = set()
    used_offsets = set()
    history = []
    for _ in range(50):
        keys = np.unique(rng.integers(0, 100001, 10000)).astype(np.int64)
        off, sik, sip, sok, sop = om.get_swap_pairs_and_key2offset(keys)
        new = set(keys.tolist()) - cached
        assert set(sik.tolist()) == new and sik.size == len(new)
        cached |= set(keys.tolist())
        history.insert(0, set(keys.tolist()))
        del history[2:]
        for k in sok.tolist():
            assert all(k not in h for h in history)
            assert k in cached
        cached -= set(sok.tolist())
        assert len(cached) <= cache
        assert set(sop.tolist()) <= used_offsets
        used_offsets -= set(sop.tolist())
        assert not (set(sip.tolist()) & used_offsets)
        used_offsets |= set(sip.tolist())
        assert len(set(off.tolist())) == keys.size
