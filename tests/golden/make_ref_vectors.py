"""Writes tests/golden/ref_vectors.npz: input/output vectors recorded from the REFERENCE's own code (SwapManager,
FeatureFilter, IdsMapper, UniqueParallel), run through oracle/_ref/libref_torch.so, which `make -C oracle -f ref.mk`
compiles from the reference checkout.  Only data is stored: seeded inputs and the outputs the reference produced.

    python tests/golden/make_ref_vectors.py        (needs the reference checkout and the built checker)
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
from oracle import ref_loader  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_vectors.npz")


def swap_case(tag, cache, mem_start, universe, steps, seed, store):
    rng = np.random.default_rng(seed)
    ref = ref_loader.RefSwap(cache, mem_start)
    store[f"{tag}_cfg"] = np.array([cache, mem_start, steps], dtype=np.int64)
    for s in range(steps):
        n = int(rng.integers(1, max(2, (cache - mem_start) // 3)))
        keys = rng.integers(0, universe, n)
        keys = np.where(rng.random(n) < 0.05, -1, keys).astype(np.int64)
        out = ref.compute_swap_info(keys)
        store[f"{tag}_{s}_keys"] = keys
        for name, a in zip(("so_keys", "so_offs", "si_keys", "si_offs", "batch_offs"), out):
            store[f"{tag}_{s}_{name}"] = np.asarray(a, dtype=np.int64)
        rm = rng.integers(0, universe, 10).astype(np.int64) if s % 7 == 6 else np.zeros(0, np.int64)
        store[f"{tag}_{s}_remove"] = rm
        if rm.size:
            ref.remove_keys(rm)


def filter_case(tag, admit, evict, interval, steps, seed, store):
    rng = np.random.default_rng(seed)
    ref = ref_loader.RefFilter(admit, evict, interval)
    store[f"{tag}_cfg"] = np.array([admit, evict, interval, steps], dtype=np.int64)
    for s in range(steps):
        keys = rng.integers(0, 80, 50).astype(np.int64)
        counts = rng.integers(-1, 4, 50).astype(np.int64)
        stamps = (s + rng.integers(0, 2, 50)).astype(np.int64)
        ref.statistics_key_count(keys, counts)
        filtered = ref.count_filter(keys)
        evicted = ref.record_timestamp(keys, stamps)
        store[f"{tag}_{s}_keys"] = keys
        store[f"{tag}_{s}_counts"] = counts
        store[f"{tag}_{s}_stamps"] = stamps
        store[f"{tag}_{s}_filtered"] = np.asarray(filtered, dtype=np.int64)
        store[f"{tag}_{s}_evicted_sorted"] = np.sort(np.asarray(evicted, dtype=np.int64))


def ids_case(tag, T, steps, seed, store):
    rng = np.random.default_rng(seed)
    ref = ref_loader.RefIdsMapper([10 ** 6] * T)
    store[f"{tag}_cfg"] = np.array([T, steps], dtype=np.int64)
    for s in range(steps):
        lens = rng.integers(0, 400, T)
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        ids = rng.integers(0, 300, int(offs[-1])).astype(np.int64)
        hash_idx, uniq, uniq_ids, inv, uoff = ref.parallel_unique_hash_out(ids, offs)
        for name, a in zip(("offs", "ids", "hash_idx", "uniq", "uniq_ids", "inv", "uoff"),
                           (offs, ids, hash_idx, uniq, uniq_ids, inv, uoff)):
            store[f"{tag}_{s}_{name}"] = np.asarray(a, dtype=np.int64)


def unique_parallel_case(tag, seed, store):
    rng = np.random.default_rng(seed)
    for j, n in enumerate((1, 100, 5000)):
        ids = rng.integers(-(1 << 62), 1 << 62, n).astype(np.int64)
        ids[rng.integers(0, n, n // 2)] = ids[0]
        u, inv = ref_loader.ref_unique_parallel(ids)
        store[f"{tag}_{j}_ids"] = ids
        store[f"{tag}_{j}_unique"] = u
        store[f"{tag}_{j}_inverse"] = inv


def main():
    if not ref_loader.available():
        raise SystemExit("oracle/_ref/libref_torch.so is not built: make -C oracle -f ref.mk")
    store = {}
    swap_case("swap_a", 64, 0, 200, 40, 64, store)
    swap_case("swap_b", 300, 1, 1000, 40, 300, store)
    filter_case("filter_a", 3, 4, 2, 14, 3, store)
    ids_case("ids_a", 3, 5, 4, store)
    unique_parallel_case("uniqpar", 6, store)
    np.savez_compressed(OUT, **store)
    print(OUT, os.path.getsize(OUT), "bytes,", len(store), "arrays")


if __name__ == "__main__":
    main()
