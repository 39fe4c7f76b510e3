"""The CPU oracle against vectors recorded from the REFERENCE's own code (tests/golden/ref_vectors.npz, written by
tests/golden/make_ref_vectors.py through the reference build under oracle/_ref).  Unlike
test_oracle_vs_reference_build.py this runs wherever the repository is, also without the reference checkout."""
import os

import numpy as np
import pytest

import oracle

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors.npz"), allow_pickle=False)


@pytest.mark.parametrize("tag", ["swap_a", "swap_b"])
def test_swap_manager_sequences(tag):
    cache, mem_start, steps = (int(x) for x in G[f"{tag}_cfg"])
    orc = oracle.Swap(cache, mem_start)
    for s in range(steps):
        got = orc.compute_swap_info(G[f"{tag}_{s}_keys"])
        for name, g in zip(("so_keys", "so_offs", "si_keys", "si_offs", "batch_offs"), got):
            np.testing.assert_array_equal(g, G[f"{tag}_{s}_{name}"], err_msg=f"{tag} step {s} {name}")
        rm = G[f"{tag}_{s}_remove"]
        if rm.size:
            orc.remove_keys(rm)


def test_feature_filter_sequence():
    admit, evict, interval, steps = (int(x) for x in G["filter_a_cfg"])
    orc = oracle.Filter(admit, evict, interval)
    for s in range(steps):
        keys = G[f"filter_a_{s}_keys"]
        orc.statistics_key_count(keys, G[f"filter_a_{s}_counts"])
        np.testing.assert_array_equal(orc.count_filter(keys), G[f"filter_a_{s}_filtered"])
        ev = orc.record_timestamp(keys, G[f"filter_a_{s}_stamps"])
        ev = np.zeros(0, np.int64) if ev is None else np.sort(ev)
        np.testing.assert_array_equal(ev, G[f"filter_a_{s}_evicted_sorted"])


def test_ids_mapper_is_dedup_plus_first_seen_slots():
    T, steps = (int(x) for x in G["ids_a_cfg"])
    tabs = [oracle.Table(10 ** 6) for _ in range(T)]
    for s in range(steps):
        offs, ids = G[f"ids_a_{s}_offs"], G[f"ids_a_{s}_ids"]
        uoff = G[f"ids_a_{s}_uoff"]
        for t in range(T):
            split, _, restore, _ = oracle.hash_split(ids[offs[t]:offs[t + 1]], 1)
            slots, _ = tabs[t].key2offset(split, 0)
            np.testing.assert_array_equal(G[f"ids_a_{s}_uniq_ids"][uoff[t]:uoff[t + 1]], split)
            np.testing.assert_array_equal(G[f"ids_a_{s}_uniq"][uoff[t]:uoff[t + 1]], slots)
            np.testing.assert_array_equal(G[f"ids_a_{s}_inv"][offs[t]:offs[t + 1]], restore)
            np.testing.assert_array_equal(G[f"ids_a_{s}_hash_idx"][offs[t]:offs[t + 1]], slots[restore])


def test_unique_parallel():
    for j in range(3):
        u, inv = oracle.unique_sorted(G[f"uniqpar_{j}_ids"])
        np.testing.assert_array_equal(u, G[f"uniqpar_{j}_unique"])
        np.testing.assert_array_equal(inv, G[f"uniqpar_{j}_inverse"])
