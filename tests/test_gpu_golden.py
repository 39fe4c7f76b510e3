"""GPU parity against vectors recorded from the REFERENCE's own code (tests/golden/ref_vectors.npz): the device
cache planner, the ids mapper and the sorted unique, through the C ABI, bit for bit."""
import os

import numpy as np
import pytest
import torch

from recsdk_amd import host

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors.npz"), allow_pickle=False)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)).to(DEV)


@pytest.mark.parametrize("tag", ["swap_a", "swap_b"])
def test_swap_manager_matches_reference_vectors(tag):
    cache, mem_start, steps = (int(x) for x in G[f"{tag}_cfg"])
    sm = host.SwapManager(cache, mem_start, max_keys=4096)
    for s in range(steps):
        got = sm.compute_swap_info(dev(G[f"{tag}_{s}_keys"]))
        for name, g in zip(("so_keys", "so_offs", "si_keys", "si_offs", "batch_offs"), got):
            np.testing.assert_array_equal(g.cpu().numpy(), G[f"{tag}_{s}_{name}"], err_msg=f"{tag} step {s} {name}")
        rm = G[f"{tag}_{s}_remove"]
        if rm.size:
            sm.remove_keys(dev(rm))


def test_unique_parallel_matches_reference_vectors():
    for j in range(3):
        u, inv = host.unique_parallel(dev(G[f"uniqpar_{j}_ids"]))
        np.testing.assert_array_equal(u.cpu().numpy(), G[f"uniqpar_{j}_unique"])
        np.testing.assert_array_equal(inv.cpu().numpy(), G[f"uniqpar_{j}_inverse"])


def test_ids_mapper_matches_reference_vectors():
    T, steps = (int(x) for x in G["ids_a_cfg"])
    mapper = host.IdsMapper([10 ** 6] * T, max_keys=4096)
    for s in range(steps):
        offs, ids = G[f"ids_a_{s}_offs"], G[f"ids_a_{s}_ids"]
        hash_idx, uniq, uniq_ids, inv, uoff = mapper.parallel_unique_hash_out(dev(ids), dev(offs))
        np.testing.assert_array_equal(uoff.cpu().numpy(), G[f"ids_a_{s}_uoff"])
        np.testing.assert_array_equal(uniq_ids.cpu().numpy(), G[f"ids_a_{s}_uniq_ids"])
        np.testing.assert_array_equal(uniq.cpu().numpy(), G[f"ids_a_{s}_uniq"])
        np.testing.assert_array_equal(inv.cpu().numpy(), G[f"ids_a_{s}_inv"])
        np.testing.assert_array_equal(hash_idx.cpu().numpy(), G[f"ids_a_{s}_hash_idx"])
