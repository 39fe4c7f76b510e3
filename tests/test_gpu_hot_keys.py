"""GPU parity: hot-key staging of the restore vector (HotHashSplit / ComputeHotPos / UpdateHotMap for one rank)
through the C ABI, bit-exact against the CPU oracle, one oracle object per table."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import host

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def zipf_keys(rng, n, universe, a=1.2):
    return (rng.zipf(a, size=n) % universe).astype(np.int64) * 7919 - 3


def run_batches(sizes, universes, hot_counts, step, batches, seed):
    rng = np.random.default_rng(seed)
    T = len(sizes)
    kp = host.KeyProcess(max(sum(sizes), 1), T)
    kp.enable_hot_keys(hot_counts, hot_emb_update_step=step)
    orcs = [oracle.HotKeys(c) for c in hot_counts]
    for batch_id in range(batches):
        parts = [zipf_keys(rng, sizes[t], universes[t]) for t in range(T)]
        keys = np.concatenate(parts) if T else np.zeros(0, np.int64)
        offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
        uk, restore, hot_pos, cnt, uo = kp.hot_hash_split(torch.from_numpy(keys).to(DEV), batch_id,
                                                          torch.from_numpy(offs).to(DEV))
        uk, restore, hot_pos, cnt, uo = (x.cpu().numpy() for x in (uk, restore, hot_pos, cnt, uo))
        want_uk, want_restore, want_pos, want_cnt = [], [], [], []
        for t in range(T):
            s, r, p, c = orcs[t].hot_hash_split(parts[t], batch_id % step == 0)
            want_uk.append(s), want_restore.append(r), want_pos.append(p), want_cnt.append(c)
        msg = f"batch {batch_id}"
        np.testing.assert_array_equal(uk, np.concatenate(want_uk), err_msg=msg)
        np.testing.assert_array_equal(restore, np.concatenate(want_restore), err_msg=msg)
        np.testing.assert_array_equal(hot_pos, np.concatenate(want_pos), err_msg=msg)
        np.testing.assert_array_equal(cnt.view(np.uint32), np.concatenate(want_cnt), err_msg=msg)
        np.testing.assert_array_equal(np.diff(uo), [len(s) for s in want_uk], err_msg=msg)
    kp.close()


def test_small_known_answer():
    kp = host.KeyProcess(16, 1)
    kp.enable_hot_keys([2], hot_emb_update_step=1000)
    k1 = torch.tensor([5, 9, 5, 7, 9, 5, 1], dtype=torch.int64, device=DEV)
    uk, restore, hot_pos, cnt, _ = kp.hot_hash_split(k1, 0)
    assert uk.tolist() == [5, 9, 7, 1] and restore.tolist() == [2, 3, 2, 4, 3, 2, 5] and hot_pos.tolist() == [0, 0]
    k2 = torch.tensor([4, 9, 5, 9, 4, 8], dtype=torch.int64, device=DEV)
    uk, restore, hot_pos, cnt, _ = kp.hot_hash_split(k2, 1)
    assert uk.tolist() == [4, 9, 5, 8] and restore.tolist() == [2, 0, 1, 0, 2, 5] and hot_pos.tolist() == [1, 2]


@pytest.mark.parametrize("sizes,universes,hot_counts,step", [
    ([3000], [400], [32], 3),
    ([5000, 1, 0, 7000], [50, 5, 5, 100000], [64, 4, 4, 128], 2),   # hot set larger than the table's key universe
    ([4096, 4096, 4096], [1000, 2000, 4000], [0, 16, 1], 4),        # a table without hot keys
    ([100000, 50000], [20000, 3], [1024, 8], 3),                    # many tiles; tables that start inside a tile
])
def test_batches_match_oracle(sizes, universes, hot_counts, step):
    run_batches(sizes, universes, hot_counts, step, batches=7, seed=sum(sizes) + step)


def test_full_batch_26_tables():
    T = 26
    run_batches([65536] * T, [1 << 20] * T, [2048] * T, 2, batches=3, seed=26)


def test_rejects_mismatched_tables():
    kp = host.KeyProcess(64, 2)
    kp.enable_hot_keys([4], hot_emb_update_step=10)
    keys = torch.arange(10, dtype=torch.int64, device=DEV)
    offs = torch.tensor([0, 5, 10], dtype=torch.int64, device=DEV)
    with pytest.raises(RuntimeError):
        kp.hot_hash_split(keys, 0, offs)
