"""GPU parity of the allocation-free dedup entry point: recsdk_unique_run_noalloc (workspace = a static device array
inside the library) against recsdk_unique_run + recsdk_unique_fetch on the same keys, bit for bit, through the C ABI.
Two calls in a row share the array, the second with a smaller input, so stale contents of the first must not show."""
import numpy as np
import pytest
import torch

from recsdk_amd import capi, host
from tests.util import zipf_keys

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MAX_KEYS = 65536
MAX_TABLES = 64


def _ptr(t):
    return None if t is None else t.data_ptr()


def noalloc(tables, counts=None, skip_key=None, want_counts=True):
    keys = np.concatenate(tables + [np.zeros(0, np.int64)]).astype(np.int64)
    offs = np.concatenate([[0], np.cumsum([len(t) for t in tables])]).astype(np.int64)
    n, T = keys.size, len(tables)
    dk = torch.from_numpy(keys).to(DEV)
    do = torch.from_numpy(offs).to(DEV)
    dc = torch.from_numpy(counts.astype(np.int32)).to(DEV) if counts is not None else None
    # outputs pre-filled so that untouched entries are recognisable
    uk = torch.full((max(n, 1),), -7, dtype=torch.int64, device=DEV)
    uo = torch.full((T + 1,), -7, dtype=torch.int64, device=DEV)
    inv = torch.full((max(n, 1),), -7, dtype=torch.int32, device=DEV)
    cnt = torch.full((max(n, 1),), -7, dtype=torch.int32, device=DEV) if want_counts else None
    stream = torch.cuda.current_stream().cuda_stream
    capi.check(capi.lib().recsdk_unique_run_noalloc(_ptr(dk), _ptr(dc), _ptr(do), T, n, 0 if skip_key is None else 1,
                                                    0 if skip_key is None else int(skip_key), _ptr(uk), _ptr(uo),
                                                    _ptr(inv), _ptr(cnt), stream))
    torch.cuda.synchronize()
    uo_h = uo.cpu().numpy()
    u = int(uo_h[T])
    return (uk.cpu().numpy()[:u], uo_h, inv.cpu().numpy()[:n], cnt.cpu().numpy()[:u] if want_counts else None)


def with_handle(tables, counts=None, skip_key=None):
    keys = np.concatenate(tables + [np.zeros(0, np.int64)]).astype(np.int64)
    offs = np.concatenate([[0], np.cumsum([len(t) for t in tables])]).astype(np.int64)
    uq = host.Unique(max(keys.size, 1), len(tables), position_lists=False)
    dc = torch.from_numpy(counts.astype(np.int32)).to(DEV) if counts is not None else None
    uk, uo, inv, cnt = uq.run(torch.from_numpy(keys).to(DEV), torch.from_numpy(offs).to(DEV), in_counts=dc,
                              skip_key=skip_key).fetch()
    return uk.cpu().numpy(), uo.cpu().numpy(), inv.cpu().numpy(), cnt.cpu().numpy()


def same(a, b):
    for x, y in zip(a, b):
        if x is not None:
            np.testing.assert_array_equal(x, y)


def test_two_calls_in_a_row_second_smaller():
    rng = np.random.default_rng(11)
    big = [zipf_keys(rng, 1.05, 1000 * (t + 1), 2500, table=t) for t in range(26)]   # 65000 keys, 26 tables
    small = [rng.integers(-50, 50, 700), np.zeros(0, np.int64), rng.integers(0, 2**62, 1025)]
    got_big = noalloc(big)
    got_small = noalloc(small)
    same(got_big, with_handle(big))
    same(got_small, with_handle(small))
    # and once more the large one over the small one's leftovers, without the counts output
    same(noalloc(big, want_counts=False), with_handle(big))


def test_limits_counts_skip_key_and_empty():
    rng = np.random.default_rng(12)
    full = [rng.integers(0, 3000, MAX_KEYS)]
    same(noalloc(full), with_handle(full))
    # input counts are summed per distinct key; a skipped key gets inverse -1
    keys = [np.array([5, -1, 5, 9, -1, 2**63 - 1, -2**63, 9, 5]), np.array([-1, -1, 4])]
    cnts = np.arange(1, 13)
    same(noalloc(keys, counts=cnts), with_handle(keys, counts=cnts))
    same(noalloc(keys, skip_key=-1), with_handle(keys, skip_key=-1))
    uk, uo, inv, cnt = noalloc([np.zeros(0, np.int64), np.zeros(0, np.int64)])
    assert uk.size == 0 and uo.tolist() == [0, 0, 0] and inv.size == 0
    many = [rng.integers(0, 9, 5) for _ in range(MAX_TABLES)]
    same(noalloc(many), with_handle(many))


def test_sizes_beyond_the_static_workspace_are_rejected():
    L = capi.lib()
    one = torch.zeros(8, dtype=torch.int64, device=DEV)
    args = (_ptr(one), None, _ptr(one))
    outs = (0, 0, _ptr(one), _ptr(one), _ptr(one), None, None)
    assert L.recsdk_unique_run_noalloc(*args, 1, MAX_KEYS + 1, *outs) == capi.ECAPACITY
    assert b"RECSDK_UNIQUE_NOALLOC_MAX_KEYS" in L.recsdk_last_error()
    assert L.recsdk_unique_run_noalloc(*args, MAX_TABLES + 1, 4, *outs) == capi.ECAPACITY
    assert L.recsdk_unique_run_noalloc(*args, 0, 4, *outs) == capi.ECAPACITY
