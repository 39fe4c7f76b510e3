"""GPU parity: by-address lookup / update, LazyAdam, Sgd through the C ABI vs the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
from recsdk_amd import host

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _tables(seed, rows, dim, dtype=np.float32):
    rng = np.random.default_rng(seed)
    if dtype == np.int32:
        return rng.integers(-1000, 1000, (rows, dim)).astype(np.int32)
    return rng.normal(0, 1, (rows, dim)).astype(dtype)


@pytest.mark.parametrize("dim,dtype", [(8, torch.float32), (16, torch.float32), (128, torch.float32), (384, torch.float32),
                                       (7, torch.float32), (9, torch.float16), (64, torch.float16), (8, torch.int32),
                                       (64, torch.bfloat16)])
def test_lookup_by_address_bit_exact(dim, dtype):
    emb_size, addr_num = 100000, 21632  # the shape of the reference's gen_lookup_data.py
    rng = np.random.default_rng(0)
    offset = rng.integers(0, emb_size, addr_num)
    npdt = {torch.float32: np.float32, torch.float16: np.float16, torch.int32: np.int32,
            torch.bfloat16: np.float32}[dtype]
    emb = _tables(1, emb_size, dim, npdt)
    demb = torch.from_numpy(emb).to(DEV).to(dtype).contiguous()
    hemb = demb.cpu()
    hview = hemb.view(torch.int16).numpy() if dtype == torch.bfloat16 else hemb.numpy()
    esize = demb.element_size()
    skip = rng.random(addr_num) < 0.05
    daddr = torch.from_numpy(np.where(skip, 0, demb.data_ptr() + offset * dim * esize)).to(DEV)
    haddr = np.where(skip, 0, hview.ctypes.data + offset * dim * esize)
    got = host.embedding_lookup_by_address(daddr, dim, dtype)
    want = oracle.lookup_by_addr(haddr, dim, hview.dtype)
    g = got.cpu()
    g = g.view(torch.int16).numpy() if dtype == torch.bfloat16 else g.numpy()
    np.testing.assert_array_equal(g, want)


def test_lookup_by_address_empty_and_all_invalid():
    daddr = torch.zeros(0, dtype=torch.int64, device=DEV)
    assert host.embedding_lookup_by_address(daddr, 8).shape == (0, 8)
    daddr = torch.zeros(33, dtype=torch.int64, device=DEV)
    assert (host.embedding_lookup_by_address(daddr, 24) == 0).all()


@pytest.mark.parametrize("dim", [8, 128, 6])
def test_update_by_address_overwrite_distinct_rows(dim):
    rng = np.random.default_rng(2)
    emb_size, n = 50000, 20000
    rows = rng.permutation(emb_size)[:n]
    emb = _tables(3, emb_size, dim)
    upd = rng.uniform(1, 10, (n, dim)).astype(np.float32)
    demb = torch.from_numpy(emb).to(DEV)
    daddr = torch.from_numpy(demb.data_ptr() + rows * dim * 4).to(DEV)
    host.embedding_update_by_address(daddr, torch.from_numpy(upd).to(DEV), update_type=1)
    want = emb.copy()
    oracle.update_by_addr(want.ctypes.data + rows * dim * 4, upd, 1)
    np.testing.assert_array_equal(demb.cpu().numpy(), want)


@pytest.mark.parametrize("dim", [8, 96])
def test_update_by_address_atomic_add_with_duplicates(dim):
    """Duplicates accumulate; the order of the atomic adds is not fixed, so rows hit more than once are
    compared within 1e-6 relative to the sum of magnitudes, rows hit once exactly."""
    rng = np.random.default_rng(4)
    emb_size, n = 5000, 21632
    rows = rng.integers(0, emb_size, n)
    skip = rng.random(n) < 0.03
    emb = (np.arange(emb_size * dim) * 0.01).astype(np.float32).reshape(emb_size, dim)
    upd = rng.uniform(1, 10, (n, dim)).astype(np.float32)
    demb = torch.from_numpy(emb).to(DEV)
    daddr = torch.from_numpy(np.where(skip, 0, demb.data_ptr() + rows * dim * 4)).to(DEV)
    host.embedding_update_by_address(daddr, torch.from_numpy(upd).to(DEV), update_type=0)
    want = emb.copy()
    oracle.update_by_addr(np.where(skip, 0, want.ctypes.data + rows * dim * 4), upd, 0)
    got = demb.cpu().numpy()
    hits = np.bincount(rows[~skip], minlength=emb_size)
    once = hits <= 1
    np.testing.assert_array_equal(got[once], want[once])
    scale = np.abs(emb).copy()
    np.add.at(scale, rows[~skip], np.abs(upd[~skip]))
    assert (np.abs(got - want) <= 1e-6 * scale).all()


def test_update_by_address_int32_and_fp16():
    rng = np.random.default_rng(5)
    emb_size, n, dim = 1000, 4000, 10
    rows = rng.integers(0, emb_size, n)
    emb = rng.integers(-100, 100, (emb_size, dim)).astype(np.int32)
    upd = rng.integers(-5, 5, (n, dim)).astype(np.int32)
    demb = torch.from_numpy(emb).to(DEV)
    daddr = torch.from_numpy(demb.data_ptr() + rows * dim * 4).to(DEV)
    host.embedding_update_by_address(daddr, torch.from_numpy(upd).to(DEV), 0)
    want = emb.copy()
    np.add.at(want, rows, upd)
    np.testing.assert_array_equal(demb.cpu().numpy(), want)
    # fp16: distinct rows so that the sum is a single rounding
    rows = rng.permutation(emb_size)[:500]
    e16 = rng.normal(0, 1, (emb_size, dim)).astype(np.float16)
    u16 = rng.normal(0, 1, (500, dim)).astype(np.float16)
    d16 = torch.from_numpy(e16).to(DEV)
    a16 = torch.from_numpy(d16.data_ptr() + rows * dim * 2).to(DEV)
    host.embedding_update_by_address(a16, torch.from_numpy(u16).to(DEV), 0)
    w16 = e16.copy()
    w16[rows] = (e16[rows].astype(np.float32) + u16.astype(np.float32)).astype(np.float16)
    np.testing.assert_array_equal(d16.cpu().numpy(), w16)


@pytest.mark.parametrize("dim", [32, 128, 10])
def test_lazy_adam_bit_exact(dim):
    rng = np.random.default_rng(6)
    rows, n = 200000, 56409
    var = rng.uniform(1, 2, (rows, dim)).astype(np.float32)
    m = rng.uniform(1, 2, (rows, dim)).astype(np.float32)
    v = rng.uniform(1, 2, (rows, dim)).astype(np.float32)
    idx = rng.permutation(rows)[:n].astype(np.int32)
    idx[::41] = -1
    grad = rng.uniform(1, 2, (n, dim)).astype(np.float32)
    dm, dv, dvar = (torch.from_numpy(x).to(DEV) for x in (m, v, var))
    host.lazy_adam(torch.from_numpy(grad).to(DEV), torch.from_numpy(idx).to(DEV), dm, dv, dvar, 0.001, 0.9, 0.999,
                   1e-7)
    oracle.lazy_adam(grad, idx, m, v, var, 0.001, 0.9, 0.999, 1e-7)
    # tolerance of the path is 1e-6 relative; the kernel rounds like the scalar definition, so it is exact
    np.testing.assert_array_equal(dm.cpu().numpy(), m)
    np.testing.assert_array_equal(dv.cpu().numpy(), v)
    np.testing.assert_array_equal(dvar.cpu().numpy(), var)


@pytest.mark.parametrize("wd", [0.0, 0.01])
def test_sgd_distinct_exact_and_duplicates_within_tolerance(wd):
    rng = np.random.default_rng(7)
    rows, n, dim = 50000, 20000, 24
    var = rng.normal(0, 1, (rows, dim)).astype(np.float32)
    idx = rng.permutation(rows)[:n].astype(np.int32)
    idx[::29] = -1
    grad = rng.normal(0, 1, (n, dim)).astype(np.float32)
    dvar = torch.from_numpy(var).to(DEV)
    host.sgd(torch.from_numpy(grad).to(DEV), torch.from_numpy(idx).to(DEV), dvar, 0.05, wd)
    want = var.copy()
    oracle.sgd(grad, idx, want, 0.05, wd)
    np.testing.assert_array_equal(dvar.cpu().numpy(), want)
    # duplicates without weight decay: sums of the same terms in another order
    idx2 = rng.integers(0, 100, n).astype(np.int32)
    dvar = torch.from_numpy(var).to(DEV)
    host.sgd(torch.from_numpy(grad).to(DEV), torch.from_numpy(idx2).to(DEV), dvar, 0.05, 0.0)
    want = var.copy()
    oracle.sgd(grad, idx2, want, 0.05, 0.0)
    scale = np.abs(var).copy()
    np.add.at(scale, idx2, 0.05 * np.abs(grad))
    assert (np.abs(dvar.cpu().numpy() - want) <= 1e-6 * scale).all()
