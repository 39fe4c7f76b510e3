"""Pins the oracle's batch-ingestion restatement (ReadEmbKeyV2) and padding mask against plain numpy slicing / np.isin."""
import numpy as np
import pytest

import oracle


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
@pytest.mark.parametrize("with_ts", [False, True])
def test_read_emb_key_is_slicing(dtype, with_ts):
    rng = np.random.default_rng(3)
    splits = np.array([5, 0, 17, 1, 300, 64], dtype=np.int64)
    used = np.array([1, 1, 0, 1, 1, 0], dtype=np.uint8)
    body = rng.integers(-2**31, 2**31 - 1, int(splits.sum())).astype(dtype)
    if with_ts:
        if dtype == np.int64:
            data = np.concatenate([[1_700_000_000], body]).astype(dtype)
            want_ts = 1_700_000_000
        else:
            # the time is read as 8 bytes from the start of the tensor while keys start at element 1
            data = np.concatenate([[123456], body]).astype(dtype)
            want_ts = int(data[:2].view(np.int64)[0])
            if want_ts <= 0:
                data[1] = abs(int(data[1])) or 1
                body = data[1:]
                want_ts = int(data[:2].view(np.int64)[0])
    else:
        data = body
        want_ts = -1
    for tu in (None, used):
        sample, offsets, ts = oracle.read_emb_key(data, splits, tu, with_ts)
        bounds = np.concatenate([[0], np.cumsum(splits)])
        pieces = [body[bounds[i]:bounds[i + 1]].astype(np.int64) for i in range(splits.size)
                  if tu is None or tu[i]]
        np.testing.assert_array_equal(sample, np.concatenate(pieces))
        np.testing.assert_array_equal(offsets, np.concatenate([[0], np.cumsum([p.size for p in pieces])]))
        assert ts == want_ts


def test_timestamp_checks():
    splits = np.array([3, 2], dtype=np.int64)
    with pytest.raises(ValueError, match="not found"):
        oracle.read_emb_key(np.arange(5, dtype=np.int64), splits, None, True)          # no extra element
    with pytest.raises(ValueError, match="greater than 0"):
        oracle.read_emb_key(np.array([0, 1, 2, 3, 4, 5], dtype=np.int64), splits, None, True)
    with pytest.raises(ValueError, match="greater than 0"):
        oracle.read_emb_key(np.array([-7, 1, 2, 3, 4, 5], dtype=np.int64), splits, None, True)


def test_padding_mask_is_isin():
    rng = np.random.default_rng(5)
    values = rng.integers(0, 50, 1000).astype(np.int64)
    for pad in ([], [7], [0, 49, 13, 999]):
        want = 1 - np.isin(values, np.array(pad, dtype=np.int64)).astype(np.int32)
        np.testing.assert_array_equal(oracle.padding_keys_mask(values, pad), want)
