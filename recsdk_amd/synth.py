"""Deterministic synthetic inputs of the benchmark configurations (numpy PCG64 + splitmix64 only)."""
import numpy as np

GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def splitmix64(x):
    """Vectorised splitmix64 finaliser on uint64 arrays; returns int64 keys."""
    x = np.asarray(x, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = x + GOLDEN
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z.view(np.int64)


class ZipfSampler:
    """Zipf(alpha) ranks on the finite support [0, support) by inverse CDF."""

    def __init__(self, alpha, support):
        w = 1.0 / np.power(np.arange(1, support + 1, dtype=np.float64), alpha)
        self.cdf = np.cumsum(w)
        self.cdf /= self.cdf[-1]

    def ranks(self, rng, size):
        return np.searchsorted(self.cdf, rng.random(size), side="left").astype(np.int64)


def zipf_ranks(rng, alpha, support, size):
    return ZipfSampler(alpha, support).ranks(rng, size)


def ranks_to_keys(ranks, table=0):
    """64-bit ids: splitmix64(rank xor table<<56)."""
    return splitmix64(np.asarray(ranks).astype(np.uint64) ^ (np.uint64(table) << np.uint64(56)))


def zipf_keys(rng, alpha, support, size, table=0):
    return ranks_to_keys(zipf_ranks(rng, alpha, support, size), table)


def dlrm_table_rows(num_tables=26, total_rows=60_000_000, lo=1e3, hi=8e6, seed=1):
    """Row counts log-uniform in [lo, hi], rescaled so that they sum to about total_rows."""
    rng = np.random.default_rng(seed)
    rows = np.exp(rng.uniform(np.log(lo), np.log(hi), num_tables))
    rows = np.maximum(np.round(rows * (total_rows / rows.sum())), 16).astype(np.int64)
    return rows
