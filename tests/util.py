"""Seeded synthetic inputs shared by the parity tests (numpy PCG64 only)."""
import numpy as np

MASK64 = (1 << 64) - 1


def splitmix64(x):
    """Vectorised splitmix64 finaliser on uint64 arrays; returns int64 keys."""
    x = np.asarray(x, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = x + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z.view(np.int64)


def zipf_ranks(rng, alpha, support, size):
    """Zipf(alpha) ranks on the finite support [0, support) by inverse CDF."""
    w = 1.0 / np.power(np.arange(1, support + 1, dtype=np.float64), alpha)
    cdf = np.cumsum(w)
    cdf /= cdf[-1]
    return np.searchsorted(cdf, rng.random(size), side="left").astype(np.int64)


def zipf_keys(rng, alpha, support, size, table=0):
    """Zipf ranks hashed to 64-bit ids (table id folded into the top byte before hashing)."""
    r = zipf_ranks(rng, alpha, support, size).astype(np.uint64)
    return splitmix64(r ^ (np.uint64(table) << np.uint64(56)))
