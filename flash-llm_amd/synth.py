"""Seeded synthetic operands for the SpMM tests and benchmark.

Counter-based (splitmix64 of seed, stream and element index), so any row
block can be generated on its own and in parallel, and the same seed gives the
same bits everywhere.  Shapes and distributions follow the reference's
benchmark operands (kernel_benchmark/spmm_test_utils.h:103-118: Bernoulli
keep-mask on A, B dense) with real-valued nonzeros instead of its all-ones A.
"""
from concurrent.futures import ThreadPoolExecutor

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(x):
    with np.errstate(over="ignore"):
        z = x + _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def _key(seed, stream):
    return _mix(_mix(np.uint64(seed)) ^ np.uint64(stream))


def uniform01_at(seed, stream, idx):
    """float64 in [0,1) for the element indices in idx (uint64 array)."""
    with np.errstate(over="ignore"):
        z = _mix(idx * _GOLDEN + _key(seed, stream))
    return (z >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def uniform01(seed, stream, start, count):
    """float64 in [0,1) for element indices start .. start+count-1."""
    return uniform01_at(seed, stream, np.arange(start, start + count, dtype=np.uint64))


def _values_at(seed, stream, idx, dist, sigma):
    """The value of every element index in idx: a function of (seed, stream, index) alone."""
    if dist == "uniform":  # U[-1, 1]
        return uniform01_at(seed, stream, idx) * 2.0 - 1.0
    if dist == "normal":  # Box-Muller
        u1 = uniform01_at(seed, stream, idx)
        u2 = uniform01_at(seed, stream + 1, idx)
        return sigma * np.sqrt(-2.0 * np.log1p(-u1)) * np.cos(2.0 * np.pi * u2)
    if dist == "ones":  # the reference's own test data
        return np.ones(idx.size)
    raise ValueError(dist)


def _values(seed, stream, start, count, dist, sigma):
    return _values_at(seed, stream, np.arange(start, start + count, dtype=np.uint64), dist, sigma)


def row_keep_ratio(m, seed, mean=0.2):
    """Per-row keep probability ~ Beta(2, 8) (second smallest of nine uniforms),
    rescaled so that the mean over the rows is `mean`."""
    u = uniform01(seed, 7, 0, m * 9).reshape(m, 9)
    p = np.sort(u, axis=1)[:, 1]
    return np.clip(p * (mean / p.mean()), 0.0, 1.0)


def sparse_matrix(m, k, sparsity, seed, dist="uniform", sigma=0.02, row_beta=False, threads=8):
    """Row-major (m, k) float16 with an unstructured Bernoulli keep-mask."""
    out = np.empty((m, k), dtype=np.float16)
    keep_row = row_keep_ratio(m, seed, 1.0 - sparsity) if row_beta else None
    step = max(1, (1 << 22) // k)

    def block(r0):
        r1 = min(m, r0 + step)
        n = (r1 - r0) * k
        u = uniform01(seed, 3, r0 * k, n)
        if keep_row is None:
            keep = u < (1.0 - sparsity)
        else:
            keep = u.reshape(r1 - r0, k) < keep_row[r0:r1, None]
            keep = keep.reshape(-1)
        # values only where the mask keeps them: an element's value depends on its index alone
        kept = np.flatnonzero(keep)
        blk = np.zeros(n, dtype=np.float16)
        blk[kept] = _values_at(seed, 1, kept.astype(np.uint64) + np.uint64(r0 * k), dist, sigma).astype(np.float16)
        out[r0:r1] = blk.reshape(r1 - r0, k)

    starts = list(range(0, m, step))
    if threads > 1 and len(starts) > 1:
        with ThreadPoolExecutor(threads) as pool:
            list(pool.map(block, starts))
    else:
        for r0 in starts:
            block(r0)
    return out


def dense_b(k, n, seed, dist="uniform", sigma=1.0):
    """Column-major K x N activations, returned as an (n, k) float16 array."""
    return _values(seed, 11, 0, n * k, dist, sigma).astype(np.float16).reshape(n, k)
