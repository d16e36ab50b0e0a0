"""Independent numpy restatement of the synthetic-input definitions.

TEST INFRASTRUCTURE ONLY.  Written separately from bam_oracle.c (vectorised,
different control flow) so that a slip in either shows up as a mismatch.
"""
import numpy as np

_G = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def splitmix64(seed, i):
    """i-th output of the SplitMix64 stream started at `seed` (i may be an array)."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + (np.asarray(i, dtype=np.uint64) + np.uint64(1)) * _G
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def rmat_edges(seed, scale, first, n):
    e = np.arange(first, first + n, dtype=np.uint64)
    u = np.zeros(n, dtype=np.uint64)
    v = np.zeros(n, dtype=np.uint64)
    t1 = np.uint64(int(0.57 * 2**32))
    t2 = t1 + np.uint64(int(0.19 * 2**32))
    t3 = t2 + np.uint64(int(0.19 * 2**32))
    for l in range(scale):
        x = splitmix64(seed, e * np.uint64(scale) + np.uint64(l)) >> np.uint64(32)
        q = (x >= t1).astype(np.uint64) + (x >= t2) + (x >= t3)
        u = (u << np.uint64(1)) | (q >> np.uint64(1))
        v = (v << np.uint64(1)) | (q & np.uint64(1))
    return u, v


def uniform_edges(seed, n_vertices, first, n):
    p = np.arange(first, first + n, dtype=np.uint64)
    return (splitmix64(seed, p * np.uint64(2)) % np.uint64(n_vertices),
            splitmix64(seed, p * np.uint64(2) + np.uint64(1)) % np.uint64(n_vertices))


def build_csr(n_vertices, u, v):
    keep = u != v
    u, v = u[keep], v[keep]
    a = np.concatenate([u, v])
    b = np.concatenate([v, u])
    pairs = np.unique(np.stack([a, b], axis=1), axis=0) if len(a) else np.zeros((0, 2), dtype=np.uint64)
    off = np.zeros(n_vertices + 1, dtype=np.uint64)
    np.add.at(off, pairs[:, 0].astype(np.int64) + 1, 1)
    return np.cumsum(off, dtype=np.uint64), pairs[:, 1].astype(np.uint64)
