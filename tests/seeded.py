"""Seeded input generator shared by every parity test and the benchmark.

splitmix64 (Steele/Lea/Flood) over a counter; residues are drawn as
hi64(x * q), i.e. floor(x*q / 2^64), which is uniform on [0, q) up to 2^-64.
"""
import numpy as np

_M = (1 << 64) - 1


def splitmix64(seed, n):
    """n consecutive outputs of splitmix64 started at `seed` (numpy uint64)."""
    with np.errstate(over="ignore"):
        z = (np.uint64(seed & _M) + np.arange(1, n + 1, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def _mulhi(x, q):
    q = np.uint64(q)
    m32 = np.uint64(0xFFFFFFFF)
    s32 = np.uint64(32)
    with np.errstate(over="ignore"):
        xl, xh = x & m32, x >> s32
        ql, qh = q & m32, q >> s32
        ll = xl * ql
        lh = xl * qh
        hl = xh * ql
        hh = xh * qh
        mid = (ll >> s32) + (lh & m32) + (hl & m32)
        return hh + (lh >> s32) + (hl >> s32) + (mid >> s32)


def uniform_limb(seed, q, n):
    """n residues uniform in [0, q), int64."""
    return _mulhi(splitmix64(seed, n), q).astype(np.int64)


def uniform_poly(seed, primes, n):
    """limb-major polynomial: limb t uniform mod primes[t], seeded by (seed, t)."""
    return np.concatenate([uniform_limb(seed * 1000003 + t * 7919 + 1, q, n) for t, q in enumerate(primes)])
