"""The key-switch and rotation workloads at the headline configuration (N = 2^16, 24 limbs of 50-bit primes,
7 special primes, 3 digits), built the same way by the benchmark that times them and by the tests that check them.

Everything derives from a few seeded polynomials: operand p of the HMult batch is the seeded ciphertext plus p in
every coefficient of every limb, rotation key i is the seeded key plus i + 1.  The derived operands are formed on
the device (a Hw_modadd_scalar per limb) and, for the ones a test compares with the oracle, on the host as well.
"""
import numpy as np

import seeded

N, LIMBS = 65536, 24
CFG = (N, LIMBS, 50, 50, 3)
PAIRS, ROTATIONS = 16, 32


def seeded_key(primes):
    """One switch key: [digit][b|a][all Q limbs then the P limbs], uniform residues."""
    return np.concatenate([seeded.uniform_poly(2000 + i, primes, N) for i in range(6)])


def seeded_ciphertexts(primes, level):
    """Four polynomials of `level` limbs: (a0, a1, b0, b1) of the HMult, (c0, c1) = the first two for rotations."""
    return [seeded.uniform_poly(3000 + i, primes[:level], N) for i in range(4)]


def shifted_host(x, shift, primes):
    """x + shift in every coefficient, limb t modulo primes[t]."""
    limbs = x.reshape(len(primes), -1)
    q = np.asarray(primes, np.int64)[:, None]
    return ((limbs + np.int64(shift)) % q).ravel()


def shifted_device(g, dst, dst_off, src, shift, prime_idx):
    """The same on the device: limb t of src plus shift into dst at dst_off, limb by limb."""
    n = g.N
    for t, pi in enumerate(prime_idx):
        g.hw("modadd_scalar", dst.view(dst_off + t * n, n), src.view(t * n, n), shift, pi)


def hmult_operands(g, cts, level, pairs, stride):
    """Four device buffers of `pairs` operands `stride` words apart: operand p = seeded ciphertext + p."""
    ops = [g.alloc(pairs * stride) for _ in range(4)]
    for k in range(4):
        for p in range(pairs):
            shifted_device(g, ops[k], p * stride, cts[k], p, range(level))
    return ops


def rotation_indices():
    """32 distinct rotation amounts: 2^0 .. 2^14, -1, and 16 seeded ones in [1, N/2)."""
    rots = [1 << i for i in range(15)] + [-1] + [int(v) for v in 1 + seeded.splitmix64(7, 16) % np.uint64(N // 2 - 1)]
    assert len(set(rots)) == ROTATIONS
    return rots


def key_prime_idx(g):
    """Prime of every limb of a switch key, in storage order."""
    T = g.L + g.K
    return [t for _ in range(2 * g.parts) for t in range(T)]


def rotation_keys(g, swk, count):
    """`count` device keys: key i = seeded key + (i + 1)."""
    idx = key_prime_idx(g)
    keys = []
    for i in range(count):
        k = g.alloc(swk.n)
        shifted_device(g, k, 0, swk, i + 1, idx)
        keys.append(k)
    return keys


def rotation_key_host(g, swk_host, i):
    return shifted_host(swk_host, i + 1, [g.primes[t] for t in key_prime_idx(g)])
