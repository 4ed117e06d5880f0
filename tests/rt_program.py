"""Builds the input file of tests/programs/keyswitch_program and the oracle's expectation for its outputs."""
import os
import subprocess

import numpy as np

import seeded

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAM = os.path.join(ROOT, "tests", "programs", "keyswitch_program")


def make_inputs(o, cfg, rots, seed):
    """cfg = (N, num_q, q0_bits, sf_bits, parts); returns (file bytes, dict of the arrays)."""
    N, num_q, q0_bits, sf_bits, parts = cfg
    L, K = o.L, o.K
    assert L == num_q

    def key(s):
        return np.concatenate([seeded.uniform_poly(s + i, o.primes, N) for i in range(2 * parts)])

    relin = key(seed + 100)
    rot_keys = [key(seed + 200 + 10 * i) for i in range(len(rots))]
    c0 = seeded.uniform_poly(seed + 1, o.primes[:L], N)
    c1 = seeded.uniform_poly(seed + 2, o.primes[:L], N)
    head = np.array([N, num_q - 1, q0_bits, sf_bits, parts, len(rots)] + list(rots), dtype=np.int64)
    blob = b"".join(a.astype("<i8").tobytes() for a in [head, relin] + rot_keys + [c0, c1])
    return blob, dict(relin=relin, rot_keys=rot_keys, c0=c0, c1=c1)


def expected_outputs(o, data, rots):
    """What the program must write, from the oracle: [(level, c0, c1)] in output order."""
    L = o.L
    m0, m1 = o.mul_relin_rescale(data["c0"], data["c1"], data["c0"], data["c1"], data["relin"], L)
    level = L - 1
    digits = o.precomp(m1, level, True)
    rot = []
    for r, k in zip(rots, data["rot_keys"]):
        order = o.automorphism_order(o.find_automorphism_index(r), True)
        rot.append((level,) + tuple(o.fast_rotate(m0, digits, k, order, level)))
    return [(level, m0, m1)] + rot + [(level, m0, m1)] + rot


def read_outputs(path, N):
    raw = np.fromfile(path, dtype="<i8")
    out, pos = [], 0
    while pos < raw.size:
        level = int(raw[pos])
        n = level * N
        out.append((level, raw[pos + 1:pos + 1 + n], raw[pos + 1 + n:pos + 1 + 2 * n]))
        pos += 1 + 2 * n
    return out


def run_program(in_path, out_path, timeout=300):
    return subprocess.run([PROGRAM, in_path, out_path], capture_output=True, text=True, timeout=timeout)
