"""Runs the compiled reference (oracle/_ref/ref_driver) on harness inputs.  Test infrastructure."""
import os
import subprocess
import tempfile

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "oracle", "_ref", "ref_driver")

(OP_NTT, OP_INTT, OP_HW, OP_DECOMP_MODUP, OP_PRECOMP, OP_MOD_DOWN, OP_RESCALE, OP_DOT_PROD,
 OP_AUTO_ORDER, OP_AUTO_INDEX, OP_AUTOMORPHISM, OP_EXTEND, OP_TBL_MODUP, OP_TBL_MODDOWN,
 OP_TBL_RESCALE, OP_POLY, OP_TWIDDLES, OP_MOD_UP, OP_MOD_DOWN_RESCALE, OP_REDUCE_RESCALE_MODUP,
 OP_FROM_LEVEL0, OP_ENCODE, OP_DECODE, OP_EMBEDDING, OP_TIME_NTT, OP_ENCODE_SCALED, OP_TIME_KEYSWITCH,
 OP_TIME_PRIMITIVES) = range(1, 29)

HW_OPS = {"modadd": 0, "modsub": 1, "modmul": 2, "modmuladd": 3, "modadd_scalar": 4,
          "modsub_scalar": 5, "modmul_scalar": 6, "modmuladd_scalar": 7, "rotate": 8}


def available():
    return os.path.exists(DRIVER) and os.path.exists("/opt/conda/lib/libgmp.so.10")


class RefSession:
    """Collects ops, runs them in one driver process, returns the outputs in order."""

    def __init__(self, degree, num_q, q0_bits, sf_bits, parts):
        self.hdr = [degree, num_q, q0_bits, sf_bits, parts]
        self.ops = []

    def add(self, code, a1=0, a2=0, a3=0, a4=0, *arrays):
        data = [np.ascontiguousarray(a, dtype=np.int64).ravel() for a in arrays]
        n = sum(d.size for d in data)
        self.ops.append((np.array([code, a1, a2, a3, a4, n], np.int64), data))
        return len(self.ops) - 1

    def run(self):
        with tempfile.TemporaryDirectory() as td:
            req, resp = os.path.join(td, "req.bin"), os.path.join(td, "resp.bin")
            with open(req, "wb") as f:
                np.array(self.hdr + [len(self.ops)], np.int64).tofile(f)
                for h, data in self.ops:
                    h.tofile(f)
                    for d in data:
                        d.tofile(f)
            subprocess.check_call([DRIVER, req, resp])
            out = np.fromfile(resp, dtype=np.int64)
        L, K, ps = (int(x) for x in out[:3])
        pos = 3
        T = L + K
        info = {"L": L, "K": K, "part_size": ps,
                "primes": [int(x) for x in out[pos:pos + T]],
                "roots": [int(x) for x in out[pos + T:pos + 2 * T]],
                "modulus": out[pos + 2 * T:pos + 7 * T].reshape(T, 5).copy()}
        pos += 7 * T
        res = []
        for _ in self.ops:
            n = int(out[pos])
            res.append(out[pos + 1:pos + 1 + n].copy())
            pos += 1 + n
        assert pos == out.size
        return info, res
