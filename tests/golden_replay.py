"""Replays the golden fixture plan (tests/golden) through any implementation.

An implementation is an object with ntt/intt/decomp_modup/mod_down/rescale/
dot_prod/find_automorphism_index taking and returning numpy int64 arrays (the
oracle binding already has that shape; the GPU adapter below wraps the C-ABI).
"""
import hashlib
import json
import os

import numpy as np

import refdrv
from golden.make_golden import CONFIGS, plan

HERE = os.path.dirname(os.path.abspath(__file__))


def load():
    meta = json.load(open(os.path.join(HERE, "golden", "golden.json")))
    vec = np.load(os.path.join(HERE, "golden", "small_ring_vectors.npz"))
    return meta, vec


def run_op(impl, code, args, arrays):
    if code in (refdrv.OP_NTT, refdrv.OP_INTT):
        idx, x = arrays
        return impl.ntt(x, list(idx)) if code == refdrv.OP_NTT else impl.intt(x, list(idx))
    if code == refdrv.OP_DECOMP_MODUP:
        return impl.decomp_modup(arrays[0], args[0], args[1], bool(args[2]))
    if code == refdrv.OP_MOD_DOWN:
        return impl.mod_down(arrays[0], args[0], bool(args[1]))
    if code == refdrv.OP_RESCALE:
        return impl.rescale(arrays[0], args[0], bool(args[1]))
    if code == refdrv.OP_MOD_DOWN_RESCALE:
        out, left = impl.mod_down_rescale(arrays[0], args[0], bool(args[1]))
        return np.concatenate([out, left, [1]])
    if code == refdrv.OP_REDUCE_RESCALE_MODUP:
        return np.concatenate(impl.reduce_rescale_modup(arrays[0], args[0], bool(args[1])))
    if code == refdrv.OP_FROM_LEVEL0:
        return impl.transform_from_level0(arrays[0], args[0])
    if code == refdrv.OP_DOT_PROD:
        return impl.dot_prod(arrays[0], arrays[1], args[1], args[0])
    if code == refdrv.OP_AUTO_INDEX:
        return np.array([impl.find_automorphism_index(args[0])], np.int64)
    raise ValueError(code)


def check(impl, name, meta, vec):
    entry = meta[name]
    assert impl.primes == entry["primes"], "prime chain differs from the reference's"
    assert impl.roots == entry["roots"], "2N-th roots differ from the reference's"
    assert (impl.L, impl.K, impl.part_size) == (entry["L"], entry["K"], entry["part_size"])
    info = {"K": entry["K"], "primes": entry["primes"], "part_size": entry["part_size"]}
    for opname, code, args, arrays in plan(tuple(entry["cfg"]), info):
        out = np.ascontiguousarray(run_op(impl, code, args, arrays), dtype=np.int64).ravel()
        g = entry["ops"][opname]
        assert out.size == g["n"], opname
        assert [int(v) for v in out[:4]] == g["head"], "%s/%s: leading words differ" % (name, opname)
        assert hashlib.sha256(out.tobytes()).hexdigest() == g["sha256"], "%s/%s: digest differs" % (name, opname)
        if name == "small":
            assert (out == vec[opname]).all(), opname


class GpuImpl:
    """numpy-in / numpy-out adapter over the C-ABI, shaped like the oracle binding."""

    def __init__(self, cfg):
        import acefhe
        self.g = acefhe.Context(*cfg)
        assert self.g.has_device
        for a in ("primes", "roots", "L", "K", "part_size", "N"):
            setattr(self, a, getattr(self.g, a))

    def close(self):
        self.g.close()

    def ntt(self, x, idx, inverse=False):
        d = self.g.upload(x)
        self.g.ntt(d, d, idx, inverse=inverse)
        out = d.get()
        d.free()
        return out

    def intt(self, x, idx):
        return self.ntt(x, idx, inverse=True)

    def _unary(self, fn, x, n_out, *a):
        d, r = self.g.upload(x), self.g.alloc(n_out)
        fn(r, d, *a)
        out = r.get()
        d.free()
        r.free()
        return out

    def decomp_modup(self, x, level, part, is_ntt):
        return self._unary(self.g.decomp_modup, x, (level + self.K) * self.N, level, part, is_ntt)

    def mod_down(self, x, level, is_ntt):
        return self._unary(self.g.mod_down, x, level * self.N, level, is_ntt)

    def rescale(self, x, level, is_ntt):
        return self._unary(self.g.rescale, x, (level - 1) * self.N, level, is_ntt)

    def mod_down_rescale(self, x, level, is_ntt):
        d, r = self.g.upload(x), self.g.alloc((level - 1) * self.N)
        self.g.mod_down_rescale(r, d, level, is_ntt)
        out = r.get(), d.get()
        d.free()
        r.free()
        return out

    def reduce_rescale_modup(self, x, level, is_ntt):
        nd = self.g.num_decomp(level - 1)
        d, r, up = self.g.upload(x), self.g.alloc(level * self.N), self.g.alloc(nd * (level - 1 + self.K) * self.N)
        self.g.reduce_rescale_modup(r, up, d, level, is_ntt)
        out = r.get(), up.get(), d.get()
        for b in (d, r, up):
            b.free()
        return out

    def transform_from_level0(self, x, level):
        return self._unary(self.g.transform_from_level0, x, level * self.N, level)

    def dot_prod(self, digits, key, n_parts, level):
        dd, dk, r = self.g.upload(digits), self.g.upload(key), self.g.alloc((level + self.K) * self.N)
        self.g.dot_prod(r, dd, dk, key.size // n_parts, n_parts, level)
        out = r.get()
        for b in (dd, dk, r):
            b.free()
        return out

    def find_automorphism_index(self, rot):
        return self.g.find_automorphism_index(rot)
