#!/usr/bin/env python3
"""Writes the golden fixtures of tests/golden from the reference's own compiled code.

Run in a container that has the reference tree (it drives oracle/_ref/ref_driver,
which `make -C oracle ref` links against the reference sources).  Inputs are
regenerated from the seeded generator in tests/seeded.py, so only outputs are
stored: full vectors for a small ring, SHA-256 digests plus the leading words
for the Gemm (N=8192) and headline (N=65536, 24x50-bit, dnum 3) configurations.

    python tests/golden/make_golden.py
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))

import refdrv  # noqa: E402
import seeded  # noqa: E402
from refdrv import RefSession  # noqa: E402

CONFIGS = {"small": (64, 7, 45, 40, 3), "gemm": (8192, 5, 40, 40, 3), "headline": (65536, 24, 50, 50, 3)}


def plan(cfg, info):
    """The list of (name, opcode, args, input arrays) every consumer of the fixtures replays."""
    N, L = cfg[0], cfg[1]
    K, primes = info["K"], info["primes"]
    ops = []
    allidx = list(range(L + K))
    x = seeded.uniform_poly(1, primes, N)
    ops.append(("ntt_all", refdrv.OP_NTT, (L + K, 0, 0, 0), [np.array(allidx), x]))
    ops.append(("intt_all", refdrv.OP_INTT, (L + K, 0, 0, 0), [np.array(allidx), x]))
    for level in sorted({L, max(2, L - 2)}):
        qp = [primes[i] for i in list(range(level)) + [L + j for j in range(K)]]
        c = seeded.uniform_poly(100 + level, primes[:level], N)
        e = seeded.uniform_poly(200 + level, qp, N)
        nd = -(-level // info["part_size"])
        nd = min(nd, cfg[4])
        for part in range(nd):
            ops.append(("decomp_modup_l%d_p%d" % (level, part), refdrv.OP_DECOMP_MODUP, (level, part, 1, 0), [c]))
        ops.append(("decomp_modup_coef_l%d_p0" % level, refdrv.OP_DECOMP_MODUP, (level, 0, 0, 0), [c]))
        ops.append(("mod_down_l%d" % level, refdrv.OP_MOD_DOWN, (level, 1, 0, 0), [e]))
        ops.append(("mod_down_coef_l%d" % level, refdrv.OP_MOD_DOWN, (level, 0, 0, 0), [e]))
        ops.append(("rescale_l%d" % level, refdrv.OP_RESCALE, (level, 1, 0, 0), [c]))
        ops.append(("rescale_coef_l%d" % level, refdrv.OP_RESCALE, (level, 0, 0, 0), [c]))
        # output, then the operand as the call leaves it (coefficient form), then the result's NTT flag
        ops.append(("mod_down_rescale_l%d" % level, refdrv.OP_MOD_DOWN_RESCALE, (level, 1, 0, 0), [e]))
        ops.append(("mod_down_rescale_coef_l%d" % level, refdrv.OP_MOD_DOWN_RESCALE, (level, 0, 0, 0), [e]))
        # res as left by the call, the raised digits, the operand afterwards
        ops.append(("reduce_rescale_modup_l%d" % level, refdrv.OP_REDUCE_RESCALE_MODUP, (level, 1, 0, 0), [e]))
        ops.append(("from_level0_l%d" % level, refdrv.OP_FROM_LEVEL0, (level, 0, 0, 0), [c[:N]]))
        digits = np.concatenate([seeded.uniform_poly(300 + d, qp, N) for d in range(nd)])
        key = np.concatenate([seeded.uniform_poly(400 + d, primes, N) for d in range(nd)])
        ops.append(("dot_prod_l%d" % level, refdrv.OP_DOT_PROD, (level, nd, 0, 0), [digits, key]))
    for rot in (1, -1, 7):
        ops.append(("auto_index_%d" % rot, refdrv.OP_AUTO_INDEX, (rot, 0, 0, 0), []))
    return ops


def context_info(cfg):
    info, _ = RefSession(*cfg).run()
    return info


def main():
    if not refdrv.available():
        sys.exit("oracle/_ref/ref_driver is not built (needs the reference tree): make -C oracle ref")
    meta = {}
    full = {}
    for name, cfg in CONFIGS.items():
        info = context_info(cfg)
        ops = plan(cfg, info)
        s = RefSession(*cfg)
        for _, code, args, arrays in ops:
            s.add(code, *args, *arrays)
        info, res = s.run()
        entry = {"cfg": list(cfg), "L": info["L"], "K": info["K"], "part_size": info["part_size"],
                 "primes": info["primes"], "roots": info["roots"], "ops": {}}
        for (opname, _, _, _), out in zip(ops, res):
            entry["ops"][opname] = {"n": int(out.size), "sha256": hashlib.sha256(out.tobytes()).hexdigest(),
                                    "head": [int(v) for v in out[:4]]}
            if name == "small":
                full[opname] = out
        meta[name] = entry
    with open(os.path.join(HERE, "golden.json"), "w") as f:
        json.dump(meta, f, indent=1)
    np.savez_compressed(os.path.join(HERE, "small_ring_vectors.npz"), **full)
    print("wrote golden.json (%d configs) and small_ring_vectors.npz (%d vectors)" % (len(meta), len(full)))


if __name__ == "__main__":
    main()
