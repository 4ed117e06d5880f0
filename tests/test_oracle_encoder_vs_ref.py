"""Encoder of the oracle vs. the reference's compiled encoder (embedding, encode, decode), bit for bit:
the floating-point steps are the same IEEE operations in the same order, so the doubles agree exactly."""
import numpy as np
import pytest

import refdrv
import seeded
from oracle_lib import Oracle
from refdrv import RefSession

pytestmark = pytest.mark.skipif(not refdrv.available(), reason="compiled reference not built")

CONFIGS = [(64, 4, 50, 40, 2), (1024, 5, 45, 40, 3), (8192, 5, 40, 40, 3), (16384, 4, 60, 50, 2)]


def bits(a):
    return np.ascontiguousarray(a).view(np.int64).ravel()


@pytest.mark.parametrize("cfg", CONFIGS, ids=lambda c: "N%d_L%d" % (c[0], c[1]))
def test_embedding_encode_decode(cfg):
    N = cfg[0]
    o = Oracle(*cfg)
    s = RefSession(*cfg)
    rng = np.random.default_rng(cfg[0])
    want = []
    for slots in sorted({N // 2, max(1, N // 8), 4, 1}):
        z = rng.uniform(-1, 1, slots) + 1j * rng.uniform(-1, 1, slots)
        for inv in (0, 1):
            s.add(refdrv.OP_EMBEDDING, inv, 0, 0, 0, bits(z))
            want.append(bits(o.embedding(z, bool(inv))))
        for level, deg, pc in ((o.L, 1, 0), (2, 1, 0), (o.L, 2, 0), (o.L, 3, 0), (o.L - 1, 1, o.K)):
            if deg * cfg[3] >= cfg[2] + (level - 1) * cfg[3]:
                continue  # the reference asserts: scaling factor too large for the level
            n_val = max(1, slots - 1)  # a vector shorter than the slot count is zero-padded
            zz = z[:n_val] * 3.0
            s.add(refdrv.OP_ENCODE, level, slots, deg, pc, bits(zz))
            pt = o.encode(zz, slots, level, deg, pc)
            assert pt is not None
            sc = float(2 ** cfg[3]) ** deg
            want.append(np.concatenate([pt, [slots, deg], bits(np.array([sc]))]))
            if pc == 0:
                for is_ntt in (1, 0):
                    poly = pt if is_ntt else o.intt(pt, list(range(level)))
                    s.add(refdrv.OP_DECODE, level, slots, is_ntt, int(bits(np.array([sc]))[0]), poly)
                    dec = o.decode(poly, level, slots, sc, bool(is_ntt))
                    want.append(bits(dec))
                    assert np.abs(dec[:n_val] - zz).max() < 1e-6
        # an explicit scale that is no power of the scaling factor (Encode_at_level_with_scale), with and without P limbs
        for level, scale, pc in ((o.L, 1.5 * 2.0 ** cfg[3], 0), (2, 2.0 ** (cfg[3] - 7) * 1.1, 0), (o.L, 1.25 * 2.0 ** (cfg[3] + 5), o.K)):
            if np.log2(scale) + 3 >= cfg[2] + (level - 1) * cfg[3]:
                continue
            zz = z[:max(1, slots - 1)] * 3.0
            s.add(refdrv.OP_ENCODE_SCALED, level, slots, int(bits(np.array([scale]))[0]), pc, bits(zz))
            pt = o.encode_scaled(zz, slots, level, scale, pc)
            assert pt is not None
            deg = int(np.floor(np.log2(scale) / cfg[3]))
            deg += scale > float(2 ** cfg[3]) ** deg
            want.append(np.concatenate([pt, [slots, deg], bits(np.array([scale]))]))
    # decode of arbitrary residues: large centred values, both signs
    for level in (o.L, 3, 1):
        poly = seeded.uniform_poly(90 + level, o.primes[:level], N)
        s.add(refdrv.OP_DECODE, level, N // 2, 0, int(bits(np.array([2.0 ** 30]))[0]), poly)
        want.append(bits(o.decode(poly, level, N // 2, 2.0 ** 30, False)))
    _, res = s.run()
    assert len(res) == len(want)
    for i, (g, w) in enumerate(zip(res, want)):
        assert g.size == w.size, i
        assert np.array_equal(g, w), "op %d (code %d) differs in %d of %d words" % (
            i, s.ops[i][0][0], int((g != w).sum()), w.size)
    o.close()
