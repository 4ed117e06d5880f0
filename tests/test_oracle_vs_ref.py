"""Oracle vs. the reference's own compiled hot-path functions (oracle/_ref/ref_driver).

Skipped where the driver was not built (it needs the reference tree at build
time); the committed fixtures under tests/golden cover that case.
"""
import numpy as np
import pytest

import refdrv
import seeded
from oracle_lib import Oracle
from refdrv import RefSession

pytestmark = pytest.mark.skipif(not refdrv.available(), reason="compiled reference not built")

CONFIGS = [
    (16, 10, 60, 59, 3),     # ring degree 16 hits the reference's hard-coded root table
    (64, 7, 45, 40, 3),
    (64, 6, 50, 50, 2),      # last digit shorter than the others at lower levels
    (8192, 5, 40, 40, 3),    # Gemm configuration
]


def run_config(cfg, levels, heavy=True):
    N, nq, q0, sf, parts = cfg
    o = Oracle(*cfg)
    s = RefSession(*cfg)
    exp = []

    def q(code, want, *a):
        s.add(code, *a)
        exp.append(np.asarray(want).ravel())

    L, K = o.L, o.K
    allidx = list(range(L + K))
    x = seeded.uniform_poly(1, o.primes, N)
    q(refdrv.OP_NTT, o.ntt(x, allidx), L + K, 0, 0, 0, np.array(allidx), x)
    q(refdrv.OP_INTT, o.intt(x, allidx), L + K, 0, 0, 0, np.array(allidx), x)
    for pi in (0, L - 1, L, L + K - 1):
        tw = np.concatenate([o.twiddles(pi, k).astype(np.int64) for k in range(4)])
        s.add(refdrv.OP_TWIDDLES, pi)
        exp.append(tw)  # compared without the trailing ninv pair
    for pi in (0, L + K - 1):
        pq = o.primes[pi]
        a = seeded.uniform_limb(10 + pi, pq, N)
        b = seeded.uniform_limb(20 + pi, pq, N)
        r = seeded.uniform_limb(30 + pi, pq, N)
        sc = int(seeded.uniform_limb(40 + pi, pq, 1)[0])
        for name, code in refdrv.HW_OPS.items():
            if name == "rotate":
                k = o.find_automorphism_index(3)
                order = o.automorphism_order(k, True)
                q(refdrv.OP_HW, o.hw(name, a, order, pi), code, pi, N, 0, r, a, order)
            elif name.endswith("_scalar"):
                q(refdrv.OP_HW, o.hw(name, a, sc, pi, r=r), code, pi, N, 0, r, a, np.full(N, sc))
            else:
                q(refdrv.OP_HW, o.hw(name, a, b, pi, r=r), code, pi, N, 0, r, a, b)
    for rot in (1, 2, -1, -5, N // 2 - 1, 2 * N - 1):
        k = o.find_automorphism_index(rot)
        q(refdrv.OP_AUTO_INDEX, [k], rot)
        q(refdrv.OP_AUTO_ORDER, o.automorphism_order(k, True), k, 1)
        q(refdrv.OP_AUTO_ORDER, o.automorphism_order(k, False), k, 0)
    phat_inv, phat, pinv, pmod = o.tbl_moddown()
    q(refdrv.OP_TBL_MODDOWN, np.concatenate([phat_inv, phat.ravel(), pinv, pmod]))
    for level in levels:
        pr_q = o.primes[:level]
        pr_qp = [o.primes[i] for i in o.limb_primes(level)]
        nd = o.num_decomp(level)
        for part in range(nd):
            hat_inv, hat, cidx = o.tbl_modup(level, part)
            want = np.concatenate([[len(hat_inv), len(cidx)], hat_inv, hat.ravel(), [o.primes[j] for j in cidx]])
            q(refdrv.OP_TBL_MODUP, want, level, part)
        if level >= 2:
            a, b = o.tbl_rescale(level)
            q(refdrv.OP_TBL_RESCALE, np.concatenate([a, b]), level)
        if not heavy:
            continue
        c = seeded.uniform_poly(100 + level, pr_q, N)
        for is_ntt in (1, 0):
            for part in range(nd):
                q(refdrv.OP_DECOMP_MODUP, o.decomp_modup(c, level, part, is_ntt), level, part, is_ntt, 0, c)
                q(refdrv.OP_MOD_UP, o.decomp_modup(c, level, part, is_ntt), level, part, is_ntt, 0, c)
            q(refdrv.OP_PRECOMP, o.precomp(c, level, is_ntt, True), level, is_ntt, 1, 0, c)
            q(refdrv.OP_PRECOMP, o.precomp(c, level, is_ntt, False), level, is_ntt, 0, 0, c)
            e = seeded.uniform_poly(200 + level, pr_qp, N)
            q(refdrv.OP_MOD_DOWN, o.mod_down(e, level, is_ntt), level, is_ntt, 0, 0, e)
            if level >= 2:
                q(refdrv.OP_RESCALE, o.rescale(c, level, is_ntt), level, is_ntt, 0, 0, c)
                out, left = o.mod_down_rescale(e, level, is_ntt)
                q(refdrv.OP_MOD_DOWN_RESCALE, np.concatenate([out, left, [1]]), level, is_ntt, 0, 0, e)
                res_, raised, left = o.reduce_rescale_modup(e, level, is_ntt)
                q(refdrv.OP_REDUCE_RESCALE_MODUP, np.concatenate([res_, raised, left]), level, is_ntt, 0, 0, e)
        q(refdrv.OP_FROM_LEVEL0, o.transform_from_level0(c[:N], level), level, 0, 0, 0, c[:N])
        q(refdrv.OP_EXTEND, o.extend(c, level), level, 0, 0, 0, c)
        digits = np.concatenate([seeded.uniform_poly(300 + d, pr_qp, N) for d in range(nd)])
        key = np.concatenate([seeded.uniform_poly(400 + d, o.primes, N) for d in range(nd)])
        for fast in (0, 1):
            q(refdrv.OP_DOT_PROD, o.dot_prod(digits, key, nd, level, fast), level, nd, fast, 0, digits, key)
        k = o.find_automorphism_index(7)
        e = seeded.uniform_poly(500 + level, pr_qp, N)
        for is_ntt in (1, 0):
            order = o.automorphism_order(k, is_ntt)
            want = np.concatenate([o.hw("rotate", e[t * N:(t + 1) * N], order, pi) for t, pi in enumerate(o.limb_primes(level))])
            q(refdrv.OP_AUTOMORPHISM, want, level, 1, is_ntt, 0, e, order)
        e2 = seeded.uniform_poly(600 + level, pr_qp, N)
        for w, name in enumerate(("add", "sub", "mul")):
            q(refdrv.OP_POLY, o.poly(name, e, e2, level, True), w, level, 1, 0, e, e2)
    info, res = s.run()
    assert info["primes"] == o.primes
    assert info["roots"] == o.roots
    assert (info["L"], info["K"], info["part_size"]) == (o.L, o.K, o.part_size)
    mods = np.array([o.modulus(i) for i in range(L + K)], dtype=np.uint64).astype(np.int64)
    assert (info["modulus"] == mods).all()
    for i, (got, want) in enumerate(zip(res, exp)):
        want = np.asarray(want, dtype=np.int64)
        got = got[: want.size] if s.ops[i][0][0] == refdrv.OP_TWIDDLES else got
        assert got.size == want.size, "op %d (code %d): size" % (i, s.ops[i][0][0])
        assert (got == want).all(), "op %d (code %d, args %s) differs" % (i, s.ops[i][0][0], s.ops[i][0][1:5])
    o.close()


@pytest.mark.parametrize("cfg", CONFIGS[:3])
def test_small_rings_all_levels(cfg):
    run_config(cfg, list(range(1, cfg[1] + 1)))


def test_gemm_config():
    run_config(CONFIGS[3], [5, 4, 2, 1])


def test_headline_config_tables_and_one_keyswitch():
    """N=2^16, 24x50-bit, dnum=3 (k=7): context, all tables, and one full-size pass of each poly op."""
    cfg = (65536, 24, 50, 50, 3)
    run_config(cfg, list(range(1, 25)), heavy=False)
    N = cfg[0]
    o = Oracle(*cfg)
    s = RefSession(*cfg)
    level = 24
    c = seeded.uniform_poly(1, o.primes[:level], N)
    e = seeded.uniform_poly(2, [o.primes[i] for i in o.limb_primes(level)], N)
    s.add(refdrv.OP_DECOMP_MODUP, level, 2, 1, 0, c)
    s.add(refdrv.OP_MOD_DOWN, level, 1, 0, 0, e)
    s.add(refdrv.OP_RESCALE, level, 1, 0, 0, c)
    info, res = s.run()
    assert (res[0] == o.decomp_modup(c, level, 2, True)).all()
    assert (res[1] == o.mod_down(e, level, True)).all()
    assert (res[2] == o.rescale(c, level, True)).all()
    o.close()


def test_mod_down_rescale_with_a_small_first_prime():
    """q_0 of 40 bits under 50-bit scaling primes: the last-limb value exceeds q_0, so Sub_mul_const_mod's
    difference stays negative after its single +q and the reference's casts decide the result."""
    cfg = (64, 4, 40, 50, 2)
    N = cfg[0]
    o = Oracle(*cfg)
    s = RefSession(*cfg)
    want = []
    for level in (4, 3, 2):
        e = seeded.uniform_poly(7 + level, [o.primes[i] for i in o.limb_primes(level)], N)
        for is_ntt in (1, 0):
            out, left = o.mod_down_rescale(e, level, is_ntt)
            s.add(refdrv.OP_MOD_DOWN_RESCALE, level, is_ntt, 0, 0, e)
            want.append(np.concatenate([out, left, [1]]))
            res_, raised, left = o.reduce_rescale_modup(e, level, is_ntt)
            s.add(refdrv.OP_REDUCE_RESCALE_MODUP, level, is_ntt, 0, 0, e)
            want.append(np.concatenate([res_, raised, left]))
    _, res = s.run()
    for got, w in zip(res, want):
        assert np.array_equal(got, w)
    o.close()
