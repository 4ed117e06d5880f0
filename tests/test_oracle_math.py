"""Oracle vs. what the mathematics fixes, with Python big integers.

Each check is chosen so that a plausible slip (wrong twiddle index, dropped
term, transposed table, wrong centring) fails it; none re-types the oracle's
own formula: the NTT is compared with direct polynomial evaluation, base
conversion with the textbook sum over big-integer cofactors, rescale with
rounded big-integer division, the tables with the reference's big-integer
recipes (util/src/crt.c:232-352, 459-566).
"""
import math

import numpy as np
import pytest

import seeded
from oracle_lib import Oracle, lib


def bitrev(i, w):
    return int(format(i, "0%db" % w)[::-1], 2) if w else 0


@pytest.fixture(scope="module")
def ctx():
    o = Oracle(64, 7, 45, 40, 3)
    yield o
    o.close()


def test_modular_closed_forms():
    L = lib()
    rng = np.random.default_rng(1)
    for q in (1099510824961, 1125899877875713, 1152921504606584833, 97):
        for _ in range(200):
            a, b = (int(x) for x in rng.integers(0, q, 2))
            assert L.orc_add_mod(a, b, q) == (a + b) % q
            assert L.orc_sub_mod(a, b, q) == (a - b) % q
            w = b
            wp = L.orc_precompute_const(w, q)
            assert wp == (w << 64) // q
            assert L.orc_fast_mul_const(a, w, wp, q) == a * w % q
    o = Oracle(4, 2, 60, 50, 1)
    for i in range(o.L + o.K):
        q = o.primes[i]
        m = o.modulus(i)
        # br_k uses a double-precision log2 (include/util/modular.h:69)
        assert m[0] == q and m[1] == 2 * (int(math.log2(float(q))) + 1) and m[2] == (1 << m[1]) // q
        assert m[3] + (m[4] << 64) == (1 << 128) // q
        for _ in range(200):
            a, b = (int(x) for x in rng.integers(0, q, 2))
            assert L.orc_mul_mod_barrett(o.h, i, a, b) == a * b % q
        assert L.orc_mul_mod_barrett(o.h, i, q - 1, q - 1) == 1
    o.close()


def test_switch_modulus_is_centred_lift():
    L = lib()
    rng = np.random.default_rng(2)
    for old, new in [(1125899877875713, 1125899935285249), (1125899935285249, 1125899877875713),
                     (1125899877875713, 1099510824961), (1099510824961, 1152921504606584833)]:
        for v in [0, 1, old // 2, old // 2 + 1, old - 1] + [int(x) for x in rng.integers(0, old, 100)]:
            centred = v - old if v > old // 2 else v
            assert L.orc_switch_modulus(v, old, new) == centred % new


def test_prime_generation_rules():
    # Appendix-style lists printed by the compiled reference (N=8192, 5x40 bit, 3 parts)
    o = Oracle(8192, 5, 40, 40, 3)
    assert o.primes == [1099510824961, 1099510890497, 1099512004609, 1099511480321, 1099511922689,
                        1152921504606830593, 1152921504606748673]
    assert (o.K, o.part_size) == (2, 2)
    o.close()
    o = Oracle(65536, 24, 50, 50, 3)
    assert o.K == 7 and o.part_size == 8
    assert o.primes[:4] == [1125899877875713, 1125899935285249, 1125899879710721, 1125899930959873]
    assert o.primes[20:24] == [1125899902124033, 1125899911168001, 1125899903827969, 1125899908022273]
    assert o.primes[24:] == [1152921504606584833, 1152921504598720513, 1152921504597016577, 1152921504595968001,
                             1152921504592822273, 1152921504592429057, 1152921504589938689]
    for i, q in enumerate(o.primes):
        assert q % (2 * 65536) == 1
        psi = o.roots[i]
        assert pow(psi, 65536, q) == q - 1  # primitive 2N-th root
    o.close()


def test_twiddle_tables(ctx):
    o = ctx
    w = o.N.bit_length() - 1
    for i in (0, o.L - 1, o.L, o.L + o.K - 1):
        q, psi = o.primes[i], o.roots[i]
        rou, roup, roui, rouip = (o.twiddles(i, k) for k in range(4))
        for j in range(o.N):
            assert int(rou[bitrev(j, w)]) == pow(psi, j, q)
            assert int(roui[bitrev(j, w)]) == pow(psi, -j, q)
        assert [int(x) for x in roup] == [(int(v) << 64) // q for v in rou]
        assert [int(x) for x in rouip] == [(int(v) << 64) // q for v in roui]


def test_ntt_is_evaluation_at_odd_powers(ctx):
    o = ctx
    N, w = o.N, o.N.bit_length() - 1
    idx = [0, 3, o.L, o.L + 1]
    x = seeded.uniform_poly(5, [o.primes[i] for i in idx], N)
    y = o.ntt(x, idx)
    for t, pi in enumerate(idx):
        q, psi = o.primes[pi], o.roots[pi]
        a = [int(v) for v in x[t * N:(t + 1) * N]]
        for j in range(N):
            e = 2 * bitrev(j, w) + 1
            assert int(y[t * N + j]) == sum(a[n] * pow(psi, e * n, q) for n in range(N)) % q
    assert (o.intt(y, idx) == x).all()


def test_negacyclic_convolution(ctx):
    o = ctx
    N = o.N
    idx = [1, o.L]
    pr = [o.primes[i] for i in idx]
    a = seeded.uniform_poly(7, pr, N)
    b = seeded.uniform_poly(8, pr, N)
    lev = np.concatenate([o.hw("modmul", o.ntt(a, idx)[t * N:(t + 1) * N], o.ntt(b, idx)[t * N:(t + 1) * N], idx[t]) for t in range(2)])
    c = o.intt(lev, idx)
    for t, q in enumerate(pr):
        aa = [int(v) for v in a[t * N:(t + 1) * N]]
        bb = [int(v) for v in b[t * N:(t + 1) * N]]
        ref = [0] * N
        for i in range(N):
            for j in range(N):
                k = i + j
                if k < N:
                    ref[k] += aa[i] * bb[j]
                else:
                    ref[k - N] -= aa[i] * bb[j]
        assert [int(v) for v in c[t * N:(t + 1) * N]] == [v % q for v in ref]


def test_automorphism_ntt_table_matches_coefficient_map(ctx):
    """sigma_k on coefficients (x -> x^k) followed by NTT == gather of the NTT with the NTT-form table."""
    o = ctx
    N = o.N
    for rot in (1, 3, -2, 2 * N - 1):
        k = o.find_automorphism_index(rot)
        if rot == 2 * N - 1:
            assert k == 2 * N - 1
        else:
            assert k == pow(5, rot, 2 * N)
        x = seeded.uniform_poly(11 + rot, [o.primes[2]], N)
        q = o.primes[2]
        sig = [0] * N
        for j in range(N):
            e = (j * k) % (2 * N)
            if e < N:
                sig[e] = int(x[j])
            else:
                sig[e - N] = (-int(x[j])) % q
        want = o.ntt(np.array(sig, np.int64), [2])
        got = o.hw("rotate", o.ntt(x, [2]), o.automorphism_order(k, True), 2)
        assert (want == got).all()
        # coefficient-form table does the same map directly (q - 0 = q is reduced here)
        got_c = o.hw("rotate", x, o.automorphism_order(k, False), 2) % q
        assert [int(v) for v in got_c] == sig


def _digit(o, level, part):
    nd = o.num_decomp(level)
    start = o.part_size * part
    ln = level - start if part == nd - 1 else o.part_size
    dig = list(range(start, start + ln))
    comp = [i for i in range(level) if i not in dig] + [o.L + j for j in range(o.K)]
    return dig, comp


@pytest.mark.parametrize("level", [7, 5, 2])
def test_modup_tables_bigint(ctx, level):
    o = ctx
    for part in range(o.num_decomp(level)):
        dig, comp = _digit(o, level, part)
        D = 1
        for i in dig:
            D *= o.primes[i]
        hat_inv, hat, cidx = o.tbl_modup(level, part)
        assert list(cidx) == comp
        for a, i in enumerate(dig):
            h = D // o.primes[i]
            assert int(hat_inv[a]) == pow(h, -1, o.primes[i])
            assert [int(v) for v in hat[a]] == [h % o.primes[j] for j in comp]


def test_moddown_and_rescale_tables_bigint(ctx):
    o = ctx
    P = 1
    for j in range(o.K):
        P *= o.primes[o.L + j]
    phat_inv, phat, pinv, pmod = o.tbl_moddown()
    for j in range(o.K):
        pj = o.primes[o.L + j]
        assert int(phat_inv[j]) == pow(P // pj, -1, pj)
    for i in range(o.L):
        qi = o.primes[i]
        assert [int(v) for v in phat[i]] == [(P // o.primes[o.L + j]) % qi for j in range(o.K)]
        assert int(pmod[i]) == P % qi and int(pinv[i]) == pow(P, -1, qi)
    Q = 1
    for i in range(o.L):
        Q *= o.primes[i]
    for level in range(2, o.L + 1):
        ql = o.primes[level - 1]
        a, b = o.tbl_rescale(level)
        H = Q // ql  # the reference uses the full-Q cofactor at every level
        c = (H * pow(H, -1, ql)) // ql
        for i in range(level - 1):
            assert int(a[i]) == pow(ql, -1, o.primes[i])
            assert int(b[i]) == c % o.primes[i]


@pytest.mark.parametrize("level", [7, 4])
def test_decomp_modup_bigint(ctx, level):
    o = ctx
    N = o.N
    x = seeded.uniform_poly(21, o.primes[:level], N)
    for part in range(o.num_decomp(level)):
        dig, comp = _digit(o, level, part)
        D = 1
        for i in dig:
            D *= o.primes[i]
        out = o.decomp_modup(x, level, part, is_ntt=False)
        for n in range(0, N, 5):
            acc = 0
            for i in dig:
                qi = o.primes[i]
                h = D // qi
                acc += (int(x[i * N + n]) * pow(h, -1, qi) % qi) * h
            for t in range(level + o.K):
                pi = t if t < level else o.L + (t - level)
                if pi in dig:
                    assert out[t * N + n] == x[pi * N + n]
                else:
                    assert int(out[t * N + n]) == acc % o.primes[pi]
        # NTT-form path = same thing between INTT and NTT
        xn = o.ntt(x, list(range(level)))
        outn = o.decomp_modup(xn, level, part, is_ntt=True)
        assert (o.intt(outn, o.limb_primes(level)) == out).all()


@pytest.mark.parametrize("level", [7, 3])
def test_mod_down_bigint(ctx, level):
    o = ctx
    N, K = o.N, o.K
    pr = [o.primes[i] for i in o.limb_primes(level)]
    x = seeded.uniform_poly(31, pr, N)
    P = 1
    for j in range(K):
        P *= o.primes[o.L + j]
    out = o.mod_down(x, level, is_ntt=False)
    for n in range(0, N, 3):
        acc = 0
        for j in range(K):
            pj = o.primes[o.L + j]
            h = P // pj
            acc += (int(x[(level + j) * N + n]) * pow(h, -1, pj) % pj) * h
        for i in range(level):
            qi = o.primes[i]
            assert int(out[i * N + n]) == (int(x[i * N + n]) - acc) * pow(P, -1, qi) % qi
    xn = o.ntt(x, o.limb_primes(level))
    assert (o.intt(o.mod_down(xn, level, is_ntt=True), list(range(level))) == out).all()


@pytest.mark.parametrize("level", [7, 2])
def test_rescale_bigint(ctx, level):
    o = ctx
    N = o.N
    x = seeded.uniform_poly(41, o.primes[:level], N)
    ql = o.primes[level - 1]
    # coefficient form: plain residue of the last limb (rns_poly.c:380-400)
    out = o.rescale(x, level, is_ntt=False)
    for i in range(level - 1):
        qi = o.primes[i]
        for n in range(N):
            assert int(out[i * N + n]) == (int(x[i * N + n]) - int(x[(level - 1) * N + n]) % qi) * pow(ql, -1, qi) % qi
    # NTT form: centred lift of the last limb (rns_poly.c:333-378)
    xn = o.ntt(x, list(range(level)))
    outn = o.intt(o.rescale(xn, level, is_ntt=True), list(range(level - 1)))
    for i in range(level - 1):
        qi = o.primes[i]
        for n in range(N):
            c = int(x[(level - 1) * N + n])
            c = c - ql if c > ql // 2 else c
            assert int(outn[i * N + n]) == (int(x[i * N + n]) - c) * pow(ql, -1, qi) % qi


def test_dot_prod_and_fast_variant(ctx):
    o = ctx
    N, level = o.N, 5
    nd = o.num_decomp(level)
    pr = [o.primes[i] for i in o.limb_primes(level)]
    digits = np.concatenate([seeded.uniform_poly(50 + d, pr, N) for d in range(nd)])
    allp = o.primes
    key = np.concatenate([seeded.uniform_poly(60 + d, allp, N) for d in range(nd)])
    out = o.dot_prod(digits, key, nd, level, fast=False)
    assert (out == o.dot_prod(digits, key, nd, level, fast=True)).all()
    T = level + o.K
    for t in range(T):
        pi = t if t < level else o.L + (t - level)
        q = o.primes[pi]
        for n in range(0, N, 7):
            s = sum(int(digits[(d * T + t) * N + n]) * int(key[(d * (o.L + o.K) + pi) * N + n]) for d in range(nd))
            assert int(out[t * N + n]) == s % q


def test_keyswitch_decrypts(ctx):
    """Relinearisation with a genuine key: Dec(relin(d0,d1,d2)) ~ d0 + d1 s + d2 s^2 (small error)."""
    o = ctx
    N, L, K = o.N, o.L, o.K
    rng = np.random.default_rng(9)
    allp = o.primes
    allidx = list(range(L + K))
    Q = 1
    for i in range(L):
        Q *= allp[i]
    P = 1
    for j in range(K):
        P *= allp[L + j]

    def rns(vals, idx):
        return np.concatenate([np.array([int(v) % allp[i] for v in vals], np.int64) for i in idx])

    s = rng.integers(-1, 2, N)
    s_ntt = o.ntt(rns(s, allidx), allidx)
    s2_ntt = np.concatenate([o.hw("modmul", s_ntt[i * N:(i + 1) * N], s_ntt[i * N:(i + 1) * N], i) for i in allidx])
    # switch key for s^2 -> s (key_gen.c:127-200): b_d = e + P*s^2*[digit d] - a_d*s
    swk = []
    for d in range(o.parts):
        a = seeded.uniform_poly(70 + d, allp, N)
        e = o.ntt(rns(rng.integers(-3, 4, N), allidx), allidx)
        b = np.zeros((L + K) * N, np.int64)
        for i in allidx:
            q = allp[i]
            sl = slice(i * N, (i + 1) * N)
            v = o.hw("modsub", e[sl], o.hw("modmul", a[sl], s_ntt[sl], i), i)
            if i < L and d * o.part_size <= i < (d + 1) * o.part_size:
                v = o.hw("modadd", v, o.hw("modmul_scalar", s2_ntt[sl], P % q, i), i)
            b[sl] = v
        swk += [b, a]
    swk = np.concatenate(swk)
    level = L
    idx = list(range(level))
    d2 = seeded.uniform_poly(80, allp[:level], N)
    zero = np.zeros(level * N, np.int64)
    r0, r1 = o.relin(zero, zero, d2, swk, level)
    # decrypt r0 + r1*s  and compare with d2*s^2 over the integers mod Q
    dec = np.concatenate([o.hw("modadd", r0[i * N:(i + 1) * N], o.hw("modmul", r1[i * N:(i + 1) * N], s_ntt[i * N:(i + 1) * N], i), i) for i in idx])
    want = np.concatenate([o.hw("modmul", d2[i * N:(i + 1) * N], s2_ntt[i * N:(i + 1) * N], i) for i in idx])
    diff = o.intt(np.concatenate([o.hw("modsub", dec[i * N:(i + 1) * N], want[i * N:(i + 1) * N], i) for i in idx]), idx)
    for n in range(N):
        v = 0
        for i in idx:
            q = allp[i]
            h = Q // q
            v += int(diff[i * N + n]) * pow(h, -1, q) * h
        v %= Q
        v = v - Q if v > Q // 2 else v
        assert abs(v) < 2 ** 30, "key-switch noise too large: wrong digit/key/limb pairing"


def test_sub_mul_const_matches_its_c_semantics():
    """(v1 - v2) * w mod q where it is a plain modular product, and the wrapped value where v2 > v1 + q."""
    import ctypes as C
    from oracle_lib import lib
    L_ = lib()
    q = (1 << 40) + 15 * 128 + 1
    rng = np.random.default_rng(5)
    for _ in range(200):
        w = int(rng.integers(1, q))
        wp = (w << 64) // q
        v1, v2 = int(rng.integers(0, q)), int(rng.integers(0, q))
        assert L_.orc_sub_mul_const(v1, v2, w, wp, q) == (v1 - v2) * w % q
        big = int(rng.integers(2 * q, 1 << 50))  # a residue of a larger prime
        s_ = v1 - big + q
        assert s_ < 0
        m64 = (1 << 64) - 1
        qq = ((s_ % (1 << 128)) * wp >> 64) & m64
        y = ((s_ & m64) * w - qq * q) & m64
        assert L_.orc_sub_mul_const(v1, big, w, wp, q) == C.c_int64(y - q if y >= q else y).value
