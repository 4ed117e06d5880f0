"""Oracle vs. the known-answer vectors held by the reference's own unit tests.

Sources (fhe-cmplr/rtlib/ant/unittest): ut_test_number_theory.cxx:14-106,
ut_ntt.cxx:14-91, ut_poly.cxx:97,185-214,382-480.
"""
import numpy as np
import pytest

from oracle_lib import Oracle, lib


def test_mod_exp_kat():
    L = lib()
    assert L.orc_mod_exp(12312, 53, 9393333) == 2678490
    assert L.orc_mod_exp(3880, 391, 9000) == 1000
    assert L.orc_mod_exp(-1, 432413, 88) == 87
    assert L.orc_mod_exp(1230911482, 268435451, 8796092858369) == 3778006589735
    assert L.orc_mod_exp(2, 432413, 9999) == 1526


def test_mod_inv_kat():
    L = lib()
    for v, m, e in [(7, 19, 11), (43, 103, 12), (94, 97, 32), (25, 32, 9)]:
        assert L.orc_mod_inv(v, m) == e


def test_generator_and_root_kat():
    L = lib()
    assert [L.orc_find_generator(q) for q in (5, 7, 11)] == [2, 3, 2]
    assert L.orc_root_of_unity(2, 5) == 4
    assert L.orc_root_of_unity(3, 7) == 2
    assert L.orc_root_of_unity(5, 11) == 4


def test_is_prime_kat():
    L = lib()
    for p in (2, 3, 5, 7, 11, 7919, 0x7fffffd8001, 0x7fffffc8001, 0xfffffffc001, 0xffffff6c001):
        assert L.orc_is_prime(p)
    for c in (12, 14, 15, 21, 25, 7921):
        assert not L.orc_is_prime(c)


def test_precompute_const_128_kat():
    import ctypes as C
    out = (C.c_uint64 * 2)()
    lib().orc_precompute_const_128(576460752298835969, out)
    assert out[1] == 32 and out[0] == 4697619456


def test_mul_barrett_kat():
    o = Oracle(4, 1, 0, 0, 1, primes=[1001 * 0 + 4503599626321921])
    assert o.L_.orc_mul_mod_barrett(o.h, 0, 12312, 53) == (12312 * 53) % 4503599626321921
    o.close()


def test_ntt_kat():
    o = Oracle(4, 1, 0, 0, 1, primes=[4503599626321921])
    x = np.array([0, 1, 2, 3], np.int64)
    y = np.array([1168890670389420, 2803840134912590, 1418812602632428, 3615655844709404], np.int64)
    assert (o.ntt(x, [0]) == y).all()
    assert (o.intt(y, [0]) == x).all()
    o.close()


@pytest.fixture(scope="module")
def ut_poly_ctx():
    o = Oracle(4, 10, 60, 59, 3)  # ut_poly.cxx:26-33
    yield o
    o.close()


def _to_rns(o, vals, nlimbs):
    return np.concatenate([np.array([v % o.primes[t] for v in vals], np.int64) for t in range(nlimbs)])


def _crt_signed(o, rns, nlimbs):
    N = o.N
    Q = 1
    for t in range(nlimbs):
        Q *= o.primes[t]
    out = []
    for n in range(N):
        v = 0
        for t in range(nlimbs):
            q = o.primes[t]
            h = Q // q
            v += int(rns[t * N + n]) * pow(h, -1, q) * h
        v %= Q
        out.append(v - Q if v > Q // 2 else v)
    return out


def test_mul_poly_kat(ut_poly_ctx):
    o = ut_poly_ctx
    idx = list(range(10))
    a = o.ntt(_to_rns(o, [0, 1, 4, 5], 10), idx)
    b = o.ntt(_to_rns(o, [1, 2, 4, 3], 10), idx)
    p = o.intt(o.poly("mul", a, b, 10), idx)
    assert _crt_signed(o, p, 10) == [-29, -31, -9, 17]
    s = o.poly("add", _to_rns(o, [0, 1, 4, 5], 10), _to_rns(o, [1, 2, 4, 3], 10), 10)
    assert _crt_signed(o, s, 10) == [1, 3, 8, 8]
    d = o.poly("sub", _to_rns(o, [0, 1, 4, 5], 10), _to_rns(o, [1, 2, 4, 3], 10), 10)
    assert _crt_signed(o, d, 10) == [-1, -1, 0, 2]


def test_rotate_poly_kat(ut_poly_ctx):
    o = ut_poly_ctx
    x = _to_rns(o, [0, 1, 4, 59], 10)
    k = o.find_automorphism_index(3)
    order = o.automorphism_order(k, is_ntt=False)
    r = o.poly("automorphism", x, order, 10)
    got = _crt_signed(o, r % np.repeat(np.array(o.primes[:10], np.int64), 4), 10)
    assert got == [0, -1, 4, -59]
    k = o.find_automorphism_index(6)
    order = o.automorphism_order(k, is_ntt=False)
    r = o.poly("automorphism", x, order, 10)
    assert _crt_signed(o, r % np.repeat(np.array(o.primes[:10], np.int64), 4), 10) == [0, 1, 4, 59]


@pytest.mark.parametrize("is_ntt", [True, False])
def test_precompute_fused_equals_unfused(ut_poly_ctx, is_ntt):
    o = ut_poly_ctx
    x = _to_rns(o, [0, 1, 4, 5], 10)
    if is_ntt:
        x = o.ntt(x, list(range(10)))
    assert (o.precomp(x, 10, is_ntt, fused=True) == o.precomp(x, 10, is_ntt, fused=False)).all()


def test_extend_mod_down_identity(ut_poly_ctx):
    o = ut_poly_ctx
    x = _to_rns(o, [0, 1, 4, 5], 10)
    e = o.extend(x, 10)
    r = o.mod_down(e, 10, is_ntt=False)
    assert _crt_signed(o, r, 10) == [0, 1, 4, 5]
