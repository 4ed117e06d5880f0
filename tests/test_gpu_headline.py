"""The batched entry points the benchmark times, at the benchmark's own configuration (N = 2^16, 24 limbs, 7 special
primes, 3 digits of 8 limbs), against the oracle and against the single-operand entry points (needs an MI355X).

Reference: Mul_ciphertext3 + Relinearize_ciph3 + Rescale_ciphertext (ckks/src/evaluator.c:142-190,288-306,342-362),
Fast_switch_key / Fast_rotate (:411-462,503-522), Rotate_batch_ciph (ckks/src/cipher.c:459-479)."""
import numpy as np
import pytest

import acefhe
import headline
from oracle_lib import Oracle
from test_gpu_parity import eq

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def big():
    g = acefhe.Context(*headline.CFG)
    assert g.has_device, "no GPU visible"
    assert (g.L, g.K, g.part_size) == (24, 7, 8)
    o = Oracle(*headline.CFG)
    swk = headline.seeded_key(g.primes)
    cts = headline.seeded_ciphertexts(g.primes, g.L)
    yield g, o, swk, cts
    g.close()
    o.close()


def test_hmult_batch_of_16_pairs(big):
    """16 pairs in one call, operands one limb apart: pairs 0, 7 and 15 against the oracle, every pair against the
    single-operand entry point; the padding between results stays untouched."""
    g, o, swk, cts = big
    print("ace_mul_relin_rescale_batch, 16 pairs, level 24", flush=True)
    N, level, pairs = g.N, g.L, headline.PAIRS
    in_stride, out_stride = (level + 1) * N, level * N
    dk = g.upload(swk)
    dcts = [g.upload(c) for c in cts]
    ops = headline.hmult_operands(g, dcts, level, pairs, in_stride)
    r0, r1 = g.alloc(pairs * out_stride), g.alloc(pairs * out_stride)
    g.mul_relin_rescale_batch(r0, r1, out_stride, ops[0], ops[1], ops[2], ops[3], in_stride, dk, level, pairs)
    got0, got1 = r0.get(), r1.get()
    n = (level - 1) * N
    for p in (0, 7, 15):
        a = [headline.shifted_host(c, p, g.primes[:level]) for c in cts]
        eq(ops[2].view(p * in_stride, level * N), a[2], "operand %d as derived on the device" % p)
        m0, m1 = o.mul_relin_rescale(*a, swk, level)
        eq(got0[p * out_stride:p * out_stride + n], m0, "pair %d c0 vs oracle" % p)
        eq(got1[p * out_stride:p * out_stride + n], m1, "pair %d c1 vs oracle" % p)
    s0, s1 = g.alloc(n), g.alloc(n)
    for p in range(pairs):
        g.mul_relin_rescale(s0, s1, *(x.view(p * in_stride, level * N) for x in ops), dk, level)
        eq(got0[p * out_stride:p * out_stride + n], s0.get(), "pair %d c0 vs single call" % p)
        eq(got1[p * out_stride:p * out_stride + n], s1.get(), "pair %d c1 vs single call" % p)
        assert not got0[p * out_stride + n:(p + 1) * out_stride].any(), "padding written"
        assert not got1[p * out_stride + n:(p + 1) * out_stride].any(), "padding written"
    # the benchmark's own layout: operands back to back
    tight_in, tight_out = level * N, n
    tops = headline.hmult_operands(g, dcts, level, pairs, tight_in)
    t0, t1 = g.alloc(pairs * tight_out), g.alloc(pairs * tight_out)
    g.mul_relin_rescale_batch(t0, t1, tight_out, tops[0], tops[1], tops[2], tops[3], tight_in, dk, level, pairs)
    h0, h1 = t0.get(), t1.get()
    for p in range(pairs):
        eq(h0[p * n:(p + 1) * n], got0[p * out_stride:p * out_stride + n], "tight layout, pair %d c0" % p)
        eq(h1[p * n:(p + 1) * n], got1[p * out_stride:p * out_stride + n], "tight layout, pair %d c1" % p)
    for b in ops + tops + dcts + [r0, r1, s0, s1, t0, t1, dk]:
        b.free()


def test_rotation_batch_of_32(big):
    """The benchmark's 32 rotation amounts in one call: +1, -1, 2^14 and two of the seeded amounts against the
    oracle's Fast_rotate on the oracle's hoisted digits, all 32 against the single-rotation entry point."""
    g, o, swk, cts = big
    print("ace_rotate_batch, 32 rotations, level 24", flush=True)
    N, level = g.N, g.L
    rots = headline.rotation_indices()
    dk = g.upload(swk)
    dc0, dc1 = g.upload(cts[0]), g.upload(cts[1])
    keys = headline.rotation_keys(g, dk, len(rots))
    ks = [g.find_automorphism_index(r) for r in rots]
    orders = [g.automorphism_order(k, True) for k in ks]
    n = level * N
    r0s, r1s = g.alloc(len(rots) * n), g.alloc(len(rots) * n)
    g.rotate_batch(r0s, r1s, dc0, dc1, keys, orders, level)
    got0, got1 = r0s.get(), r1s.get()
    digits = o.precomp(cts[1], level, True)
    for i in (0, 15, 14, 16, 31):  # +1, -1, 2^14, seeded, seeded
        assert ks[i] == o.find_automorphism_index(rots[i])
        key = headline.rotation_key_host(g, swk, i)
        eq(keys[i], key, "key %d as derived on the device" % i)
        w0, w1 = o.fast_rotate(cts[0], digits, key, o.automorphism_order(ks[i], True), level)
        eq(got0[i * n:(i + 1) * n], w0, "rotation by %d, c0 vs oracle" % rots[i])
        eq(got1[i * n:(i + 1) * n], w1, "rotation by %d, c1 vs oracle" % rots[i])
    T = level + g.K
    dd = g.alloc(g.num_decomp(level) * T * N)
    g.precomp(dd, dc1, level, True)
    eq(dd, digits, "hoisted digits vs oracle")
    s0, s1 = g.alloc(n), g.alloc(n)
    for i in range(len(rots)):
        g.fast_rotate(s0, s1, dc0, dd, keys[i], orders[i], level)
        eq(got0[i * n:(i + 1) * n], s0.get(), "rotation %d c0 vs single call" % i)
        eq(got1[i * n:(i + 1) * n], s1.get(), "rotation %d c1 vs single call" % i)
    for b in keys + orders + [dk, dc0, dc1, r0s, r1s, dd, s0, s1]:
        b.free()


def test_ntt_batch_of_32_polynomials(big):
    """The benchmark's NTT batch: the forward transform of polynomials 0, 13 and 31 of the 32 x 24-limb batch against
    the oracle (the round trip alone would accept a wrong pair of mutually inverse transforms)."""
    g, o, _, _ = big
    import seeded
    N, limbs, polys = g.N, headline.LIMBS, 32
    idx = list(range(limbs))
    per_poly = limbs * N
    check = (0, 13, 31)
    x = g.alloc(polys * per_poly)
    hosts = {}
    for p in range(polys):
        if p in check:
            hosts[p] = seeded.uniform_poly(1000 + p, g.primes[:limbs], N)
            x.view(p * per_poly, per_poly).set(hosts[p])
        else:
            g.sample_uniform(x.view(p * per_poly, per_poly), limbs, False, 99, p)
    g.ntt(x, x, idx, n_polys=polys, poly_stride_limbs=limbs)
    for p in check:
        eq(x.view(p * per_poly, per_poly), o.ntt(hosts[p], idx), "forward, polynomial %d of the batch" % p)
    g.intt(x, x, idx, n_polys=polys, poly_stride_limbs=limbs)
    for p in check:
        eq(x.view(p * per_poly, per_poly), hosts[p], "round trip, polynomial %d" % p)
    x.free()


@pytest.mark.parametrize("polys,limbs,stride", [(16, 24, 24), (19, 24, 24), (17, 24, 25), (33, 3, 3)])
def test_transforms_of_many_polynomials_equal_single_transforms(big, polys, limbs, stride):
    """Launches large enough to fill the machine twice over, with all limbs below 2^50.2, take the chunk passes that
    work through runs of eight or four polynomials with the next one's words on their way into LDS (ace_ntt.hip:
    ntt_fwd_chunk_run, ntt_inv_half_run, run_length); smaller ones (the last case) take the one-polynomial kernels.
    Every polynomial of the batch must come out as it does alone: in place and into another buffer, counts that the
    run length does not divide, a gap limb between the polynomials that must survive, and two of them against the
    oracle."""
    g, o, _, _ = big
    import seeded
    N = g.N
    idx = list(range(limbs))
    per, gap = stride * N, (stride - limbs) * N
    host = np.zeros(polys * per, np.int64)
    marker = np.arange(N, dtype=np.int64) * 3 + 1
    for p in range(polys):
        host[p * per:p * per + limbs * N] = seeded.uniform_poly(3000 + p, g.primes[:limbs], N)
        if gap:
            host[p * per + limbs * N:(p + 1) * per] = marker
    x, y, one = g.upload(host), g.upload(np.zeros(polys * per, np.int64)), g.alloc(limbs * N)
    g.ntt(y, x, idx, n_polys=polys, poly_stride_limbs=stride)      # into another buffer
    g.ntt(x, x, idx, n_polys=polys, poly_stride_limbs=stride)      # in place
    fwd = x.get()
    for p in range(polys):
        s = slice(p * per, p * per + limbs * N)
        one.set(host[s])
        g.ntt(one, one, idx)
        eq(fwd[s], one.get(), "forward in place, polynomial %d" % p)
        eq(y.view(p * per, limbs * N), fwd[s], "forward into another buffer, polynomial %d" % p)
        if gap:
            eq(fwd[p * per + limbs * N:(p + 1) * per], marker, "gap limb after polynomial %d" % p)
    for p in (0, polys - 1):
        s = slice(p * per, p * per + limbs * N)
        eq(fwd[s], o.ntt(host[s], idx), "forward against the oracle, polynomial %d" % p)
    y.set(np.zeros(polys * per, np.int64))
    g.intt(y, x, idx, n_polys=polys, poly_stride_limbs=stride)     # into another buffer
    g.intt(x, x, idx, n_polys=polys, poly_stride_limbs=stride)     # in place
    back = x.get()
    for p in range(polys):
        s = slice(p * per, p * per + limbs * N)
        eq(back[s], host[s], "round trip in place, polynomial %d" % p)
        eq(y.view(p * per, limbs * N), host[s], "inverse into another buffer, polynomial %d" % p)
        if gap:
            eq(back[p * per + limbs * N:(p + 1) * per], marker, "gap limb after the inverse, polynomial %d" % p)
    for b in (x, y, one):
        b.free()
