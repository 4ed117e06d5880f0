"""HIP path vs. the CPU oracle, bit for bit, through the C-ABI (needs an MI355X)."""
import numpy as np
import pytest

import acefhe
import seeded
from oracle_lib import Oracle

pytestmark = pytest.mark.gpu

SMALL = [(4, 3, 40, 40, 1), (16, 10, 60, 59, 3), (64, 7, 45, 40, 3), (64, 6, 50, 50, 2), (2048, 4, 55, 50, 2),
         (4096, 3, 40, 40, 1)]
LARGE = [(8192, 5, 40, 40, 3), (16384, 4, 60, 50, 2), (32768, 3, 50, 50, 3), (65536, 6, 50, 50, 3),
         (131072, 2, 50, 45, 1)]


class Pair:
    def __init__(self, cfg):
        self.cfg = cfg
        self.g = acefhe.Context(*cfg)
        assert self.g.has_device, "no GPU visible"
        self.o = Oracle(*cfg)

    def close(self):
        self.g.close()
        self.o.close()


@pytest.fixture(scope="module", params=SMALL + LARGE, ids=lambda c: "N%d_L%d" % (c[0], c[1]))
def pair(request):
    print("config", request.param, flush=True)
    p = Pair(request.param)
    yield p
    p.close()


def eq(dev, want, what):
    got = dev.get() if hasattr(dev, "get") else dev
    want = np.asarray(want, dtype=np.int64).ravel()
    assert got.shape == want.shape, what
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, "%s: %d of %d words differ, first at %d (got %d want %d)" % (
        what, bad.size, want.size, bad[0], got[bad[0]], want[bad[0]])


def big_ring_skip(N):
    """The tests of the bootstrap's and the recorded runs' kernels run on the small rings and on N = 65536, the only
    size whole models use; the other large rings are skipped to bound the run time."""
    if N > 8192 and N != 65536:
        pytest.skip("covered at the smaller rings and at N = 65536")


def draw_poly(g, seed, level, with_p):
    """(host, device) copies of a polynomial of `level` Q limbs (+ the P limbs) with uniform residues: from the seeded
    host generator on small rings, drawn on the device and downloaded on large ones (the host generator takes
    0.7 us per word)."""
    if g.N <= 8192:
        x = seeded.uniform_poly(seed, [g.primes[i] for i in g.limb_primes(level, with_p)], g.N)
        return x, g.upload(x)
    d = g.alloc((level + (g.K if with_p else 0)) * g.N)
    g.sample_uniform(d, level, with_p, 0xACE, seed)
    return d.get(), d


def test_ntt_all_primes(pair):
    g, o = pair.g, pair.o
    N = g.N
    idx = list(range(g.L + g.K))
    x = seeded.uniform_poly(1, g.primes, N)
    dx = g.upload(x)
    dy = g.alloc(x.size)
    g.ntt(dy, dx, idx)
    eq(dy, o.ntt(x, idx), "forward")
    eq(dx, x, "source untouched")
    g.intt(dy, dy, idx)
    eq(dy, x, "round trip in place")
    g.intt(dy, dx, idx)
    eq(dy, o.intt(x, idx), "inverse")
    # edge values: all zero, all q-1, a single one
    e = np.concatenate([np.zeros(N, np.int64), np.full(N, g.primes[1 % len(idx)] - 1, np.int64)])
    e2 = np.zeros(N, np.int64)
    e2[N - 1] = 1
    e = np.concatenate([e, e2])
    pidx = [0, 1 % len(idx), len(idx) - 1]
    de = g.upload(e)
    g.ntt(de, de, pidx)
    eq(de, o.ntt(e, pidx), "edge values forward")
    g.intt(de, de, pidx)
    eq(de, e, "edge values round trip")


@pytest.mark.parametrize("N,primes", [(8192, [1289999999795201, 1289999999582209]),
                                      (65536, [1289999997075457, 1289999994191873]),
                                      (131072, [1289999988293633, 1289999986720769])])
def test_ntt_largest_primes_of_the_fp64_back_end(N, primes):
    """Primes just under the bound up to which the transform carries residues in FP64, with inputs made of
    0, 1, (q-1)/2, (q+1)/2 and q-1: the partial sums between reductions grow fastest for these."""
    for q in primes:  # the moduli are what they are said to be (Fermat tests to three bases)
        assert q < 1290000000000000 and q % (2 * N) == 1 and all(pow(a, q - 1, q) == 1 for a in (2, 3, 5))
    g = acefhe.Context(N, len(primes), primes=primes)
    o = Oracle(N, len(primes), 0, 0, 1, primes=primes)
    try:
        idx = list(range(len(primes)))
        rng = np.random.Generator(np.random.PCG64(N))
        for case in range(3):
            limbs = []
            for q in primes:
                pool = np.array([0, 1, (q - 1) // 2, (q + 1) // 2, q - 1], np.int64)
                pick = rng.integers(0, 5, N) if case < 2 else np.full(N, 4)
                limbs.append(pool[pick] if case != 1 else np.where(rng.random(N) < 0.5, q - 1, (q + 1) // 2))
            x = np.concatenate(limbs).astype(np.int64)
            dx = g.upload(x)
            g.ntt(dx, dx, idx)
            eq(dx, o.ntt(x, idx), "forward, case %d" % case)
            g.intt(dx, dx, idx)
            eq(dx, x, "round trip, case %d" % case)
            dx.set(x)
            g.intt(dx, dx, idx)
            eq(dx, o.intt(x, idx), "inverse, case %d" % case)
            dx.free()
    finally:
        g.close()
        o.close()


def test_conversion_with_a_51_bit_first_prime():
    """A 51-bit first prime over 46-bit ones (the shape of the reference's model programs): the prime is both a
    source and a target of the base conversion's FP64 path.  Inputs are chosen so that the words entering the
    conversion are q-1, (q+1)/2 or 1 in every source limb, besides seeded uniform ones."""
    cfg = (8192, 7, 51, 46, 3)
    g, o = acefhe.Context(*cfg), Oracle(*cfg)
    try:
        N, level = g.N, g.L
        q = [int(x) for x in g.primes[:level]]
        assert 2 ** 50.9 < q[0] < 3 << 50 and all(x < 1 << 47 for x in q[1:])
        rng = np.random.Generator(np.random.PCG64(51))
        for case in range(4):
            limbs = []
            for t in range(level):
                part = t // g.part_size
                digit = q[part * g.part_size:min(level, (part + 1) * g.part_size)]
                rest = 1
                for m in digit:
                    rest *= m if m != q[t] else 1
                pool = [(v * rest) % q[t] for v in (q[t] - 1, (q[t] + 1) // 2, 1)]
                if case == 3:
                    limbs.append(rng.integers(0, q[t], N))
                else:
                    limbs.append(np.array(pool, np.int64)[rng.integers(0, 3, N) if case else np.zeros(N, np.int64)])
            x = np.concatenate(limbs).astype(np.int64)
            dx = g.upload(x)
            for is_ntt in (False, True):
                dr = g.alloc(g.num_decomp(level) * (level + g.K) * N)
                g.precomp(dr, dx, level, is_ntt)
                eq(dr, o.precomp(x, level, is_ntt), "precomp case %d ntt %d" % (case, is_ntt))
                dr.free()
            dx.free()
        # Mod_down: the 60-bit special primes are the sources, the 51-bit prime one of the targets
        pr = [g.primes[i] for i in g.limb_primes(level)]
        for case in range(2):
            e = seeded.uniform_poly(5100 + case, pr, N)
            if case:  # the largest source words
                e = np.concatenate([np.full(N, int(m) - 1, np.int64) for m in pr])
            de = g.upload(e)
            for is_ntt in (False, True):
                dr = g.alloc(level * N)
                g.mod_down(dr, de, level, is_ntt)
                eq(dr, o.mod_down(e, level, is_ntt), "mod_down case %d ntt %d" % (case, is_ntt))
                dr.free()
            de.free()
    finally:
        g.close()
        o.close()


@pytest.mark.parametrize("matrix", ["1", "0"], ids=["matrix_cores", "vector_units"])
@pytest.mark.parametrize("cfg", [(8192, 7, 51, 46, 3), (2048, 9, 60, 56, 3), (256, 5, 60, 59, 2), (65536, 13, 60, 56, 4)],
                         ids=lambda c: "N%d_L%d_%d_%d" % c[:4])
def test_conversion_on_the_matrix_cores_and_on_the_vector_units(cfg, matrix, monkeypatch):
    """The base conversion has two implementations for rings of 256 coefficients and more: int8 matrix products over
    the signed bytes of the source words (the default) and 128-bit / FP64 multiply-accumulates (ACE_CONV_MATRIX=0 when
    the context is made).  Both must give the oracle's words, also where the words entering the conversion are
    m-1, (m+1)/2, 1, or have every byte at 0x80, 0x7F or 0xFF (where the signed bytes carry), in every source limb."""
    monkeypatch.setenv("ACE_CONV_MATRIX", matrix)
    g, o = acefhe.Context(*cfg), Oracle(*cfg)
    try:
        N, level = g.N, g.L
        q = [int(x) for x in g.primes[:level]]
        rng = np.random.Generator(np.random.PCG64(77))
        for case in range(3):
            limbs = []
            for t in range(level):
                part = t // g.part_size
                digit = q[part * g.part_size:min(level, (part + 1) * g.part_size)]
                rest = 1
                for m in digit:
                    rest *= m if m != q[t] else 1
                want = [q[t] - 1, (q[t] + 1) // 2, 1, 0x8080808080808080 % q[t], 0x7F7F7F7F7F7F7F7F % q[t],
                        0xFFFFFFFFFFFFFFFF % q[t], 0x0080008000800080 % q[t]]
                pool = np.array([(v * rest) % q[t] for v in want], np.int64)  # times (Q_d / q_t)^-1 these become `want`
                if case == 2:
                    limbs.append(rng.integers(0, q[t], N))
                else:
                    limbs.append(pool[rng.integers(0, len(pool), N)] if case else np.full(N, pool[0]))
            x = np.concatenate(limbs).astype(np.int64)
            dx = g.upload(x)
            for is_ntt in (False, True):
                dr = g.alloc(g.num_decomp(level) * (level + g.K) * N)
                g.precomp(dr, dx, level, is_ntt)
                eq(dr, o.precomp(x, level, is_ntt), "precomp case %d ntt %d" % (case, is_ntt))
                dr.free()
            dx.free()
        for lvl in sorted({level, max(1, level - 3)}):
            pr = [g.primes[i] for i in g.limb_primes(lvl)]
            for case in range(2):
                e = seeded.uniform_poly(5200 + case, pr, N)
                if case:  # the largest source words
                    e = np.concatenate([np.full(N, int(m) - 1, np.int64) for m in pr])
                de = g.upload(e)
                for is_ntt in (False, True):
                    dr = g.alloc(lvl * N)
                    g.mod_down(dr, de, lvl, is_ntt)
                    eq(dr, o.mod_down(e, lvl, is_ntt), "mod_down level %d case %d ntt %d" % (lvl, case, is_ntt))
                    dr.free()
                de.free()
    finally:
        g.close()
        o.close()


def test_precomp_and_mod_down_batches_equal_single_calls(pair):
    """ace_precomp_batch / ace_mod_down_batch over polynomials at a constant stride (with a gap between them, as the
    c1 halves of a bootstrap level's inner sums lie) give the words of one call per polynomial, which the oracle pins."""
    g, o = pair.g, pair.o
    N, K = g.N, g.K
    big_ring_skip(N)
    count = 3
    for level in levels_of(g)[-2:]:
        T, nd = level + K, g.num_decomp(level)
        pr = [g.primes[i] for i in g.limb_primes(level)]
        for is_ntt in (True, False):
            ext = [seeded.uniform_poly(7700 + 10 * level + k, pr, N) for k in range(count)]
            stride = 2 * T * N  # every other polynomial of the buffer
            slab = np.zeros(count * stride, np.int64)
            for k in range(count):
                slab[k * stride + T * N:(k + 1) * stride] = ext[k]
            dslab = g.upload(slab)
            low = g.alloc(count * level * N)
            g.mod_down_batch(low, level * N, dslab.view(T * N, (count - 1) * stride + T * N), stride, count, level, is_ntt)
            want_low = [o.mod_down(e, level, is_ntt) for e in ext]
            eq(low, np.concatenate(want_low), "mod_down_batch l=%d ntt=%d" % (level, is_ntt))
            eq(dslab, slab, "mod_down_batch leaves its operands")
            dig = g.alloc(count * nd * T * N)
            g.precomp_batch(dig, nd * T * N, low, level * N, count, level, is_ntt)
            eq(dig, np.concatenate([o.precomp(w, level, is_ntt) for w in want_low]), "precomp_batch l=%d ntt=%d" % (level, is_ntt))
            for b in (dslab, low, dig):
                b.free()
    with pytest.raises(acefhe.AceError):
        a = g.alloc(2 * (g.L + K) * N)
        g.mod_down_batch(a, g.L * N, a, (g.L + K) * N, 2, g.L)  # results over operands


def test_conversion_with_strided_pass_equals_the_two_kernels(pair):
    """Launches of at least 192 converted limbs at N = 65536 run the base conversion and the strided pass of the
    transform that follows it in one kernel (Mod_down and Precomp of many polynomials, and, with the shared
    transform's prologue, HMult + relinearise + rescale of many pairs); single calls stay below that size and take
    the two kernels, which the other tests pin against the oracle.  Same words either way."""
    g = pair.g
    N, K, level = g.N, g.K, g.L
    if N != 65536:
        pytest.skip("the kernel serves N = 65536")
    T, nd = level + K, g.num_decomp(level)
    count, distinct = 40, 4
    assert count * level >= 192
    ext = [draw_poly(g, 8800 + k, level, True)[1] for k in range(distinct)]
    slab = g.alloc(count * T * N)
    for k in range(count):
        g.copy(slab.view(k * T * N, T * N), ext[k % distinct])
    low = g.alloc(count * level * N)
    g.mod_down_batch(low, level * N, slab, T * N, count, level, True)
    one = g.alloc(level * N)
    singles = []
    for k in range(distinct):
        g.mod_down(one, ext[k], level, True)
        singles.append(one.get())
    got = low.get().reshape(count, level * N)
    for k in range(count):
        eq(got[k], singles[k % distinct], "Mod_down of polynomial %d of %d" % (k, count))
    dig = g.alloc(count * nd * T * N)
    g.precomp_batch(dig, nd * T * N, low, level * N, count, level, True)
    one_dig = g.alloc(nd * T * N)
    want = []
    for k in range(distinct):
        g.precomp(one_dig, low.view(k * level * N, level * N), level, True)
        want.append(one_dig.get())
    got = dig.get().reshape(count, nd * T * N)
    for k in range(count):
        eq(got[k], want[k % distinct], "Precomp of polynomial %d of %d" % (k, count))
    for b in (slab, low, one, dig, one_dig):
        b.free()
    # pairs of ciphertexts: 2 * nb polynomials of `level` targets each through the shared Mod_down + Rescale transform
    nb = 20
    assert 2 * nb * level >= 192
    dk = g.alloc(2 * g.parts * (g.L + K) * N)
    for i in range(2 * g.parts):
        g.sample_uniform(dk.view(i * (g.L + K) * N, (g.L + K) * N), g.L, True, 0xACE, 8900 + i)
    ops = [[draw_poly(g, 8910 + 4 * b + i, level, False)[1] for i in range(4)] for b in range(distinct)]
    stride = level * N
    dev = [g.alloc(nb * stride) for _ in range(4)]
    for b in range(nb):
        for i in range(4):
            g.copy(dev[i].view(b * stride, stride), ops[b % distinct][i])
    r0, r1 = g.alloc(nb * stride), g.alloc(nb * stride)
    g.mul_relin_rescale_batch(r0, r1, stride, dev[0], dev[1], dev[2], dev[3], stride, dk, level, nb)
    s0, s1 = g.alloc(stride), g.alloc(stride)
    n = (level - 1) * N
    want = []
    for b in range(distinct):
        g.mul_relin_rescale(s0, s1, *ops[b], dk, level)
        want.append((s0.get()[:n], s1.get()[:n]))
    got0, got1 = r0.get().reshape(nb, stride), r1.get().reshape(nb, stride)
    for b in range(nb):
        eq(got0[b][:n], want[b % distinct][0], "pair %d of %d, c0" % (b, nb))
        eq(got1[b][:n], want[b % distinct][1], "pair %d of %d, c1" % (b, nb))
    for b in [dk, r0, r1, s0, s1] + dev + ext + [x for o4 in ops for x in o4]:
        b.free()


def test_ntt_batched_polys(pair):
    g, o = pair.g, pair.o
    N = g.N
    nl, npoly, stride = min(3, g.L), 3, min(3, g.L) + 1
    idx = list(range(nl))
    buf = np.zeros(npoly * stride * N, np.int64)
    for p in range(npoly):
        buf[p * stride * N:(p * stride + nl) * N] = seeded.uniform_poly(10 + p, g.primes[:nl], N)
    marker = np.arange(N, dtype=np.int64)
    for p in range(npoly):
        buf[(p * stride + nl) * N:(p + 1) * stride * N] = marker  # gap limb must survive
    d = g.upload(buf)
    g.ntt(d, d, idx, n_polys=npoly, poly_stride_limbs=stride)
    want = buf.copy()
    for p in range(npoly):
        s = slice(p * stride * N, (p * stride + nl) * N)
        want[s] = o.ntt(buf[s], idx)
    eq(d, want, "batched forward")
    g.intt(d, d, idx, n_polys=npoly, poly_stride_limbs=stride)
    eq(d, buf, "batched round trip")


def test_strided_passes_of_small_and_large_launches_on_integer_limbs():
    """At N = 65536 a transform of a few limbs on the integer back end spreads each column of its strided pass over
    four waves; a launch of many limbs keeps a column in one thread.  Both must give the oracle's words: a single
    polynomial (forward, inverse, and the Rescale whose strided pass forms its input from the dropped limb), then 40
    copies of it in one launch, every one of which must come out like the single polynomial."""
    cfg = (65536, 4, 60, 56, 2)
    g, o = acefhe.Context(*cfg), Oracle(*cfg)
    try:
        N, L = g.N, g.L
        idx = list(range(L + g.K))
        pr = [g.primes[i] for i in idx]
        nl = len(idx)
        x = seeded.uniform_poly(91, pr, N)
        d = g.upload(x)
        g.ntt(d, d, idx)
        fwd = o.ntt(x, idx)
        eq(d, fwd, "forward, one polynomial")
        g.intt(d, d, idx)
        eq(d, x, "round trip, one polynomial")
        d.free()
        copies = 40
        many = np.tile(x, copies)
        d = g.upload(many)
        g.ntt(d, d, idx, n_polys=copies, poly_stride_limbs=nl)
        eq(d, np.tile(fwd, copies), "forward, 40 polynomials")
        g.intt(d, d, idx, n_polys=copies, poly_stride_limbs=nl)
        eq(d, many, "round trip, 40 polynomials")
        d.free()
        for level in range(2, L + 1):
            c = seeded.uniform_poly(95 + level, g.primes[:level], N)
            dc = g.upload(c)
            for is_ntt in (True, False):
                dr = g.alloc((level - 1) * N)
                g.rescale(dr, dc, level, is_ntt)
                eq(dr, o.rescale(c, level, is_ntt), "rescale l=%d ntt=%d" % (level, is_ntt))
                dr.free()
            dc.free()
    finally:
        g.close()
        o.close()


def test_hw_ops(pair):
    g, o = pair.g, pair.o
    N = g.N
    for pi in sorted({0, g.L - 1, g.L, g.L + g.K - 1}):
        q = g.primes[pi]
        a = seeded.uniform_limb(20 + pi, q, N)
        b = seeded.uniform_limb(30 + pi, q, N)
        r = seeded.uniform_limb(40 + pi, q, N)
        a[:4] = [0, q - 1, q - 1, 1]
        b[:4] = [0, q - 1, 1, q - 1]
        sc = int(seeded.uniform_limb(50 + pi, q, 1)[0])
        da, db = g.upload(a), g.upload(b)
        for name in ("modadd", "modsub", "modmul", "modmuladd"):
            dr = g.upload(r)
            g.hw(name, dr, da, db, pi)
            eq(dr, o.hw(name, a, b, pi, r=r), name)
            dr = g.upload(r)
            g.hw(name + "_scalar", dr, da, sc, pi)
            eq(dr, o.hw(name + "_scalar", a, sc, pi, r=r), name + "_scalar")
        # in-place and odd lengths
        n = N - 1 if N > 4 else N
        dr = g.upload(a)
        g.hw("modmul", dr, dr, db, pi, n=n)
        want = a.copy()
        want[:n] = o.hw("modmul", a[:n], b[:n], pi)
        eq(dr, want, "in-place modmul, n=%d" % n)
        for rot, is_ntt in ((1, True), (-2, True), (3, False), (2 * N - 1, True)):
            k = g.find_automorphism_index(rot)
            assert k == o.find_automorphism_index(rot)
            dord = g.automorphism_order(k, is_ntt)
            eq(dord, o.automorphism_order(k, is_ntt), "order table")
            dr = g.alloc(N)
            g.hw("rotate", dr, da, dord, pi)
            eq(dr, o.hw("rotate", a, o.automorphism_order(k, is_ntt), pi), "rotate %d" % rot)


def test_poly_ops(pair):
    g, o = pair.g, pair.o
    N = g.N
    for level in sorted({1, g.L}):
        for with_p in (False, True):
            pr = [g.primes[i] for i in g.limb_primes(level, with_p)]
            a = seeded.uniform_poly(60 + level, pr, N)
            b = seeded.uniform_poly(70 + level, pr, N)
            da, db, dr = g.upload(a), g.upload(b), g.alloc(a.size)
            for name in ("add", "sub", "mul"):
                g.poly(name, dr, da, db, level, with_p)
                eq(dr, o.poly(name, a, b, level, with_p), "poly_%s level %d p %d" % (name, level, with_p))
            k = g.find_automorphism_index(5)
            dord = g.automorphism_order(k, True)
            g.poly("automorphism", dr, da, dord, level, with_p)
            eq(dr, o.poly("automorphism", a, o.automorphism_order(k, True), level, with_p), "automorphism")


def levels_of(g):
    return sorted({1, 2, g.part_size, min(g.L, g.part_size + 1), g.L} & set(range(1, g.L + 1)))


def test_decomp_modup_and_precomp(pair):
    g, o = pair.g, pair.o
    N = g.N
    for level in levels_of(g):
        c = seeded.uniform_poly(100 + level, g.primes[:level], N)
        dc = g.upload(c)
        nd = g.num_decomp(level)
        T = level + g.K
        for is_ntt in (True, False):
            for part in range(nd):
                dr = g.alloc(T * N)
                g.decomp_modup(dr, dc, level, part, is_ntt)
                want = o.decomp_modup(c, level, part, is_ntt)
                eq(dr, want, "decomp_modup l=%d part=%d ntt=%d" % (level, part, is_ntt))
                # Decomp then Mod_up: the digit handed over as a compact copy
                start = g.part_size * part
                length = min(g.part_size, level - start)
                dd = g.upload(c[start * N:(start + length) * N])
                dr2 = g.alloc(T * N)
                g.mod_up(dr2, dd, level, part, is_ntt)
                eq(dr2, want, "mod_up l=%d part=%d ntt=%d" % (level, part, is_ntt))
            dr = g.alloc(nd * T * N)
            g.precomp(dr, dc, level, is_ntt)
            eq(dr, o.precomp(c, level, is_ntt), "precomp l=%d ntt=%d" % (level, is_ntt))
        eq(dc, c, "source untouched")


def test_mod_down_rescale_extend(pair):
    g, o = pair.g, pair.o
    N = g.N
    for level in levels_of(g):
        pr = [g.primes[i] for i in g.limb_primes(level)]
        e = seeded.uniform_poly(200 + level, pr, N)
        c = seeded.uniform_poly(210 + level, g.primes[:level], N)
        de, dc = g.upload(e), g.upload(c)
        for is_ntt in (True, False):
            dr = g.alloc(level * N)
            g.mod_down(dr, de, level, is_ntt)
            eq(dr, o.mod_down(e, level, is_ntt), "mod_down l=%d ntt=%d" % (level, is_ntt))
            if level >= 2:
                dr = g.alloc((level - 1) * N)
                g.rescale(dr, dc, level, is_ntt)
                eq(dr, o.rescale(c, level, is_ntt), "rescale l=%d ntt=%d" % (level, is_ntt))
        dr = g.alloc((level + g.K) * N)
        g.extend(dr, dc, level)
        eq(dr, o.extend(c, level), "extend")
        # Extend -> Mod_down is the identity (ut_poly.cxx:444-480)
        dm = g.alloc(level * N)
        g.mod_down(dm, dr, level, True)
        eq(dm, c, "extend->mod_down identity")
    if g.L >= 2:
        with pytest.raises(acefhe.AceError):
            g.rescale(g.alloc(N), g.alloc(N), 1, True)


def test_ext_rotate_equals_its_parts(pair):
    """The fused extended-basis rotation = two inner products with the key halves, the addend, two automorphisms
    (each of which is checked against the oracle on its own)."""
    g = pair.g
    N = g.N
    for level in sorted({g.L, max(1, g.L - 1)}):
        nd, T = g.num_decomp(level), level + g.K
        pr = [g.primes[i] for i in g.limb_primes(level)]
        digits = g.upload(np.concatenate([seeded.uniform_poly(8000 + d, pr, N) for d in range(nd)]))
        swk = g.upload(make_swk(g, 8100 + level))
        addend = g.upload(seeded.uniform_poly(8200, pr, N))
        half = (g.L + g.K) * N
        for rot in (1, -3):
            order = g.automorphism_order(g.find_automorphism_index(rot), True)
            t0, t1, w0, w1 = (g.alloc(T * N) for _ in range(4))
            g.dot_prod(t0, digits, swk, 2 * half, nd, level)
            g.dot_prod(t1, digits, swk.view(half, swk.n - half), 2 * half, nd, level)
            for with_addend in (True, False):
                if with_addend:
                    g.poly("add", t0, t0, addend, level, True)
                g.poly("automorphism", w0, t0, order, level, True)
                g.poly("automorphism", w1, t1, order, level, True)
                r0, r1 = g.alloc(T * N), g.alloc(T * N)
                g.ext_rotate(r0, r1, digits, swk, half, 2 * half, nd, addend if with_addend else None, order, level)
                eq(r0, w0.get(), "first half, level %d rot %d addend %d" % (level, rot, with_addend))
                eq(r1, w1.get(), "second half, level %d rot %d" % (level, rot))
                # running sums: the second call adds to the first half only, the third to both
                g.ext_rotate(r0, r1, digits, swk, half, 2 * half, nd, addend if with_addend else None, order, level, 1)
                g.poly("add", w0, w0, w0, level, True)
                eq(r0, w0.get(), "first half accumulated")
                eq(r1, w1.get(), "second half overwritten")
                g.ext_rotate(r0, r1, digits, swk, half, 2 * half, nd, None, order, level, 3)
                g.poly("automorphism", w0, t0, order, level, True)  # t0 still holds dot (+ addend)
                if with_addend:  # undo for the pass without
                    g.dot_prod(t0, digits, swk, 2 * half, nd, level)
                plain0 = g.alloc(T * N)
                g.poly("automorphism", plain0, t0, order, level, True)
                # r0 = 2 * sigma(dot + addend) + sigma(dot), r1 = 2 * sigma(dot1)
                want0, want1 = g.alloc(T * N), g.alloc(T * N)
                g.poly("add", want0, w0, w0, level, True)
                g.poly("add", want0, want0, plain0, level, True)
                g.poly("add", want1, w1, w1, level, True)
                eq(r0, want0.get(), "first half accumulated twice")
                eq(r1, want1.get(), "second half accumulated")
            with pytest.raises(acefhe.AceError):
                g.ext_rotate(digits.view(0, T * N), r1, digits, swk, half, 2 * half, nd, None, order, level)


def test_mod_down_and_rescale_issued_in_pairs(pair):
    """Two Mod_down (or Rescale) calls in a row go through one set of launches when their buffers allow it; the
    results are those of the calls made one at a time, also when the second reads what the first wrote, when both
    read the same operand, when the kinds or levels differ, and with recording switched off."""
    g, o = pair.g, pair.o
    N, K = g.N, g.K
    for level in [l for l in levels_of(g) if l >= 2][-2:]:
        pr = [g.primes[i] for i in g.limb_primes(level)]
        e1, e2 = seeded.uniform_poly(300 + level, pr, N), seeded.uniform_poly(310 + level, pr, N)
        c1, c2 = e1[:level * N].copy(), e2[:level * N].copy()
        for is_ntt in (True, False):
            w1, w2 = o.mod_down(e1, level, is_ntt), o.mod_down(e2, level, is_ntt)
            v1, v2 = o.rescale(c1, level, is_ntt), o.rescale(c2, level, is_ntt)
            for batching in (True, False):
                g.set_batching(batching)
                d1, d2 = g.upload(e1), g.upload(e2)
                r1, r2, r3 = g.alloc(level * N), g.alloc(level * N), g.alloc(level * N)
                g.mod_down(r1, d1, level, is_ntt)
                g.mod_down(r2, d2, level, is_ntt)  # independent: paired
                g.mod_down(r3, d1, level, is_ntt)  # waits alone; the download sends it off
                eq(r1, w1, "first of a pair")
                eq(r2, w2, "second of a pair")
                eq(r3, w1, "a call left waiting")
                g.mod_down(r1, d2, level, is_ntt)
                g.mod_down(r2, d2, level, is_ntt)  # same operand twice
                eq(r1, w2, "shared operand, first")
                eq(r2, w2, "shared operand, second")
                # the second reads what the first writes: d3 = [Mod_down(e1) | P part of e2]
                d3 = g.upload(e2)
                g.mod_down(d3.view(0, level * N), d1, level, is_ntt)
                g.mod_down(r3, d3, level, is_ntt)
                chained = np.concatenate([w1, e2[level * N:]])
                eq(r3, o.mod_down(chained, level, is_ntt), "second depends on first")
                # rescale pairs, and a rescale after a Mod_down
                dc1, dc2 = g.upload(c1), g.upload(c2)
                s1, s2 = g.alloc((level - 1) * N), g.alloc((level - 1) * N)
                g.rescale(s1, dc1, level, is_ntt)
                g.rescale(s2, dc2, level, is_ntt)
                eq(s1, v1, "rescale, first of a pair")
                eq(s2, v2, "rescale, second of a pair")
                g.mod_down(r1, d1, level, is_ntt)
                g.rescale(s1, r1, level, is_ntt)  # a different kind, and it reads the pending result
                eq(s1, o.rescale(w1, level, is_ntt), "rescale of a pending Mod_down")
                g.rescale(s1, dc1, level, is_ntt)
                g.rescale(s1, dc2, level, is_ntt)  # same destination: the later call wins
                eq(s1, v2, "two calls into one buffer")
                for b in (d1, d2, d3, r1, r2, r3, dc1, dc2, s1, s2):
                    b.free()
            g.set_batching(True)


def test_mod_down_rescale_family(pair):
    """Mod_down_rescale, Reduce_and_rescale_modup (both mutate their operand) and Transform_values_from_level0."""
    g, o = pair.g, pair.o
    N = g.N
    for level in [l for l in levels_of(g) if l >= 2]:
        pr = [g.primes[i] for i in g.limb_primes(level)]
        e = seeded.uniform_poly(250 + level, pr, N)
        for is_ntt in (True, False):
            want, left = o.mod_down_rescale(e, level, is_ntt)
            de = g.upload(e)
            dr = g.alloc((level - 1) * N)
            g.mod_down_rescale(dr, de, level, is_ntt)
            eq(dr, want, "mod_down_rescale l=%d ntt=%d" % (level, is_ntt))
            eq(de, left, "mod_down_rescale operand afterwards l=%d ntt=%d" % (level, is_ntt))
            wres, wraised, left = o.reduce_rescale_modup(e, level, is_ntt)
            de = g.upload(e)
            dres, draised = g.alloc(level * N), g.alloc(wraised.size)
            g.reduce_rescale_modup(dres, draised, de, level, is_ntt)
            eq(dres, wres, "reduce_rescale_modup res l=%d ntt=%d" % (level, is_ntt))
            eq(draised, wraised, "reduce_rescale_modup raised l=%d ntt=%d" % (level, is_ntt))
            eq(de, left, "reduce_rescale_modup operand afterwards l=%d ntt=%d" % (level, is_ntt))
    for level in levels_of(g):
        x = seeded.uniform_limb(260 + level, g.primes[0], N)
        x[:3] = [0, g.primes[0] - 1, g.primes[0] // 2 + 1][:min(3, N)]
        dx = g.upload(x)
        dr = g.alloc(level * N)
        g.transform_from_level0(dr, dx, level)
        eq(dr, o.transform_from_level0(x, level), "transform_from_level0 l=%d" % level)
    with pytest.raises(acefhe.AceError):
        g.mod_down_rescale(g.alloc(N), g.alloc(N), 1, True)


def test_encode_real_batch_equals_single_encodes(pair):
    """ace_encode_real_batch: several real-valued vectors in one set of launches give, each, the polynomial of its
    own ace_encode_real call (which test_encode compares with the oracle), with padding between the results left
    alone, for floats and doubles, scale degrees 1 and 2, with and without P limbs."""
    g = pair.g
    N, (q0_bits, sf_bits) = g.N, pair.cfg[2:4]
    rng = np.random.default_rng(N + 77)
    for slots, n in ((N // 2, N // 2), (N // 2, max(1, N // 8)), (max(1, N // 4), max(1, N // 4))):
        for level, deg, pc in ((g.L, 1, 0), (g.L, 2, 0), (max(1, g.L - 1), 1, g.K)):
            if deg * sf_bits >= q0_bits + (level - 1) * sf_bits:
                continue
            words = (level + pc) * N
            stride = words + N  # one limb of padding
            for dt in (np.float32, np.float64):
                vecs = [rng.uniform(-2, 2, n).astype(dt) for _ in range(5)]
                out = g.alloc(5 * stride)
                g.encode_real_batch(out, stride, vecs, slots, level, deg, pc)
                got = out.get()
                one = g.alloc(words)
                for v, x in enumerate(vecs):
                    g.encode_real(one, x, slots, level, deg, pc)
                    eq(got[v * stride:v * stride + words], one.get(), "vector %d of the batch (%s, slots %d, n %d, level %d, degree %d, p %d)" % (v, dt.__name__, slots, n, level, deg, pc))
                    assert not got[v * stride + words:(v + 1) * stride].any(), "padding written"
                out.free()
                one.free()
    with pytest.raises(acefhe.AceError):
        g.encode_real_batch(g.alloc(4 * N * g.L), N, [np.zeros(4), np.zeros(4)], 0, g.L, 1, 0)  # stride too small


def test_decode(pair):
    """Device decoder vs the oracle's (itself matched against the reference's compiled Decode): the same doubles.
    Operands: encoded messages (small centred values), and uniformly random residues (integers as large as Q, both
    signs, every word of the multi-word reconstruction in use), in NTT and in coefficient form."""
    g, o = pair.g, pair.o
    N, (q0_bits, sf_bits) = g.N, pair.cfg[2:4]
    rng = np.random.default_rng(N + 5)
    for slots in sorted({N // 2, max(1, N // 8), min(4, N // 2), 1}):
        z = rng.uniform(-1, 1, slots) + 1j * rng.uniform(-1, 1, slots)
        for level in sorted({g.L, min(2, g.L), 1, max(1, g.L - 1)}):
            if sf_bits >= q0_bits + (level - 1) * sf_bits:
                continue
            enc = o.encode(z, slots, level, 1, 0)
            factor = 2.0 ** sf_bits
            got = g.decode(g.upload(enc), level, slots, factor, True)
            want = o.decode(enc, level, slots, factor, True)
            assert np.array_equal(got.view(np.uint64), want.view(np.uint64)), "decode slots=%d level=%d" % (slots, level)
            assert np.abs(got - z).max() < 1e-6
            noise = np.concatenate([rng.integers(0, q, N, dtype=np.int64) for q in g.primes[:level]])
            for is_ntt in (True, False):
                d = g.upload(noise)
                got = g.decode(d, level, slots, factor * 3.0, is_ntt)
                want = o.decode(noise, level, slots, factor * 3.0, is_ntt)
                assert np.array_equal(got.view(np.uint64), want.view(np.uint64)), "decode of random residues slots=%d level=%d ntt=%d" % (slots, level, is_ntt)
                assert np.array_equal(d.get(), noise)  # the operand is left as it was
    # the integers at the sign change and the ends of the range: x = 0, 1, (Q-1)/2, (Q+1)/2, Q-1
    level = g.L
    Q = 1
    for q in g.primes[:level]:
        Q *= int(q)
    vals = [0, 1, (Q - 1) // 2, (Q + 1) // 2, Q - 1, Q // 3][:N]
    poly = np.zeros((level, N), np.int64)
    for k, v in enumerate(vals):
        for t, q in enumerate(g.primes[:level]):
            poly[t, k] = v % int(q)
    got = g.decode(g.upload(poly.reshape(-1)), level, N // 2, 1.0, False)
    want = o.decode(poly.reshape(-1), level, N // 2, 1.0, False)
    assert np.array_equal(got.view(np.uint64), want.view(np.uint64))
    with pytest.raises(acefhe.AceError):
        g.decode(g.upload(poly.reshape(-1)), g.L + 1, 0, 1.0, False)
    with pytest.raises(acefhe.AceError):
        g.decode(g.upload(poly.reshape(-1)), 1, 3, 1.0, False)


def test_encode(pair):
    """Device encoder vs the oracle's (itself matched against the reference's compiled encoder): same residues."""
    g, o = pair.g, pair.o
    N, (q0_bits, sf_bits) = g.N, pair.cfg[2:4]
    rng = np.random.default_rng(N)
    for slots in sorted({N // 2, max(1, N // 8), min(4, N // 2), 1}):
        z = rng.uniform(-1, 1, slots) + 1j * rng.uniform(-1, 1, slots)
        for level, deg, pc in ((g.L, 1, 0), (min(2, g.L), 1, 0), (g.L, 2, 0), (g.L, 3, 0), (max(1, g.L - 1), 1, g.K)):
            if deg * sf_bits >= q0_bits + (level - 1) * sf_bits:
                with pytest.raises(acefhe.AceError):
                    g.encode(g.alloc((level + pc) * N), z, slots, level, deg, pc)
                continue
            vals = z[:max(1, slots - 1)] * 3.0
            want = o.encode(vals, slots, level, deg, pc)
            assert want is not None
            dr = g.alloc((level + pc) * N)
            g.encode(dr, vals, slots, level, deg, pc)
            eq(dr, want, "encode slots=%d level=%d sf_degree=%d p=%d" % (slots, level, deg, pc))
            if deg == 1:  # an explicit scale that is no power of the scaling factor (Encode_at_level_with_scale)
                scale = 1.5 * 2.0 ** sf_bits if level > 1 else 2.0 ** (sf_bits - 7) * 1.1
                if np.log2(scale) + 3 < q0_bits + (level - 1) * sf_bits:
                    g.encode_scaled(dr, vals, slots, level, scale, pc)
                    eq(dr, o.encode_scaled(vals, slots, level, scale, pc), "encode_scaled slots=%d level=%d p=%d" % (slots, level, pc))
                for bad_scale in (0.75, 0.25, 2.0 ** (q0_bits + (level - 1) * sf_bits)):  # below 1, or too large for the level
                    with pytest.raises(acefhe.AceError, match="invalid scale"):
                        g.encode_scaled(dr, vals, slots, level, bad_scale, pc)
    # real-valued messages (doubles, floats) are widened on the device: same residues as the complex form, with
    # calls recorded and issued one by one
    for side in (True, False):
        g.set_batching(side)
        for slots, n in ((N // 2, N // 2), (N // 2, max(1, N // 8)), (max(1, N // 4), 1)):
            for level, deg, pc in ((g.L, 1, 0), (max(1, g.L - 1), 1, g.K)):
                if deg * sf_bits >= q0_bits + (level - 1) * sf_bits:
                    continue
                for dt in (np.float64, np.float32):
                    x = rng.uniform(-2, 2, n).astype(dt)
                    want = o.encode(x.astype(np.float64).astype(np.complex128), slots, level, deg, pc)
                    dr = g.alloc((level + pc) * N)
                    g.encode_real(dr, x, slots, level, deg, pc)
                    eq(dr, want, "encode_real %s n=%d slots=%d level=%d p=%d" % (dt.__name__, n, slots, level, pc))
                    # several in a row into one buffer, consumed between them
                    acc = g.alloc((level + pc) * N)
                    for rep in range(10):
                        y = rng.uniform(-1, 1, n).astype(dt)
                        g.encode_real(dr, y, slots, level, deg, pc)
                        g.copy(acc, dr)
                    eq(acc, o.encode(y.astype(np.float64).astype(np.complex128), slots, level, deg, pc), "tenth in a row")
                    dr.free()
                    acc.free()
    g.set_batching(True)
    # a value too large for the level: the reference asserts, the library reports it at the next synchronisation
    if q0_bits + (g.L - 1) * sf_bits - sf_bits < 62:
        big = np.array([2.0 ** (q0_bits + (g.L - 1) * sf_bits - sf_bits)])
        assert o.encode(big, 1, g.L, 1, 0) is None
        dr = g.alloc(g.L * N)
        g.encode(dr, big, 1, g.L, 1, 0)
        with pytest.raises(acefhe.AceError):
            g.sync()
        g.sync()  # the flag is cleared once reported


def make_swk(g, seed):
    return np.concatenate([seeded.uniform_poly(seed + i, g.primes, g.N) for i in range(2 * g.parts)])


def test_dot_prod_and_switch_key(pair):
    g, o = pair.g, pair.o
    N = g.N
    for level in sorted({g.L, max(1, g.L - 1)}):
        nd = g.num_decomp(level)
        T = level + g.K
        pr = [g.primes[i] for i in g.limb_primes(level)]
        digits = np.concatenate([seeded.uniform_poly(300 + d, pr, N) for d in range(nd)])
        swk = make_swk(g, 400)
        kpoly = (g.L + g.K) * N
        dd, dk = g.upload(digits), g.upload(swk)
        dr = g.alloc(T * N)
        g.dot_prod(dr, dd, dk, 2 * kpoly, nd, level)
        key0 = np.concatenate([swk[2 * d * kpoly:(2 * d + 1) * kpoly] for d in range(nd)])
        eq(dr, o.dot_prod(digits, key0, nd, level), "dot_prod l=%d" % level)
        o0, o1 = g.alloc(level * N), g.alloc(level * N)
        g.fast_switch_key(o0, o1, dd, dk, level)
        zero = np.zeros(level * N, np.int64)
        # oracle: relin on precomputed digits == fast_switch_key; use fast_rotate with identity order
        ident = np.arange(N, dtype=np.int64)
        w0, w1 = o.fast_rotate(zero, digits, swk, ident, level)
        eq(o0, w0, "switch key c0")
        eq(o1, w1, "switch key c1")


def test_ciphertext_ops(pair):
    g, o = pair.g, pair.o
    N = g.N
    swk = make_swk(g, 500)
    dk = g.upload(swk)
    for level in sorted({g.L, max(2, g.L - 1)} & set(range(2, g.L + 1))):
        pr = g.primes[:level]
        a0, a1, b0, b1 = (seeded.uniform_poly(600 + i, pr, N) for i in range(4))
        da0, da1, db0, db1 = (g.upload(x) for x in (a0, a1, b0, b1))
        d = [g.alloc(level * N) for _ in range(3)]
        g.mul_ciph3(d[0], d[1], d[2], da0, da1, db0, db1, level)
        w = o.mul_ciph3(a0, a1, b0, b1, level)
        for i in range(3):
            eq(d[i], w[i], "mul_ciph3 d%d" % i)
        r0, r1 = g.alloc(level * N), g.alloc(level * N)
        g.relin(r0, r1, d[0], d[1], d[2], dk, level)
        w0, w1 = o.relin(w[0], w[1], w[2], swk, level)
        eq(r0, w0, "relin c0")
        eq(r1, w1, "relin c1")
        s0, s1 = g.alloc((level - 1) * N), g.alloc((level - 1) * N)
        g.rescale_ciph(s0, s1, r0, r1, level)
        eq(s0, o.rescale(w0, level, True), "rescale_ciph c0")
        eq(s1, o.rescale(w1, level, True), "rescale_ciph c1")
        t0, t1 = g.alloc((level - 1) * N), g.alloc((level - 1) * N)
        g.mul_relin_rescale(t0, t1, da0, da1, db0, db1, dk, level)
        m0, m1 = o.mul_relin_rescale(a0, a1, b0, b1, swk, level)
        eq(t0, m0, "mul_relin_rescale c0")
        eq(t1, m1, "mul_relin_rescale c1")
        eq(s0, m0, "composite == pieces")


def test_mul_relin_rescale_batch(pair):
    """Three ciphertext pairs in one call, operands padded apart; every pair equals the oracle's single op."""
    g, o = pair.g, pair.o
    N = g.N
    if g.L < 2:
        pytest.skip("needs two levels")
    swk = make_swk(g, 900)
    dk = g.upload(swk)
    level, nb = g.L, 3
    pr = g.primes[:level]
    in_stride, out_stride = (level + 1) * N, level * N  # one limb of padding between operands
    host = [np.zeros(nb * in_stride, np.int64) for _ in range(4)]
    ops = []
    for b in range(nb):
        polys = [seeded.uniform_poly(910 + 4 * b + i, pr, N) for i in range(4)]
        ops.append(polys)
        for i in range(4):
            host[i][b * in_stride:b * in_stride + level * N] = polys[i]
    dev = [g.upload(h) for h in host]
    r0, r1 = g.alloc(nb * out_stride), g.alloc(nb * out_stride)
    g.mul_relin_rescale_batch(r0, r1, out_stride, dev[0], dev[1], dev[2], dev[3], in_stride, dk, level, nb)
    got0, got1 = r0.get(), r1.get()
    n = (level - 1) * N
    for b in range(nb):
        m0, m1 = o.mul_relin_rescale(*ops[b], swk, level)
        eq(got0[b * out_stride:b * out_stride + n], m0, "batch[%d] c0" % b)
        eq(got1[b * out_stride:b * out_stride + n], m1, "batch[%d] c1" % b)
        assert not got0[b * out_stride + n:(b + 1) * out_stride].any(), "padding written"
    g.mul_relin_rescale_batch(r0, r1, 0, dev[0], dev[1], dev[2], dev[3], 0, dk, level, 0)  # empty batch: no-op
    with pytest.raises(acefhe.AceError):
        g.mul_relin_rescale_batch(r0, r1, n - 1, dev[0], dev[1], dev[2], dev[3], in_stride, dk, level, 2)  # overlap


def test_mul_relin_double_rescale_equals_its_three_calls(pair):
    """2ab one level down in one call (Mul_ciphertext, the product added to itself, Rescale_ciphertext): the words of
    ace_mul_ciph3, ace_relin, an elementwise sum and ace_rescale_ciph issued one after the other, each of which the
    oracle pins; likewise ace_mul_relin_rescale without the sum."""
    g = pair.g
    N = g.N
    if g.L < 2:
        pytest.skip("needs two levels")
    big_ring_skip(N)
    swk = g.alloc(2 * g.parts * (g.L + g.K) * N)
    for i in range(2 * g.parts):
        g.sample_uniform(swk.view(i * (g.L + g.K) * N, (g.L + g.K) * N), g.L, True, 7, 990 + i)
    for level in sorted({g.L, max(2, g.L - 1), 2}):
        a = [draw_poly(g, 1000 + 4 * level + i, level, False)[1] for i in range(4)]
        d = [g.alloc(level * N) for _ in range(3)]
        r0, r1, s0, s1 = (g.alloc(level * N) for _ in range(4))
        n = (level - 1) * N
        for twice in (False, True):
            g.mul_ciph3(d[0], d[1], d[2], a[0], a[1], a[2], a[3], level)
            g.relin(r0, r1, d[0], d[1], d[2], swk, level)
            if twice:
                g.poly("add", r0, r0, r0, level)
                g.poly("add", r1, r1, r1, level)
            g.rescale_ciph(r0, r1, r0, r1, level)
            (g.mul_relin_double_rescale if twice else g.mul_relin_rescale)(s0, s1, a[0], a[1], a[2], a[3], swk, level)
            eq(s0.get()[:n], r0.get()[:n], "level %d twice=%d c0" % (level, twice))
            eq(s1.get()[:n], r1.get()[:n], "level %d twice=%d c1" % (level, twice))
        # ... and with a constant between the sum and the Rescale (a double-angle step of the sine evaluation):
        # residues of small and of large integers, of either parity in the dropped limb, and zero
        q = [int(g.primes[t]) for t in range(level)]
        for case, big in enumerate((12345678901234567, -3, (1 << 200) + 977, 0, -(1 << 131) - 2)):
            cst = [big % qt for qt in q]
            g.mul_ciph3(d[0], d[1], d[2], a[0], a[1], a[2], a[3], level)
            g.relin(r0, r1, d[0], d[1], d[2], swk, level)
            g.poly("add", r0, r0, r0, level)
            g.poly("add", r1, r1, r1, level)
            g.poly_scalars(False, r0, r0, cst, level)
            g.rescale_ciph(r0, r1, r0, r1, level)
            g.mul_relin_double_add_rescale(s0, s1, a[0], a[1], a[2], a[3], swk, cst, level)
            eq(s0.get()[:n], r0.get()[:n], "level %d constant %d c0" % (level, case))
            eq(s1.get()[:n], r1.get()[:n], "level %d constant %d c1" % (level, case))
        with pytest.raises(acefhe.AceError):
            g.mul_relin_double_add_rescale(s0, s1, a[0], a[1], a[2], a[3], swk, [q[0]] + [0] * (level - 1), level)
        for b in a + d + [r0, r1, s0, s1]:
            b.free()
    swk.free()


def test_mod_down_pair_rescale_equals_its_calls(pair):
    """Mod_down of the two extended halves of a ciphertext followed by Rescale_ciphertext, in one call: the words of
    ace_mod_down twice and ace_rescale_ciph issued one after the other, each of which the oracle pins; at the top
    level, one below, and the lowest that can be rescaled; overlapping operands are rejected."""
    g = pair.g
    N = g.N
    if g.L < 2:
        pytest.skip("needs two levels")
    big_ring_skip(N)
    for level in sorted({g.L, max(2, g.L - 1), 2}):
        e = [draw_poly(g, 1100 + 2 * level + i, level, True)[1] for i in range(2)]
        kept = [b.get() for b in e]
        m0, m1, r0, r1, s0, s1 = (g.alloc(level * N) for _ in range(6))
        g.mod_down(m0, e[0], level)
        g.mod_down(m1, e[1], level)
        g.rescale_ciph(r0, r1, m0, m1, level)
        g.mod_down_pair_rescale(s0, s1, e[0], e[1], level)
        n = (level - 1) * N
        eq(s0.get()[:n], r0.get()[:n], "level %d c0" % level)
        eq(s1.get()[:n], r1.get()[:n], "level %d c1" % level)
        eq(e[0], kept[0], "operand 0 untouched")
        eq(e[1], kept[1], "operand 1 untouched")
        with pytest.raises(acefhe.AceError):
            g.mod_down_pair_rescale(e[0], s1, e[0], e[1], level)
        for b in e + [m0, m1, r0, r1, s0, s1]:
            b.free()
    with pytest.raises(acefhe.AceError):
        e0, e1 = (g.alloc((1 + g.K) * N) for _ in range(2))
        try:
            g.mod_down_pair_rescale(e0, e1, e0, e1, 1)  # nothing to drop at level 1
        finally:
            e0.free()
            e1.free()


def test_two_lanes_equal_one(pair):
    """ace_fork / ace_fork_switch / ace_join: two independent sequences of calls (HMult + relinearise + rescale, a
    transform there and back, recorded elementwise calls, buffers allocated and freed on the way) issued on the two
    lanes give the results of issuing them one after the other, repeatedly, with the lanes' buffer pools warm and
    cold; misuse is rejected."""
    g = pair.g
    N = g.N
    if g.L < 2:
        pytest.skip("needs two levels")
    big_ring_skip(N)
    level = g.L
    pr = g.primes[:level]
    dk = g.upload(make_swk(g, 1900))
    idx = list(range(level - 1))

    def sequence(seed):
        a0, a1, b0, b1 = (g.upload(seeded.uniform_poly(seed + i, pr, N)) for i in range(4))
        r0, r1 = g.alloc((level - 1) * N), g.alloc((level - 1) * N)
        g.mul_relin_rescale(r0, r1, a0, a1, b0, b1, dk, level)
        t = g.alloc((level - 1) * N)
        g.intt(t, r0, idx)
        g.ntt(t, t, idx)
        for limb in range(level - 1):  # recorded calls: r1 += t * r0, limb by limb
            g.hw("modmuladd", r1.view(limb * N, N), t.view(limb * N, N), r0.view(limb * N, N), limb)
        for b in (a0, a1, b0, b1, t):
            b.free()
        return r0, r1

    want = [[x.get() for x in sequence(2000 + 10 * k)] for k in range(2)]
    for rep in range(4):
        g.fork()
        second = sequence(2010)
        g.fork_switch()
        first = sequence(2000)
        g.join()
        for k, res in enumerate((first, second)):
            for j in range(2):
                eq(res[j], want[k][j], "lane %d result %d, repetition %d" % (k, j, rep))
                res[j].free()
    g.fork()
    g.join()  # nothing issued on the second lane
    with pytest.raises(acefhe.AceError):
        g.join()
    with pytest.raises(acefhe.AceError):
        g.fork_switch()
    g.fork()
    with pytest.raises(acefhe.AceError):
        g.fork()
    g.join()


def test_contexts_of_a_family_on_two_threads(pair):
    """ace_ctx_share: a second context over the same tables, used from another host thread at the same time as the
    first: each thread's HMult + relinearise + rescale and rotation are the words of the same calls made alone, a
    buffer that one context allocated is read by the other and freed through it."""
    import threading

    g, o = pair.g, pair.o
    N, level = g.N, g.L
    if level < 2:
        pytest.skip("needs two limbs")
    if N > 8192:
        pytest.skip("covered at the smaller rings (N = 65536: the ResNet-20 program on three threads)")
    pr = g.primes[:level]
    swk = make_swk(g, 4100)
    ops = [tuple(seeded.uniform_poly(4000 + 10 * t + i, pr, N) for i in range(4)) for t in range(2)]
    want = [o.mul_relin_rescale(*ops[t], swk, level) for t in range(2)]
    h = g.share()
    try:
        dswk = g.upload(swk)  # allocated by the first context, used by both
        ctxs, got, errs = [g, h], [None, None], []

        def work(t):
            try:
                c = ctxs[t]
                d = [c.upload(v) for v in ops[t]]
                r0, r1 = c.alloc((level - 1) * N), c.alloc((level - 1) * N)
                for _ in range(8):  # long enough for the two threads' launches to interleave
                    c.mul_relin_rescale(r0, r1, d[0], d[1], d[2], d[3], dswk, level)
                got[t] = (r0.get(), r1.get())
                for b in d + [r0, r1]:
                    b.free()
            except Exception as e:  # noqa: BLE001 -- reported by the main thread
                errs.append(e)

        th = [threading.Thread(target=work, args=(t,)) for t in range(2)]
        for x in th:
            x.start()
        for x in th:
            x.join()
        assert not errs, errs
        for t in range(2):
            eq(got[t][0], want[t][0], "thread %d c0" % t)
            eq(got[t][1], want[t][1], "thread %d c1" % t)
        # a buffer of the first context freed through the second: accepted (the family keeps one record)
        before = g.memory_stats()[2]
        buf = g.alloc(N)
        assert g.memory_stats()[2] == before + 1
        h.lib.ace_free(h.h, buf.ptr)
        buf.ptr = None
        assert g.memory_stats()[2] == before
    finally:
        h.close()


def test_rotation_many(pair):
    """More rotations than one batched launch holds (small rings only: the oracle does each one)."""
    g, o = pair.g, pair.o
    N = g.N
    if N < 16 or N > 2048:
        pytest.skip("covered at one size class")
    level = g.L
    pr = g.primes[:level]
    c0, c1 = seeded.uniform_poly(750, pr, N), seeded.uniform_poly(751, pr, N)
    dc0, dc1 = g.upload(c0), g.upload(c1)
    rots = [int(r) for r in 1 + seeded.splitmix64(77, 35) % np.uint64(N // 2 - 1)]
    base = make_swk(g, 850)
    swks = [(base + i) % np.tile(np.repeat(np.array(g.primes, np.int64), N), 2 * g.parts) for i in range(len(rots))]
    orders = [o.automorphism_order(o.find_automorphism_index(r), True) for r in rots]
    digits = o.precomp(c1, level, True)
    dswk = [g.upload(s) for s in swks]
    dord = [g.automorphism_order(g.find_automorphism_index(r), True) for r in rots]
    n = level * N
    r0s, r1s = g.alloc(len(rots) * n), g.alloc(len(rots) * n)
    g.rotate_batch(r0s, r1s, dc0, dc1, dswk, dord, level)
    got0, got1 = r0s.get(), r1s.get()
    for i in range(len(rots)):
        w0, w1 = o.fast_rotate(c0, digits, swks[i], orders[i], level)
        eq(got0[i * n:(i + 1) * n], w0, "rotate_batch[%d] c0" % i)
        eq(got1[i * n:(i + 1) * n], w1, "rotate_batch[%d] c1" % i)


def test_rotation(pair):
    g, o = pair.g, pair.o
    N = g.N
    level = g.L
    pr = g.primes[:level]
    c0, c1 = seeded.uniform_poly(700, pr, N), seeded.uniform_poly(701, pr, N)
    dc0, dc1 = g.upload(c0), g.upload(c1)
    rots = [1, -1, 3] if N > 4 else [1]
    swks = [make_swk(g, 800 + i) for i in range(len(rots))]
    orders = [o.automorphism_order(o.find_automorphism_index(r), True) for r in rots]
    digits = o.precomp(c1, level, True)
    dswk = [g.upload(s) for s in swks]
    dord = [g.automorphism_order(g.find_automorphism_index(r), True) for r in rots]
    n = level * N
    r0s, r1s = g.alloc(len(rots) * n), g.alloc(len(rots) * n)
    g.rotate_batch(r0s, r1s, dc0, dc1, dswk, dord, level)
    got0, got1 = r0s.get(), r1s.get()
    for i in range(len(rots)):
        w0, w1 = o.fast_rotate(c0, digits, swks[i], orders[i], level)
        eq(got0[i * n:(i + 1) * n], w0, "rotate_batch[%d] c0" % i)
        eq(got1[i * n:(i + 1) * n], w1, "rotate_batch[%d] c1" % i)
    dd = g.upload(digits)
    r0, r1 = g.alloc(n), g.alloc(n)
    g.fast_rotate(r0, r1, dc0, dd, dswk[0], dord[0], level)
    eq(r0, got0[:n], "fast_rotate == batch[0]")
    eq(r1, got1[:n], "fast_rotate == batch[0] c1")
    # index tables the caller uploads itself: one of the automorphism's make (on large rings applied inside the
    # transform's last kernel, once the library has examined it), and a permutation that is no automorphism and
    # scatters every block of the result over the whole source (the separate pass): result[i] = value at table[i]
    k = len(rots) - 1
    mine = g.upload(np.asarray(orders[k], dtype=np.int64))
    g.fast_rotate(r0, r1, dc0, dd, dswk[k], mine, level)
    eq(r0, got0[k * n:(k + 1) * n], "caller's copy of an automorphism table")
    eq(r1, got1[k * n:(k + 1) * n], "caller's copy of an automorphism table, c1")
    scatter = (np.arange(N, dtype=np.int64) * 5 + 3) % N
    w0, w1 = o.fast_rotate(c0, digits, swks[0], scatter, level)
    other = g.upload(scatter)
    for _ in range(2):  # the second call finds the verdict on the table cached
        g.fast_rotate(r0, r1, dc0, dd, dswk[0], other, level)
        eq(r0, w0, "a table that is no automorphism")
        eq(r1, w1, "a table that is no automorphism, c1")
    # the same buffer rewritten through the library: the verdict on the old contents must not survive
    other.set(np.asarray(orders[0], dtype=np.int64))
    g.fast_rotate(r0, r1, dc0, dd, dswk[0], other, level)
    eq(r0, got0[:n], "table buffer rewritten")
    mine.set(scatter)
    g.fast_rotate(r0, r1, dc0, dd, dswk[0], mine, level)
    eq(r0, w0, "table buffer rewritten with a table that is no automorphism")
    # results that overlap c0 or the digits would be read after they are written
    with pytest.raises(acefhe.AceError, match="overlap"):
        g.fast_rotate(dc0.view(0, n), r1, dc0, dd, dswk[0], dord[0], level)
    with pytest.raises(acefhe.AceError, match="overlap"):
        g.fast_rotate(r0, dd.view(N, n), dc0, dd, dswk[0], dord[0], level)
    if len(rots) > 1:
        inside = g.alloc(len(rots) * n)
        with pytest.raises(acefhe.AceError, match="overlap"):
            g.rotate_batch(inside, r1s, inside.view(n, n), dc1, dswk, dord, level)


def test_rejected_calls(pair):
    g = pair.g
    N = g.N
    buf = g.alloc(N)
    with pytest.raises(acefhe.AceError):
        g.ntt(buf, buf, [g.L + g.K])
    with pytest.raises(acefhe.AceError):
        g.decomp_modup(buf, buf, g.L + 1, 0)
    with pytest.raises(acefhe.AceError):
        g.decomp_modup(buf, buf, g.L, g.parts)
    with pytest.raises(acefhe.AceError):
        g.hw("rotate", buf, buf, buf, 0)
    with pytest.raises(acefhe.AceError):
        g.hw("modmul_scalar", buf, buf, g.primes[0], 0)
    g.ntt(buf, buf, [], n_polys=0)  # empty input is a no-op
    g.hw("modadd", buf, buf, buf, 0, n=0)


def test_ext_plain_mac(pair):
    """Sum of plaintext products in the extended domain against limb-wise modmul / modadd of the oracle:
    plaintexts kept at a higher level than the ciphertext, 35 operands (two launches), then accumulation."""
    g, o = pair.g, pair.o
    N, L, K = g.N, g.L, g.K
    big_ring_skip(N)
    level = max(1, L - 1)
    idx_ct = list(range(level)) + list(range(L, L + K))
    count = 35
    a0, d0 = zip(*[draw_poly(g, 3000 + j, level, True) for j in range(count)])
    a1, d1 = zip(*[draw_poly(g, 3100 + j, level, True) for j in range(count)])
    pl, dp = zip(*[draw_poly(g, 3200 + j, L, True) for j in range(count)])  # L Q limbs, then the P limbs
    d0, d1, dp = list(d0), list(d1), list(dp)
    pick = np.concatenate([np.arange(level * N), np.arange(L * N, (L + K) * N)])

    def mac(acc, xs):
        out = acc.copy()
        for x, p in zip(xs, pl):
            pv = p[pick]
            for t, pi in enumerate(idx_ct):
                sl = slice(t * N, (t + 1) * N)
                out[sl] = o.hw("modadd", out[sl], o.hw("modmul", x[sl], pv[sl], pi), pi)
        return out
    zero = np.zeros((level + K) * N, np.int64)
    w0, w1 = mac(zero, a0), mac(zero, a1)
    r0, r1 = g.alloc((level + K) * N), g.alloc((level + K) * N)
    g.ext_plain_mac(r0, r1, d0, d1, dp, level, L)
    eq(r0.get(), w0, "ext_plain_mac c0")
    eq(r1.get(), w1, "ext_plain_mac c1")
    g.ext_plain_mac(r0, r1, d0[:3], d1[:3], dp[:3], level, L, accumulate=True)
    eq(r0.get(), mac(w0, a0[:3]), "ext_plain_mac accumulate c0")
    eq(r1.get(), mac(w1, a1[:3]), "ext_plain_mac accumulate c1")
    with pytest.raises(RuntimeError):
        g.ext_plain_mac(r0, r1, [r0], d1[:1], dp[:1], level, L)
    with pytest.raises(RuntimeError):
        g.ext_plain_mac(r0, r1, d0[:1], d1[:1], dp[:1], L, level)


def test_ext_plain_mac_groups_equal_single_groups(pair):
    """Several baby-step groups over the same operands in one call = one ace_ext_plain_mac per group (checked against
    the oracle above): 6 groups (two launches of up to four), 19 operands (two launches of up to sixteen), terms
    missing from some groups."""
    g = pair.g
    N, L, K = g.N, g.L, g.K
    big_ring_skip(N)
    level = max(1, L - 1)
    count, groups = 19, 6
    d0 = [draw_poly(g, 3300 + j, level, True)[1] for j in range(count)]
    d1 = [draw_poly(g, 3400 + j, level, True)[1] for j in range(count)]
    dp = [[draw_poly(g, 3500 + 40 * b + j, L, True)[1] for j in range(count)] for b in range(groups)]
    dp[1][4] = dp[5][18] = dp[5][0] = None
    T = level + K
    r0s, r1s = [g.alloc(T * N) for _ in range(groups)], [g.alloc(T * N) for _ in range(groups)]
    g.ext_plain_mac_groups(r0s, r1s, d0, d1, dp, level, L)
    w0, w1 = g.alloc(T * N), g.alloc(T * N)
    for b in range(groups):
        keep = [j for j in range(count) if dp[b][j] is not None]
        g.ext_plain_mac(w0, w1, [d0[j] for j in keep], [d1[j] for j in keep], [dp[b][j] for j in keep], level, L)
        eq(r0s[b].get(), w0.get(), "group %d, first half" % b)
        eq(r1s[b].get(), w1.get(), "group %d, second half" % b)
    with pytest.raises(RuntimeError):
        g.ext_plain_mac_groups([r0s[0], r0s[0]], r1s[:2], d0, d1, dp[:2], level, L)
    with pytest.raises(RuntimeError):
        g.ext_plain_mac_groups([d0[0]], r1s[:1], d0, d1, dp[:1], level, L)


def test_limb_scalars_and_weighted_sum(pair):
    """Per-limb scalar add / multiply and the weighted sum of ciphertexts against limb-wise oracle calls."""
    g, o = pair.g, pair.o
    N, L = g.N, g.L
    big_ring_skip(N)
    level = L
    pr = g.primes[:level]
    a, da = draw_poly(g, 4000, level, False)
    sc = np.array([int(seeded.splitmix64(4100 + t, 1)[0] % np.uint64(q)) for t, q in enumerate(pr)], np.int64)
    r = g.alloc(level * N)
    for mul, name in ((False, "modadd_scalar"), (True, "modmul_scalar")):
        g.poly_scalars(mul, r, da, sc, level)
        want = np.concatenate([o.hw(name, a[t * N:(t + 1) * N], int(sc[t]), t) for t in range(level)])
        eq(r.get(), want, name + " per limb")
    g.poly_scalars(True, da, da, sc, level)  # in place
    eq(da.get(), want, "modmul_scalar per limb, in place")
    with pytest.raises(RuntimeError):
        g.poly_scalars(True, r, da, np.array(pr, np.int64), level)  # q itself is not a residue

    count = 7
    a0, d0 = (list(v) for v in zip(*[draw_poly(g, 4200 + j, level, False) for j in range(count)]))
    a1, d1 = (list(v) for v in zip(*[draw_poly(g, 4300 + j, level, False) for j in range(count)]))
    w = np.array([[int(seeded.splitmix64(4400 + 100 * j + t, 1)[0] % np.uint64(q)) for t, q in enumerate(pr)]
                  for j in range(count)], np.int64)

    def wsum(xs):
        out = np.zeros(level * N, np.int64)
        for j, x in enumerate(xs):
            for t in range(level):
                sl = slice(t * N, (t + 1) * N)
                out[sl] = o.hw("modadd", out[sl], o.hw("modmul_scalar", x[sl], int(w[j, t]), t), t)
        return out
    r0, r1 = g.alloc(level * N), g.alloc(level * N)
    g.ciph_wsum(r0, r1, d0, d1, w, level)
    eq(r0.get(), wsum(a0), "ciph_wsum c0")
    eq(r1.get(), wsum(a1), "ciph_wsum c1")
    g.ciph_wsum(d0[0], d1[0], d0, d1, w, level)  # the result over the first operand
    eq(d0[0].get(), wsum(a0), "ciph_wsum c0 over an operand")
    eq(d1[0].get(), wsum(a1), "ciph_wsum c1 over an operand")


def test_recorded_hw_calls_equal_calls_issued_one_by_one(pair):
    """Hw_* calls are recorded and launched together; a random program of them (shared temporaries, in-place updates,
    rotates of freshly written limbs, operands that overlap out of step) must give what one launch per call gives."""
    g = pair.g
    N, L = g.N, g.L
    big_ring_skip(N)
    rng = np.random.Generator(np.random.PCG64(5 + N))
    n_limbs = 12
    prime = [int(rng.integers(0, L + g.K)) for _ in range(n_limbs)]
    host = np.concatenate([seeded.uniform_poly(6000 + t, [g.primes[prime[t]]], N) for t in range(n_limbs)])
    k = g.find_automorphism_index(1)
    order = g.automorphism_order(k, True)

    def program(buf):
        limb = lambda t: buf.view(t * N, N)
        r = np.random.Generator(np.random.PCG64(99))
        for step in range(400):
            kind = int(r.integers(0, 12))
            t = int(r.integers(0, n_limbs))
            same = [u for u in range(n_limbs) if prime[u] == prime[t]]
            a, b, d = (int(r.choice(same)) for _ in range(3))
            p = prime[t]
            if kind < 3:
                g.hw("modmul", limb(d), limb(a), limb(b), p)
            elif kind < 5:
                g.hw("modmuladd", limb(d), limb(a), limb(b), p)
            elif kind < 6:
                g.hw("modadd", limb(d), limb(d), limb(a), p)
            elif kind < 7:
                g.hw("modsub_scalar", limb(d), limb(a), int(r.integers(0, 1 << 30)), p)
            elif kind < 9:
                if d != a:
                    g.hw("rotate", limb(d), limb(a), order, p)
            elif kind == 10:
                g.copy(limb(d), limb(a))
            elif kind == 11:
                if t + 1 < n_limbs:
                    g.copy(buf.view(t * N, 2 * N), buf.view(((t + 5) % (n_limbs - 1)) * N, 2 * N)) if abs(((t + 5) % (n_limbs - 1)) - t) >= 2 else None
                g.lib.ace_zero(g.h, limb(d).ptr, N // 2)
            elif t + 1 < n_limbs and d not in (t, t + 1):
                # an operand one word out of step with limbs the run has just written: element i of it is element
                # i+1 of limb t, which another thread wrote (values need not be reduced for an addition's operand
                # to be read consistently, only the same words must be seen)
                g.hw("modadd", limb(d), limb(d), buf.view(t * N + 1, N), prime[d])
    g.set_batching(False)
    x = g.upload(host)
    program(x)
    want = x.get()
    g.set_batching(True)
    y = g.upload(host)
    program(y)
    eq(y.get(), want, "recorded run")


def test_recorded_inner_product_through_a_scratch_limb(pair):
    """The shape generated code gives a key-switch inner product: Hw_modmul into one scratch limb, Hw_modadd from it,
    limb after limb.  Recorded, the scratch limb travels in a register and its store is dropped where a later entry
    overwrites it; results, and the scratch limb's final content, are those of one launch per call -- also when the
    scratch limb is read twice, updated in place by a multiply-add, or copied before it is overwritten."""
    g = pair.g
    N, L, K = g.N, g.L, g.K
    big_ring_skip(N)
    T = min(L + K, 9)
    primes = list(range(T))
    mk = lambda seed: np.concatenate([seeded.uniform_poly(seed + t, [g.primes[primes[t]]], N) for t in range(T)])
    key, ext, acc0, spare0 = mk(7000), mk(7100), mk(7200), mk(7300)

    def program():
        dk, de, da, ds = g.upload(key), g.upload(ext), g.upload(acc0), g.upload(spare0)
        tmp, keep = g.alloc(N), g.alloc(N)
        limb = lambda buf, t: buf.view(t * N, N)
        for rep in range(2):  # the second pass starts from a scratch limb that holds a value
            for t in range(T):
                p = primes[t]
                g.hw("modmul", tmp, limb(dk, t), limb(de, t), p)
                g.hw("modadd", limb(da, t), limb(da, t), tmp, p)
                if t % 4 == 1:  # a second reader: the product has to reach memory
                    g.hw("modsub", limb(ds, t), limb(ds, t), tmp, p)
                if t % 4 == 2:  # updated in place before it is consumed
                    g.hw("modmul", tmp, limb(dk, t), limb(da, t), p)
                    g.hw("modmuladd", tmp, limb(de, t), limb(ds, t), p)
                    g.hw("modadd", limb(ds, t), limb(ds, t), tmp, p)
                if t % 4 == 3:  # copied out between the product and the sum
                    g.hw("modmul", tmp, limb(de, t), limb(de, t), p)
                    g.copy(keep, tmp)
                    g.hw("modadd", limb(da, t), limb(da, t), tmp, p)
        out = [da.get(), ds.get(), tmp.get(), keep.get()]
        for b in (dk, de, da, ds, tmp, keep):
            b.free()
        return out

    g.set_batching(False)
    want = program()
    g.set_batching(True)
    got = program()
    for w, x, what in zip(want, got, ("sums", "second readers", "scratch limb afterwards", "copy of the scratch limb")):
        eq(x, w, what)


def test_recorded_products_summed_two_halves_at_a_time(pair):
    """The shape generated code gives a convolution's sum of plaintext products: per limb, Hw_modmul of both halves
    of a ciphertext into a temporary ciphertext, then Hw_modadd of both halves into the running sum, term after term,
    the temporary freed and allocated again between terms (a released buffer that stays in the pool does not end the
    recorded run: the entries for its next owner follow those that name it now).  Results, and what the temporaries
    hold at the end, are those of one launch per call -- also where a term's product is read a second time and where
    the sum goes elsewhere than onto itself."""
    g = pair.g
    N, L = g.N, g.L
    big_ring_skip(N)
    level = min(L, 3)
    terms = 7
    mk = lambda seed: np.concatenate([seeded.uniform_poly(seed + t, [g.primes[t]], N) for t in range(level)])
    rots = [(mk(7700 + 10 * j), mk(7705 + 10 * j)) for j in range(terms)]
    plains = [mk(7800 + 10 * j) for j in range(terms)]
    start0, start1 = mk(7900), mk(7910)

    def program(realloc):
        limb = lambda buf, t: buf.view(t * N, N)
        dr = [(g.upload(a), g.upload(b)) for a, b in rots]
        dp = [g.upload(x) for x in plains]
        s0, s1, side, other = g.upload(start0), g.upload(start1), g.upload(start0), g.alloc(level * N)
        t0, t1 = g.alloc(level * N), g.alloc(level * N)
        for j in range(terms):
            if realloc and j:
                t0.free()
                t1.free()
                t0, t1 = g.alloc(level * N), g.alloc(level * N)
            for t in range(level):
                g.hw("modmul", limb(t0, t), limb(dr[j][0], t), limb(dp[j], t), t)
                g.hw("modmul", limb(t1, t), limb(dr[j][1], t), limb(dp[j], t), t)
                g.hw("modadd", limb(s0, t), limb(s0, t), limb(t0, t), t)
                if j == 2:  # the sum lands elsewhere: not a sum onto itself
                    g.hw("modadd", limb(other, t), limb(s1, t), limb(t1, t), t)
                else:
                    g.hw("modadd", limb(s1, t), limb(t1, t), limb(s1, t), t)
                if j == 4:  # a second reader of the product
                    g.hw("modsub", limb(side, t), limb(side, t), limb(t0, t), t)
        out = [s0.get(), s1.get(), side.get(), other.get(), t0.get(), t1.get()]
        for b in [s0, s1, side, other, t0, t1] + dp + [x for pr in dr for x in pr]:
            b.free()
        return out

    for realloc in (False, True):
        g.set_batching(False)
        want = program(realloc)
        g.set_batching(True)
        got = program(realloc)
        names = ("first half", "second half", "second reader", "sum elsewhere", "temporary 0 afterwards",
                 "temporary 1 afterwards")
        for w, x, what in zip(want, got, names):
            eq(x, w, "%s (temporaries allocated per term: %s)" % (what, realloc))


def test_recorded_zero_fills_that_nothing_sees(pair):
    """Generated code zero-fills every polynomial it allocates and then overwrites or accumulates into it.  Recorded,
    a fill that is overwritten before it is read is dropped, a product or a sum added to fresh zeros becomes the
    product or a copy, and a fill the flushing entry point does not touch waits for the next run.  Every buffer must
    hold what one launch per call leaves -- including a recycled buffer that held other values, which must read as
    zeros once it is looked at."""
    g = pair.g
    N, L, K = g.N, g.L, g.K
    big_ring_skip(N)
    level = min(L, 4)
    T = level
    mk = lambda seed: np.concatenate([seeded.uniform_poly(seed + t, [g.primes[t]], N) for t in range(T)])
    hx, hy = mk(7400), mk(7500)
    hext = seeded.uniform_poly(7600, [g.primes[i] for i in g.limb_primes(level)], N)

    def program():
        limb = lambda buf, t: buf.view(t * N, N)
        x, y, ext = g.upload(hx), g.upload(hy), g.upload(hext)
        dirty = g.alloc(T * N)
        for t in range(T):
            g.hw("modadd_scalar", limb(dirty, t), limb(dirty, t), 12345 + t, t)
        dirty.free()
        recycled = g.alloc(T * N)  # the buffer that held 12345...: nothing touches it until it is read back
        acc, via_tmp, over, summed, read_first, doubled, waits = (g.alloc(T * N) for _ in range(7))
        down, tmp, spare = g.alloc(level * N), g.alloc(N), g.alloc(T * N)
        for t in range(T):
            g.hw("modmuladd", limb(acc, t), limb(x, t), limb(y, t), t)  # a product added to fresh zeros
            g.hw("modmul", tmp, limb(x, t), limb(x, t), t)  # ... through a scratch limb
            g.hw("modadd", limb(via_tmp, t), limb(via_tmp, t), tmp, t)
            g.hw("modmul", limb(over, t), limb(y, t), limb(y, t), t)  # overwritten before anyone reads
            g.hw("modadd", limb(summed, t), limb(y, t), limb(summed, t), t)  # a sum with fresh zeros
            g.hw("modsub", limb(spare, t), limb(read_first, t), limb(x, t), t)  # the zeros are read
            g.hw("modadd_scalar", limb(read_first, t), limb(read_first, t), 77, t)
            g.hw("modadd", limb(doubled, t), limb(doubled, t), limb(doubled, t), t)  # 0 + 0
            g.hw("modmuladd", limb(acc, t), limb(y, t), limb(y, t), t)  # a second product on top
        g.mod_down(down, ext, level)  # names its operands: fills of other buffers wait, its result's fill is moot
        for t in range(T):
            g.hw("modmuladd_scalar", limb(waits, t), limb(x, t), 3 + t, t)
        bufs = (acc, via_tmp, over, summed, read_first, doubled, waits, recycled, down, spare)
        out = [b.get() for b in bufs]
        for b in bufs + (x, y, ext, tmp):
            b.free()
        return out

    g.set_batching(False)
    want = program()
    g.set_batching(True)
    got = program()
    names = ("product on zeros", "product through a scratch limb", "overwritten", "sum with zeros", "zeros read first",
             "zeros added to themselves", "fill that waited, then a scalar product", "recycled buffer", "mod_down result",
             "difference from zeros")
    for w, x, what in zip(want, got, names):
        eq(x, w, what)
    assert not got[7].any() and not got[5].any()


def test_key_generation_helpers(pair):
    """ace_expand_small exactly; ace_sample_uniform: in range, reproducible, streams differ, and roughly uniform
    (mean, and a chi-square over 16 buckets at 6 sigma) -- it has no counterpart to compare bits with."""
    g = pair.g
    N, L, K = g.N, g.L, g.K
    level = L
    T = level + K
    primes = list(g.primes[:level]) + list(g.primes[L:])
    rng = np.random.Generator(np.random.PCG64(8 + N))
    small = rng.integers(-3, 4, N).astype(np.int64)
    r = g.alloc(T * N)
    g.expand_small(r, small, level, True)
    want = np.concatenate([np.where(small < 0, small + int(q), small) for q in primes])
    eq(r.get(), want, "expand_small")
    with pytest.raises(RuntimeError):
        g.expand_small(r, small * (1 << 40), level, True)

    a, b, c2 = g.alloc(T * N), g.alloc(T * N), g.alloc(T * N)
    g.sample_uniform(a, level, True, 1234, 7)
    g.sample_uniform(b, level, True, 1234, 7)
    g.sample_uniform(c2, level, True, 1234, 8)
    x, y, z = a.get(), b.get(), c2.get()
    assert np.array_equal(x, y)
    if N >= 64:
        assert not np.array_equal(x, z)
    for t, q in enumerate(primes):
        v = x[t * N:(t + 1) * N]
        assert v.min() >= 0 and v.max() < int(q)
    if N >= 1024:
        u = np.concatenate([x[t * N:(t + 1) * N] / float(q) for t, q in enumerate(primes)])
        assert abs(u.mean() - 0.5) < 6 * (1 / 12) ** 0.5 / u.size ** 0.5
        counts = np.bincount((u * 16).astype(np.int64), minlength=16).astype(np.float64)
        expect = u.size / 16
        chi2 = ((counts - expect) ** 2 / expect).sum()
        assert chi2 < 15 + 6 * (2 * 15) ** 0.5
        # limbs are not copies of each other
        assert np.mean(x[:N] % 1024 == x[N:2 * N] % 1024) < 0.01 if T > 1 else True
