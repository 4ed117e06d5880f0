"""ace_mod_down_noalloc, the Mod_down that allocates nothing (its intermediates live in a device array that is part
of the library image), against ace_mod_down through the C-ABI: bit for bit, two calls in a row, the second on a
smaller input, then once more on another context of the same GPU (needs an MI355X)."""
import numpy as np
import pytest

import acefhe
import seeded

pytestmark = pytest.mark.gpu


def both(g, e, level, is_ntt):
    """(result of ace_mod_down, result of ace_mod_down_noalloc) for the extended polynomial e at `level`."""
    N = g.N
    de = g.upload(e)
    want, got = g.alloc(level * N), g.alloc(level * N)
    g.mod_down(want, de, level, is_ntt)
    w = want.get()
    before = g.memory_stats()
    g.mod_down_noalloc(got, de, level, is_ntt)
    assert g.memory_stats() == before, "the call changed the context's arena, pool or live buffers"
    r = got.get()
    assert (de.get() == e).all(), "operand changed"
    for b in (de, want, got):
        b.free()
    return w, r


@pytest.mark.parametrize("cfg", [(65536, 24, 50, 50, 3), (8192, 5, 40, 40, 3), (2048, 4, 55, 50, 2)],
                         ids=lambda c: "N%d_L%d" % (c[0], c[1]))
def test_mod_down_noalloc_equals_mod_down(cfg):
    print("config", cfg, flush=True)
    g = acefhe.Context(*cfg)
    assert g.has_device, "no GPU visible"
    try:
        N, L = g.N, g.L
        # the larger input first, then a smaller one: the second call finds the first call's words in the array
        for level in (L, max(1, L // 2), 1):
            pr = [g.primes[i] for i in g.limb_primes(level)]
            e = seeded.uniform_poly(9000 + level, pr, N)
            for is_ntt in (True, False):
                w, r = both(g, e, level, is_ntt)
                bad = np.nonzero(w != r)[0]
                assert bad.size == 0, "level %d ntt %d: %d words differ, first at %d" % (level, is_ntt, bad.size, bad[0])
        # a second context on the same GPU shares the array; used one after the other they agree as well
        h = acefhe.Context(*cfg)
        try:
            pr = [h.primes[i] for i in h.limb_primes(L)]
            e = seeded.uniform_poly(9100, pr, N)
            w, r = both(h, e, L, True)
            assert (w == r).all(), "second context"
        finally:
            h.close()
        # a few pending recorded calls are launched first; a run too long to travel as kernel arguments is refused
        # (nothing launched) and the call is accepted again after a synchronisation
        pr = [g.primes[i] for i in g.limb_primes(L)]
        e = seeded.uniform_poly(9300, pr, N)
        de, dr, want = g.upload(e), g.alloc(L * N), g.alloc(L * N)
        g.mod_down(want, de, L, True)
        w = want.get()
        g.hw("modadd", de.view(0, N), de.view(0, N), de.view(0, N), 0)  # pending: limb 0 doubled
        g.hw("modsub_scalar", de.view(0, N), de.view(0, N), 0, 0)
        g.mod_down_noalloc(dr, de, L, True)
        g.mod_down(want, de, L, True)
        assert (dr.get() == want.get()).all() and not (want.get() == w).all(), "pending calls were not launched first"
        a = g.alloc(N)
        for i in range(100):
            g.hw("modadd_scalar", a, a, 1, 0)
        with pytest.raises(acefhe.AceError, match="pending"):
            g.mod_down_noalloc(dr, de, L, True)
        g.sync()
        g.mod_down_noalloc(dr, de, L, True)
        assert (dr.get() == want.get()).all()
        assert int(a.get()[0]) == 100
        # between ace_fork and ace_join the context issues on two streams, which would share the one array: refused
        g.fork()
        with pytest.raises(acefhe.AceError, match="ace_fork"):
            g.mod_down_noalloc(dr, de, L, True)
        g.join()
        g.mod_down_noalloc(dr, de, L, True)
        assert (dr.get() == want.get()).all()
    finally:
        g.close()


def test_mod_down_noalloc_rejects_what_does_not_fit():
    g = acefhe.Context(131072, 12, 50, 50, 3)  # (12 + 4) limbs of 2^17 words = 2^21: the largest that fits
    try:
        N, L, K = g.N, g.L, g.K
        assert (L + K) * N <= 1 << 21
        e = seeded.uniform_poly(9200, [g.primes[i] for i in g.limb_primes(L)], N)
        w, r = both(g, e, L, True)
        assert (w == r).all()
    finally:
        g.close()
    g = acefhe.Context(131072, 16, 50, 50, 3)
    try:
        N, L, K = g.N, g.L, g.K
        assert (L + K) * N > 1 << 21
        de, dr = g.alloc((L + K) * N), g.alloc(L * N)
        with pytest.raises(acefhe.AceError, match="exceeds the static scratch"):
            g.mod_down_noalloc(dr, de, L, True)
        g.sync()
        g.mod_down_noalloc(dr, de, 8, True)  # a level that fits is served
        g.sync()
    finally:
        g.close()
