"""HIP path vs. the committed golden fixtures at full size (outputs of the reference's own
compiled code for N=65536, 24x50-bit limbs, dnum 3), plus size-independent properties."""
import numpy as np
import pytest

import golden_replay
import seeded

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", ["small", "gemm", "headline"])
def test_gpu_matches_reference_fixtures(name):
    meta, vec = golden_replay.load()
    impl = golden_replay.GpuImpl(tuple(meta[name]["cfg"]))
    golden_replay.check(impl, name, meta, vec)
    impl.close()


def test_headline_properties():
    """At BASELINE size: NTT round trip and linearity on a 4-polynomial batch, Extend->Mod_down
    identity, key switching is linear in the digits, rotation by r then -r restores the limbs."""
    import acefhe
    g = acefhe.Context(65536, 24, 50, 50, 3)
    N, L, K = g.N, g.L, g.K
    idx = list(range(L))
    polys = 4
    x = np.concatenate([seeded.uniform_poly(50 + p, g.primes[:L], N) for p in range(polys)])
    y = np.concatenate([seeded.uniform_poly(60 + p, g.primes[:L], N) for p in range(polys)])
    dx, dy, ds = g.upload(x), g.upload(y), g.alloc(x.size)
    for p in range(polys):
        g.poly("add", ds.view(p * L * N, L * N), dx.view(p * L * N, L * N), dy.view(p * L * N, L * N), L)
    for d in (dx, dy, ds):
        g.ntt(d, d, idx, n_polys=polys, poly_stride_limbs=L)
    dt = g.alloc(x.size)
    for p in range(polys):
        g.poly("add", dt.view(p * L * N, L * N), dx.view(p * L * N, L * N), dy.view(p * L * N, L * N), L)
    assert (dt.get() == ds.get()).all(), "NTT(x+y) != NTT(x)+NTT(y)"
    g.intt(dx, dx, idx, n_polys=polys, poly_stride_limbs=L)
    assert (dx.get() == x).all(), "round trip"
    # Extend -> Mod_down
    c = x[: L * N]
    dc, de, dm = g.upload(c), g.alloc((L + K) * N), g.alloc(L * N)
    g.extend(de, dc, L)
    g.mod_down(dm, de, L, True)
    assert (dm.get() == c).all(), "Extend->Mod_down is not the identity"
    # automorphism by k then by k^-1 (index tables compose to the identity)
    k = g.find_automorphism_index(5)
    kinv = pow(k, -1, 2 * N)
    o1, o2 = g.automorphism_order(k, True), g.automorphism_order(kinv, True)
    r1, r2 = g.alloc(L * N), g.alloc(L * N)
    g.poly("automorphism", r1, dc, o1, L)
    g.poly("automorphism", r2, r1, o2, L)
    assert (r2.get() == c).all(), "sigma_k^-1(sigma_k(x)) != x"
    # key switch is additive in the digits: ks(d1) + ks(d2) == ks(d1 + d2) up to the
    # rounding of Mod_down, which is exact here because every limb is handled exactly:
    # compare the extended inner products instead (before Mod_down), which are linear.
    T = L + K
    pr = [g.primes[i] for i in g.limb_primes(L)]
    nd = g.num_decomp(L)
    d1 = np.concatenate([seeded.uniform_poly(70 + d, pr, N) for d in range(nd)])
    d2 = np.concatenate([seeded.uniform_poly(80 + d, pr, N) for d in range(nd)])
    key = np.concatenate([seeded.uniform_poly(90 + d, g.primes, N) for d in range(nd)])
    dd1, dd2, dk = g.upload(d1), g.upload(d2), g.upload(key)
    dsum = g.alloc(d1.size)
    for d in range(nd):
        g.poly("add", dsum.view(d * T * N, T * N), dd1.view(d * T * N, T * N), dd2.view(d * T * N, T * N), L, True)
    e1, e2, e3, e12 = (g.alloc(T * N) for _ in range(4))
    ks = (L + K) * N
    g.dot_prod(e1, dd1, dk, ks, nd, L)
    g.dot_prod(e2, dd2, dk, ks, nd, L)
    g.dot_prod(e3, dsum, dk, ks, nd, L)
    g.poly("add", e12, e1, e2, L, True)
    assert (e12.get() == e3.get()).all(), "inner product with the key is not additive"
    g.close()
