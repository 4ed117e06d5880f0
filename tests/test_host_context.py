"""CPU checks of the product library: it loads, exports every declared symbol,
its host-side context (primes, roots, every table the kernels read) equals the
oracle's, and without a GPU it refuses to compute instead of falling back."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import acefhe
from oracle_lib import Oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CONFIGS = [(16, 10, 60, 59, 3), (64, 7, 45, 40, 3), (64, 6, 50, 50, 2), (8192, 5, 40, 40, 3),
           (4096, 3, 30, 25, 1), (65536, 24, 50, 50, 3), (65536, 34, 51, 46, 3)]


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "ace_hip.h")).read()
    declared = set(re.findall(r"\b(ace_[a-z0-9_]+)\s*\(", hdr))
    declared.discard("ace_ctx")
    lib = C.CDLL(acefhe.LIB_PATH)
    missing = [s for s in sorted(declared) if not hasattr(lib, s)]
    assert not missing, missing
    assert declared == set(acefhe.EXPORTS)
    # every binding declares its argument types: an undeclared one would pass 64-bit pointers as C ints
    bound = acefhe.lib()
    untyped = [s for s in sorted(declared) if getattr(bound, s).argtypes is None]
    assert not untyped, untyped


@pytest.mark.parametrize("cfg", CONFIGS)
def test_host_context_equals_oracle(cfg):
    c = acefhe.Context(*cfg)
    o = Oracle(*cfg)
    assert (c.N, c.L, c.K, c.parts, c.part_size) == (o.N, o.L, o.K, o.parts, o.part_size)
    assert c.primes == o.primes and c.roots == o.roots
    for i in range(c.L + c.K):
        assert c.modulus(i) == o.modulus(i)
    for i in sorted({0, c.L - 1, c.L, c.L + c.K - 1}):
        for which in range(4):
            assert (c.twiddles(i, which) == o.twiddles(i, which)).all()
    levels = range(1, c.L + 1) if c.N <= 8192 else (1, 2, c.part_size, c.part_size + 1, c.L - 1, c.L)
    for level in levels:
        assert c.num_decomp(level) == o.num_decomp(level)
        for part in range(c.num_decomp(level)):
            for a, b in zip(c.tbl_modup(level, part), o.tbl_modup(level, part)):
                assert a.shape == b.shape and (a == b).all()
        if level >= 2:
            for a, b in zip(c.tbl_rescale(level), o.tbl_rescale(level)):
                assert (a == b).all()
    for a, b in zip(c.tbl_moddown(), o.tbl_moddown()):
        assert (a == b).all()
    for rot in (0, 1, 5, -3, c.N // 2 - 1, 2 * c.N - 1):
        k = c.find_automorphism_index(rot)
        assert k == o.find_automorphism_index(rot)
        for is_ntt in (True, False):
            assert (c.host_automorphism_order(k, is_ntt) == o.automorphism_order(k, is_ntt)).all()
    c.close()
    o.close()


def test_single_prime_chain_and_unequal_first_prime():
    for cfg in [(32, 1, 40, 40, 1), (32, 1, 45, 40, 1), (32, 2, 40, 40, 1), (32, 2, 50, 40, 2), (32, 3, 60, 40, 3)]:
        c = acefhe.Context(*cfg)
        o = Oracle(*cfg)
        assert c.primes == o.primes and c.K == o.K
        c.close()
        o.close()


def test_invalid_parameters_are_rejected():
    with pytest.raises(acefhe.AceError):
        acefhe.Context(100, 3, 40, 40, 1)  # not a power of two
    with pytest.raises(acefhe.AceError):
        acefhe.Context(64, 0, 40, 40, 1)
    with pytest.raises(acefhe.AceError):
        acefhe.Context(64, 4, 40, 40, 5)  # more digits than primes allow


def test_no_gpu_means_no_compute():
    c = acefhe.Context(64, 3, 40, 40, 1)
    if c.has_device:
        pytest.skip("a GPU is present")
    with pytest.raises(acefhe.AceError, match="no HIP device"):
        c.alloc(64)
    lib = c.lib
    dummy = C.c_void_p(8)
    idx = (C.c_int32 * 1)(0)
    assert lib.ace_ntt(c.h, dummy, dummy, idx, 1, 1, 1) != 0
    assert b"no HIP device" in lib.ace_last_error()
    assert lib.ace_mul_relin_rescale(c.h, *([dummy] * 7), 2) != 0
    c.close()


def test_fft_tables_match_the_oracle_bit_for_bit():
    """The encoder's root table must carry the very doubles the reference computes (gcc's cos / sin of the C
    library; the oracle's table, whose encoder is matched against the reference's): at a 50-bit scaling factor
    one unit in the last place of a twiddle changes rounded coefficients.  A build of the host tables with
    another compiler's math calls differs in about one entry in a thousand."""
    import ctypes as C
    import numpy as np
    import acefhe
    from oracle_lib import Oracle
    cfg = (16384, 4, 60, 50, 2)
    g = acefhe.Context(*cfg)
    rou, rot = g.host_fft_tables()
    g.close()
    M = 2 * cfg[0]
    o = Oracle(*cfg)
    o.L_.orc_fft_rou.restype = C.POINTER(C.c_double)
    o.L_.orc_fft_rou.argtypes = [C.c_void_p]
    want = np.ctypeslib.as_array(o.L_.orc_fft_rou(o.h), shape=(2 * M,)).copy()
    assert np.array_equal(rou.view(np.int64), want.view(np.int64))
    pw = [1]
    for _ in range(cfg[0] // 2 - 1):
        pw.append(pw[-1] * 5 % M)
    assert rot.tolist() == pw
    o.close()
