"""Host-side pieces of the runtime's bootstrapping that need no GPU: the sine series and the Chebyshev division."""
import ctypes as C
import os
import re

import numpy as np
import pytest
from numpy.polynomial import chebyshev as cheb

import rt_program

REF_HEADER = "/root/reference/fhe-cmplr/rtlib/ant/include/ckks/bootstrap.h"


@pytest.fixture(scope="module")
def lib():
    return C.CDLL(os.path.join(rt_program.ROOT, "ace-compiler_amd", "librt_hip.so"))


def sin_series(lib, hw, even):
    out = np.zeros(96)
    k, r = C.c_uint32(), C.c_uint32()
    lib.Rt_sin_series.restype = C.c_size_t
    n = lib.Rt_sin_series(C.c_size_t(hw), C.c_int(even), out.ctypes.data_as(C.c_void_p), C.byref(k), C.byref(r))
    return out[:n], k.value, r.value


@pytest.mark.parametrize("hw,even", [(0, 0), (192, 0), (64, 1), (1000, 1)])
def test_sin_series_reduces_modulo_one(lib, hw, even):
    """After the double-angle steps the series is sin(2 pi K x) / (2 pi) (cos for the even form, whose argument the
    caller shifts by 1/(4K)), i.e. x - round(x) near the integers of [-K, K]: checked in floating point."""
    c, K, R = sin_series(lib, hw, even)
    x = np.linspace(-1, 1, 20001)
    y = cheb.chebval(x - (1 / (4 * K) if even else 0), np.concatenate([[c[0] / 2], c[1:]]))
    for j in range(1, R + 1):
        y = 2 * y * y - (2 * np.pi) ** (-(2.0 ** (j - R)))
    want = np.sin(2 * np.pi * K * x) / (2 * np.pi)
    assert np.abs(y - want).max() < 1e-9
    # close to an integer i/K the result is the distance to it, times K
    t = (np.arange(-K + 1, K)[:, None] + np.array([-1e-3, 0, 1e-3])[None, :]) / K
    got = cheb.chebval(t - (1 / (4 * K) if even else 0), np.concatenate([[c[0] / 2], c[1:]]))
    for j in range(1, R + 1):
        got = 2 * got * got - (2 * np.pi) ** (-(2.0 ** (j - R)))
    assert np.abs(got - np.array([-1e-3, 0, 1e-3])[None, :]).max() < 1e-7


@pytest.mark.skipif(not os.path.exists(REF_HEADER), reason="reference checkout not present")
@pytest.mark.parametrize("name,hw,even", [("G_coefficients_uniform", 0, 0), ("G_coefficients_uniform_hw_192", 192, 0),
                                          ("G_even_coefficients_uniform", 0, 1),
                                          ("G_even_coefficients_uniform_hw_192", 100, 1)])
def test_sin_series_equals_the_reference_tables(lib, name, hw, even):
    src = open(REF_HEADER).read()
    body = re.search(name + r"\[[A-Z_0-9]+\]\s*=\s*\{(.*?)\};", src, re.S).group(1)
    table = np.array([float(v) for v in re.sub(r"//.*", "", body).replace("\n", " ").split(",") if v.strip()])
    c, _, _ = sin_series(lib, hw, even)
    assert c.size == table.size
    assert np.abs(c - table).max() < 2e-14


@pytest.mark.parametrize("nf,ng,seed", [(91, 49, 1), (43, 13, 2), (13, 13, 3), (7, 10, 4), (30, 1, 5)])
def test_series_division_is_chebyshev_division(lib, nf, ng, seed):
    """f = q g + r with deg r < deg g, in the basis where entry 0 holds twice the constant term."""
    rng = np.random.default_rng(seed)
    f, g = rng.normal(size=nf), rng.normal(size=ng)
    q, r = np.zeros(nf), np.zeros(nf)
    nq, nr = C.c_size_t(), C.c_size_t()
    lib.Rt_series_divide(q.ctypes.data_as(C.c_void_p), C.byref(nq), r.ctypes.data_as(C.c_void_p), C.byref(nr),
                         f.ctypes.data_as(C.c_void_p), C.c_size_t(nf), g.ctypes.data_as(C.c_void_p), C.c_size_t(ng))
    q, r = q[:nq.value], r[:nr.value]

    def true(v):
        return np.concatenate([[v[0] / 2], v[1:]])
    back = cheb.chebadd(cheb.chebmul(true(q), true(g)), true(r))
    want = true(f)
    back = np.concatenate([back, np.zeros(max(0, want.size - back.size))])
    assert np.abs(back[:want.size] - want).max() < 1e-9 * max(1.0, np.abs(q).max())
    if nf >= ng:
        assert r.size < ng or ng == 1
    else:
        assert np.array_equal(r, f) and q.size == 1 and q[0] == 0


def test_side_file_reader_takes_the_reference_s_own_file(lib):
    """The one weight side-file in the reference tree (rtlib/ant/dataset/bootstrap_full_data.msg: a header and an
    empty table, kept under tests/golden) opens; a file written by tests/msgfile.py has the same header layout."""
    import msgfile

    path = os.path.join(rt_program.ROOT, "tests", "golden", "bootstrap_full_data.msg")
    raw = open(path, "rb").read()
    assert len(raw) == 136 and raw[:8] == b"!ANTFHE\0"
    lib.Pt_mgr_init.restype = C.c_bool
    assert lib.Pt_mgr_init(path.encode())
    lib.Pt_mgr_fini()
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        mine = os.path.join(d, "empty.msg")
        msgfile.write(mine, [])
        got = open(mine, "rb").read()
        # identical but for the creation time and the model name
        assert got[:32] == raw[:32] and got[96:136] == raw[96:136] and len(got) == 4096
        assert lib.Pt_mgr_init(mine.encode())
        lib.Pt_mgr_fini()
