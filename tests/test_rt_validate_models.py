"""The plain-float operator models of the compiler's validation mode (Conv_impl, Gemm_impl, Average_pool_impl,
Global_average_pool_impl, Rotate_impl, Relu_impl, Add_impl, Mul_impl in librt_hip.so) against the reference's own
rt_validate.c compiled as it lies (oracle/_ref/libref_validate.so): the same doubles, bit for bit, on random tensors
over shapes that exercise padding, strides, non-square planes and windows, and both rotation directions."""
import ctypes as C
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = os.path.join(ROOT, "oracle", "_ref", "libref_validate.so")
OURS = os.path.join(ROOT, "ace-compiler_amd", "librt_hip.so")

pytestmark = pytest.mark.skipif(not os.path.exists(REF), reason="built only where the reference tree is present")

_dp, _fp = C.POINTER(C.c_double), C.POINTER(C.c_float)


def _libs():
    libs = []
    for path in (REF, OURS):
        lib = C.CDLL(path)
        for name in ("Add_impl", "Mul_impl", "Rotate_impl", "Relu_impl", "Conv_impl", "Gemm_impl",
                     "Average_pool_impl", "Global_average_pool_impl"):
            getattr(lib, name).restype = _dp
        libs.append(lib)
    return libs


def _take(ptr, n):
    out = np.ctypeslib.as_array(ptr, shape=(n,)).copy()
    C.CDLL(None).free(ptr)
    return out


def _d(a):
    return a.ctypes.data_as(_dp)


def _f(a):
    return a.ctypes.data_as(_fp)


def _same(a, b, what):
    assert a.shape == b.shape, what
    assert np.array_equal(a.view(np.uint64), b.view(np.uint64)), what


def test_elementwise_rotate_relu():
    ref, ours = _libs()
    rng = np.random.default_rng(1)
    for n in (1, 7, 64, 1000):
        a, b = rng.normal(size=n), rng.normal(size=n)
        for fn in ("Add_impl", "Mul_impl"):
            _same(_take(getattr(ref, fn)(_d(a), _d(b), n), n), _take(getattr(ours, fn)(_d(a), _d(b), n), n), fn)
        _same(_take(ref.Relu_impl(_d(a), n), n), _take(ours.Relu_impl(_d(a), n), n), "relu")
        for step in sorted({0, 1, -1, n // 2, -(n // 2), n - 1, -(n - 1), n, -n}):
            _same(_take(ref.Rotate_impl(_d(a), n, step), n), _take(ours.Rotate_impl(_d(a), n, step), n),
                  "rotate n=%d step=%d" % (n, step))


@pytest.mark.parametrize("shape", [
    # n, c, h, w, kn, kh, kw, sh, sw, ph, pw
    (1, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1),
    (2, 2, 9, 7, 3, 3, 3, 2, 2, 1, 1),
    (1, 4, 6, 10, 5, 1, 1, 1, 1, 0, 0),
    (1, 1, 5, 5, 2, 5, 5, 1, 1, 0, 0),
    (1, 2, 8, 8, 2, 3, 2, 1, 2, 2, 0),
    (1, 16, 16, 16, 16, 3, 3, 1, 1, 1, 1),
])
def test_conv(shape):
    ref, ours = _libs()
    n, c, h, w, kn, kh, kw, sh, sw, ph, pw = shape
    rng = np.random.default_rng(sum(shape))
    x = rng.normal(size=n * c * h * w)
    wt = rng.normal(size=kn * c * kh * kw).astype(np.float32)
    bias = rng.normal(size=kn).astype(np.float32)
    H, W = h + 2 * ph, w + 2 * pw
    n_out = n * kn * ((H - kh) // sh + 1) * ((W - kw) // sw + 1)
    args = (n, c, h, w, _f(wt), kn, c, kh, kw, _f(bias), kn, sh, sw, 0, 0, ph, pw)
    _same(_take(ref.Conv_impl(_d(x), *args), n_out), _take(ours.Conv_impl(_d(x), *args), n_out), "conv %r" % (shape,))


def test_gemm():
    ref, ours = _libs()
    rng = np.random.default_rng(3)
    for w, wh in ((64, 10), (1, 1), (17, 33)):
        x = rng.normal(size=w)
        wt = rng.normal(size=wh * w).astype(np.float32)
        bias = rng.normal(size=wh).astype(np.float32)
        args = (1, w, _f(wt), wh, w, _f(bias), wh)
        _same(_take(ref.Gemm_impl(_d(x), *args), wh), _take(ours.Gemm_impl(_d(x), *args), wh), "gemm %d x %d" % (wh, w))


@pytest.mark.parametrize("shape", [
    # n, c, h, w, kh, kw, sh, sw, ph, pw: square planes with the stride equal to the window, as the compiler emits
    # them, then shapes where the model's own conventions show
    (1, 3, 8, 8, 2, 2, 2, 2, 0, 0),
    (2, 2, 12, 12, 3, 3, 3, 3, 0, 0),
    (1, 2, 6, 6, 2, 2, 2, 2, 1, 1),
    (1, 1, 8, 8, 2, 2, 4, 4, 0, 0),
    (1, 2, 4, 8, 2, 2, 2, 4, 0, 0),
])
def test_average_pool(shape):
    ref, ours = _libs()
    n, c, h, w, kh, kw, sh, sw, ph, pw = shape
    rng = np.random.default_rng(sum(shape) + 9)
    x = rng.normal(size=n * c * h * w)
    H, W = h + 2 * ph, w + 2 * pw
    n_out = n * c * ((H - kh) // sh + 1) * ((W - kw) // sw + 1)
    args = (n, c, h, w, kh, kw, sh, sw, 0, 0, ph, pw)
    _same(_take(ref.Average_pool_impl(_d(x), *args), n_out), _take(ours.Average_pool_impl(_d(x), *args), n_out),
          "average pool %r" % (shape,))


def test_global_average_pool():
    ref, ours = _libs()
    rng = np.random.default_rng(5)
    for n, c, h, w in ((1, 64, 8, 8), (2, 3, 5, 7), (1, 1, 1, 1)):
        x = rng.normal(size=n * c * h * w)
        _same(_take(ref.Global_average_pool_impl(_d(x), n, c, h, w), n * c),
              _take(ours.Global_average_pool_impl(_d(x), n, c, h, w), n * c), "global average pool")


def test_validate_reports_like_the_reference(capfd):
    """Validate_impl prints the verdict on stdout and goes on (it does not abort); both libraries print the same."""
    ref, ours = _libs()
    a = np.linspace(0, 1, 40)
    b = a.copy()
    b[25] += 0.5
    texts = []
    for lib in (ref, ours):
        lib.Validate_impl(_d(a), _d(a), 40, -3)
        lib.Validate_impl(_d(a), _d(b), 40, -3)
        lib.Validate_value_range(True)
        lib.Validate_value_range(False)
        texts.append(capfd.readouterr())
    assert texts[0].out == texts[1].out and "internal validation fail" in texts[0].out
    assert texts[0].err == texts[1].err and "validation failed at 25" in texts[0].err
