"""ctypes binding of the CPU oracle (oracle/liboracle.so).  Test infrastructure."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB_PATH = os.path.join(ORACLE_DIR, "liboracle.so")

_i64p = C.POINTER(C.c_int64)
_i32p = C.POINTER(C.c_int32)
_u64p = C.POINTER(C.c_uint64)


def build_oracle():
    subprocess.check_call(["make", "-s", "-C", ORACLE_DIR, LIB_PATH])


def _ptr(a):
    assert a.dtype == np.int64 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_i64p)


def _idx(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a, a.ctypes.data_as(_i32p)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build_oracle()
        L = C.CDLL(LIB_PATH)
        L.orc_ctx_create.restype = C.c_void_p
        L.orc_ctx_create.argtypes = [C.c_uint32, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t]
        L.orc_ctx_create_with_primes.restype = C.c_void_p
        L.orc_ctx_create_with_primes.argtypes = [C.c_uint32, C.c_size_t, _i64p, C.c_size_t]
        L.orc_ctx_destroy.argtypes = [C.c_void_p]
        for n in ("orc_num_q", "orc_num_p", "orc_num_parts", "orc_part_size"):
            getattr(L, n).restype = C.c_size_t
            getattr(L, n).argtypes = [C.c_void_p]
        L.orc_num_decomp.restype = C.c_size_t
        L.orc_num_decomp.argtypes = [C.c_void_p, C.c_size_t]
        L.orc_degree.restype = C.c_uint32
        L.orc_degree.argtypes = [C.c_void_p]
        L.orc_prime.restype = C.c_int64
        L.orc_prime.argtypes = [C.c_void_p, C.c_size_t]
        L.orc_root.restype = C.c_int64
        L.orc_root.argtypes = [C.c_void_p, C.c_size_t]
        L.orc_modulus.argtypes = [C.c_void_p, C.c_size_t, _u64p]
        L.orc_twiddles.restype = _u64p
        L.orc_twiddles.argtypes = [C.c_void_p, C.c_size_t, C.c_int]
        L.orc_tbl_modup.restype = C.c_size_t
        L.orc_tbl_modup.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, _i64p, _i64p, _i32p, C.POINTER(C.c_size_t)]
        L.orc_tbl_moddown.argtypes = [C.c_void_p, _i64p, _i64p, _i64p, _i64p]
        L.orc_tbl_rescale.argtypes = [C.c_void_p, C.c_size_t, _i64p, _i64p]
        for n in ("orc_add_mod", "orc_sub_mod", "orc_switch_modulus", "orc_mod_exp"):
            getattr(L, n).restype = C.c_int64
            getattr(L, n).argtypes = [C.c_int64] * 3
        L.orc_mul_mod_barrett.restype = C.c_int64
        L.orc_mul_mod_barrett.argtypes = [C.c_void_p, C.c_size_t, C.c_int64, C.c_int64]
        L.orc_precompute_const.restype = C.c_uint64
        L.orc_precompute_const.argtypes = [C.c_uint64, C.c_uint64]
        L.orc_fast_mul_const.restype = C.c_int64
        L.orc_fast_mul_const.argtypes = [C.c_uint64] * 4
        L.orc_sub_mul_const.restype = C.c_int64
        L.orc_sub_mul_const.argtypes = [C.c_uint64] * 5
        L.orc_mod_inv.restype = C.c_int64
        L.orc_mod_inv.argtypes = [C.c_int64, C.c_int64]
        L.orc_is_prime.restype = C.c_int
        L.orc_is_prime.argtypes = [C.c_int64]
        L.orc_find_generator.restype = C.c_int64
        L.orc_find_generator.argtypes = [C.c_int64]
        L.orc_root_of_unity.restype = C.c_int64
        L.orc_root_of_unity.argtypes = [C.c_int64, C.c_int64]
        L.orc_precompute_const_128.argtypes = [C.c_uint64, _u64p]
        L.orc_find_automorphism_index.restype = C.c_uint32
        L.orc_find_automorphism_index.argtypes = [C.c_int32, C.c_uint32]
        _lib = L
    return _lib


class Oracle:
    """One CRT context of the oracle; arrays are numpy int64, limb-major."""

    def __init__(self, degree, num_q, q0_bits, sf_bits, parts, primes=None):
        self.L_ = lib()
        if primes is None:
            self.h = self.L_.orc_ctx_create(degree, num_q, q0_bits, sf_bits, parts)
        else:
            p = np.ascontiguousarray(primes, dtype=np.int64)
            self.h = self.L_.orc_ctx_create_with_primes(degree, len(p), _ptr(p), parts)
        self.h = C.c_void_p(self.h)
        self.N = degree
        self.L = self.L_.orc_num_q(self.h)
        self.K = self.L_.orc_num_p(self.h)
        self.parts = self.L_.orc_num_parts(self.h)
        self.part_size = self.L_.orc_part_size(self.h)
        self.primes = [self.L_.orc_prime(self.h, i) for i in range(self.L + self.K)]
        self.roots = [self.L_.orc_root(self.h, i) for i in range(self.L + self.K)]

    def close(self):
        if self.h:
            self.L_.orc_ctx_destroy(self.h)
            self.h = None

    def num_decomp(self, level):
        return self.L_.orc_num_decomp(self.h, level)

    def modulus(self, i):
        out = (C.c_uint64 * 5)()
        self.L_.orc_modulus(self.h, i, out)
        return list(out)

    def twiddles(self, i, which):
        p = self.L_.orc_twiddles(self.h, i, which)
        return np.ctypeslib.as_array(p, shape=(self.N,)).copy()

    def limb_primes(self, level, with_p=True):
        return list(range(level)) + ([self.L + j for j in range(self.K)] if with_p else [])

    # --- tables
    def tbl_modup(self, level, part):
        hat_inv = np.zeros(64, np.int64)
        hat = np.zeros(64 * 128, np.int64)
        cidx = np.zeros(128, np.int32)
        nd = C.c_size_t()
        nc = self.L_.orc_tbl_modup(self.h, level, part, _ptr(hat_inv), _ptr(hat),
                                   cidx.ctypes.data_as(_i32p), C.byref(nd))
        nd = nd.value
        return hat_inv[:nd].copy(), hat[: nd * nc].reshape(nd, nc).copy(), cidx[:nc].copy()

    def tbl_moddown(self):
        a = np.zeros(self.K, np.int64)
        b = np.zeros(self.L * self.K, np.int64)
        c = np.zeros(self.L, np.int64)
        d = np.zeros(self.L, np.int64)
        self.L_.orc_tbl_moddown(self.h, _ptr(a), _ptr(b), _ptr(c), _ptr(d))
        return a, b.reshape(self.L, self.K), c, d

    def tbl_rescale(self, level):
        a = np.zeros(level - 1, np.int64)
        b = np.zeros(level - 1, np.int64)
        self.L_.orc_tbl_rescale(self.h, level, _ptr(a), _ptr(b))
        return a, b

    # --- NTT
    def ntt(self, data, prime_idx, inverse=False):
        data = np.ascontiguousarray(data, dtype=np.int64)
        out = np.empty_like(data)
        ia, ip = _idx(prime_idx)
        f = self.L_.orc_intt if inverse else self.L_.orc_ntt
        f(self.h, _ptr(out), _ptr(data), ip, C.c_size_t(len(ia)))
        return out

    def intt(self, data, prime_idx):
        return self.ntt(data, prime_idx, inverse=True)

    # --- per limb ops
    def hw(self, name, a, b, idx, r=None):
        a = np.ascontiguousarray(a, dtype=np.int64)
        n = a.size
        out = np.zeros(n, np.int64) if r is None else np.array(r, dtype=np.int64, copy=True)
        f = getattr(self.L_, "orc_hw_" + name)
        if name.endswith("_scalar"):
            f(self.h, _ptr(out), _ptr(a), C.c_int64(int(b)), C.c_size_t(idx), C.c_size_t(n))
        else:
            b = np.ascontiguousarray(b, dtype=np.int64)
            f(self.h, _ptr(out), _ptr(a), _ptr(b), C.c_size_t(idx), C.c_size_t(n))
        return out

    def find_automorphism_index(self, rot):
        return self.L_.orc_find_automorphism_index(rot, self.N)

    def automorphism_order(self, k, is_ntt=True):
        out = np.zeros(self.N, np.int64)
        self.L_.orc_automorphism_order(_ptr(out), C.c_uint32(k), C.c_uint32(self.N), C.c_int(int(is_ntt)))
        return out

    # --- RNS poly ops
    def decomp_modup(self, src, level, part, is_ntt=True):
        src = np.ascontiguousarray(src, dtype=np.int64)
        out = np.zeros((level + self.K) * self.N, np.int64)
        self.L_.orc_decomp_modup(self.h, _ptr(out), _ptr(src), C.c_size_t(level), C.c_size_t(part), C.c_int(int(is_ntt)))
        return out

    def precomp(self, src, level, is_ntt=True, fused=True):
        src = np.ascontiguousarray(src, dtype=np.int64)
        nd = self.num_decomp(level)
        out = np.zeros(nd * (level + self.K) * self.N, np.int64)
        self.L_.orc_precomp(self.h, _ptr(out), _ptr(src), C.c_size_t(level), C.c_int(int(is_ntt)), C.c_int(int(fused)))
        return out

    def mod_down(self, src, level, is_ntt=True):
        src = np.ascontiguousarray(src, dtype=np.int64)
        out = np.zeros(level * self.N, np.int64)
        self.L_.orc_mod_down(self.h, _ptr(out), _ptr(src), C.c_size_t(level), C.c_int(int(is_ntt)))
        return out

    def rescale(self, src, level, is_ntt=True):
        src = np.ascontiguousarray(src, dtype=np.int64)
        out = np.zeros((level - 1) * self.N, np.int64)
        self.L_.orc_rescale(self.h, _ptr(out), _ptr(src), C.c_size_t(level), C.c_int(int(is_ntt)))
        return out

    def extend(self, src, level):
        src = np.ascontiguousarray(src, dtype=np.int64)
        out = np.zeros((level + self.K) * self.N, np.int64)
        self.L_.orc_extend(self.h, _ptr(out), _ptr(src), C.c_size_t(level))
        return out

    def mod_down_rescale(self, src, level, is_ntt=True):
        """Returns (result at level-1 in NTT form, the input as the call leaves it: coefficient form)."""
        poly = np.array(src, dtype=np.int64, copy=True)
        out = np.zeros((level - 1) * self.N, np.int64)
        self.L_.orc_mod_down_rescale(self.h, _ptr(out), _ptr(poly), C.c_size_t(level), C.c_int(int(is_ntt)))
        return out, poly

    def reduce_rescale_modup(self, src, level, is_ntt=True):
        """Returns (res as left by the call: level limbs, raised digits, the input in coefficient form)."""
        poly = np.array(src, dtype=np.int64, copy=True)
        res = np.zeros(level * self.N, np.int64)
        raised = np.zeros(self.num_decomp(level - 1) * (level - 1 + self.K) * self.N, np.int64)
        self.L_.orc_reduce_rescale_modup(self.h, _ptr(res), _ptr(raised), _ptr(poly), C.c_size_t(level),
                                         C.c_int(int(is_ntt)))
        return res, raised, poly

    def transform_from_level0(self, src, level):
        src = np.ascontiguousarray(src, dtype=np.int64)
        out = np.zeros(level * self.N, np.int64)
        self.L_.orc_transform_from_level0(self.h, _ptr(out), _ptr(src), C.c_size_t(level))
        return out

    # --- encoder
    def embedding(self, values, inverse=False):
        v = np.ascontiguousarray(values, dtype=np.complex128)
        out = np.zeros_like(v)
        self.L_.orc_embedding(self.h, out.ctypes.data_as(C.c_void_p), v.ctypes.data_as(C.c_void_p),
                              C.c_size_t(v.size), C.c_int(int(inverse)))
        return out

    def encode(self, values, slots=0, level=0, sf_degree=1, p_cnt=0):
        """Plaintext polynomial (level Q limbs + p_cnt P limbs, NTT form), or None where the reference asserts."""
        v = np.ascontiguousarray(values, dtype=np.complex128)
        lv = level or self.L
        out = np.zeros((lv + p_cnt) * self.N, np.int64)
        self.L_.orc_encode.restype = C.c_int
        ok = self.L_.orc_encode(self.h, _ptr(out), v.ctypes.data_as(C.c_void_p), C.c_size_t(v.size), C.c_uint32(slots),
                                C.c_size_t(level), C.c_uint32(sf_degree), C.c_size_t(p_cnt))
        return out if ok else None

    def encode_scaled(self, values, slots, level, scale, p_cnt=0):
        """Encode_at_level_with_scale: the plaintext polynomial at an explicit scale, or None on a range failure."""
        v = np.ascontiguousarray(values, dtype=np.complex128)
        lv = level or self.L
        out = np.zeros((lv + p_cnt) * self.N, np.int64)
        self.L_.orc_encode_scaled.restype = C.c_int
        ok = self.L_.orc_encode_scaled(self.h, _ptr(out), v.ctypes.data_as(C.c_void_p), C.c_size_t(v.size),
                                       C.c_uint32(slots), C.c_size_t(level), C.c_double(scale), C.c_size_t(p_cnt))
        return out if ok else None

    def decode(self, poly, level, slots, factor, is_ntt=True):
        poly = np.ascontiguousarray(poly, dtype=np.int64)
        out = np.zeros(slots, np.complex128)
        self.L_.orc_decode(self.h, out.ctypes.data_as(C.c_void_p), _ptr(poly), C.c_size_t(level), C.c_uint32(slots),
                           C.c_double(factor), C.c_int(int(is_ntt)))
        return out

    def dot_prod(self, digits, key, n_parts, level, fast=False):
        digits = np.ascontiguousarray(digits, dtype=np.int64)
        key = np.ascontiguousarray(key, dtype=np.int64)
        out = np.zeros((level + self.K) * self.N, np.int64)
        stride = key.size // n_parts
        self.L_.orc_dot_prod(self.h, _ptr(out), _ptr(digits), _ptr(key), C.c_size_t(stride),
                             C.c_size_t(n_parts), C.c_size_t(level), C.c_int(int(fast)))
        return out

    def poly(self, name, a, b, level, with_p=False):
        a = np.ascontiguousarray(a, dtype=np.int64)
        b = np.ascontiguousarray(b, dtype=np.int64)
        out = np.zeros_like(a)
        getattr(self.L_, "orc_poly_" + name)(self.h, _ptr(out), _ptr(a), _ptr(b), C.c_size_t(level), C.c_int(int(with_p)))
        return out

    # --- ciphertext level
    def mul_relin_rescale(self, a0, a1, b0, b1, swk, level):
        n = (level - 1) * self.N
        r0 = np.zeros(n, np.int64)
        r1 = np.zeros(n, np.int64)
        args = [np.ascontiguousarray(x, dtype=np.int64) for x in (a0, a1, b0, b1, swk)]
        self.L_.orc_mul_relin_rescale(self.h, _ptr(r0), _ptr(r1), *[_ptr(x) for x in args], C.c_size_t(level))
        return r0, r1

    def mul_ciph3(self, a0, a1, b0, b1, level):
        n = level * self.N
        d = [np.zeros(n, np.int64) for _ in range(3)]
        args = [np.ascontiguousarray(x, dtype=np.int64) for x in (a0, a1, b0, b1)]
        self.L_.orc_mul_ciph3(self.h, *[_ptr(x) for x in d], *[_ptr(x) for x in args], C.c_size_t(level))
        return d

    def relin(self, d0, d1, d2, swk, level):
        n = level * self.N
        r0 = np.zeros(n, np.int64)
        r1 = np.zeros(n, np.int64)
        args = [np.ascontiguousarray(x, dtype=np.int64) for x in (d0, d1, d2, swk)]
        self.L_.orc_relin(self.h, _ptr(r0), _ptr(r1), *[_ptr(x) for x in args], C.c_size_t(level))
        return r0, r1

    def fast_rotate(self, c0, digits, swk, order, level):
        n = level * self.N
        r0 = np.zeros(n, np.int64)
        r1 = np.zeros(n, np.int64)
        args = [np.ascontiguousarray(x, dtype=np.int64) for x in (c0, digits, swk, order)]
        self.L_.orc_fast_rotate(self.h, _ptr(r0), _ptr(r1), *[_ptr(x) for x in args], C.c_size_t(level))
        return r0, r1
