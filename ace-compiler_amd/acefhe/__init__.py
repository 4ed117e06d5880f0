"""ctypes binding of libace_hip.so, the MI355X CKKS polynomial runtime.

The binding is a thin veneer over the C-ABI declared in include/ace_hip.h:
device buffers are raw HBM pointers wrapped in `DevBuf`, every method maps to
one C entry point, and a non-zero return raises `AceError` with the library's
message.  There is no CPU fallback: if the shared library is missing, import
fails; if no GPU is present, every compute call raises.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "libace_hip.so")

_i64p = C.POINTER(C.c_int64)
_i32p = C.POINTER(C.c_int32)
_u64p = C.POINTER(C.c_uint64)
_vp = C.c_void_p
_sz = C.c_size_t


class AceError(RuntimeError):
    pass


def _sig(lib):
    def f(name, res, *args):
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = list(args)

    f("ace_ctx_create", _vp, C.c_uint32, _sz, _sz, _sz, _sz)
    f("ace_ctx_create_with_primes", _vp, C.c_uint32, _sz, _i64p, _sz)
    f("ace_ctx_destroy", None, _vp)
    f("ace_has_device", C.c_int, _vp)
    f("ace_last_error", C.c_char_p)
    f("ace_degree", C.c_uint32, _vp)
    for n in ("ace_num_q", "ace_num_p", "ace_num_parts", "ace_part_size"):
        f(n, _sz, _vp)
    f("ace_num_decomp", _sz, _vp, _sz)
    f("ace_prime", C.c_int64, _vp, _sz)
    f("ace_root", C.c_int64, _vp, _sz)
    f("ace_modulus", None, _vp, _sz, _u64p)
    f("ace_host_twiddles", C.c_int, _vp, _sz, C.c_int, _u64p)
    f("ace_host_tbl_modup", C.c_int, _vp, _sz, _sz, _i64p, _i64p, _i32p, C.POINTER(_sz), C.POINTER(_sz))
    f("ace_host_tbl_moddown", C.c_int, _vp, _i64p, _i64p, _i64p, _i64p)
    f("ace_host_tbl_rescale", C.c_int, _vp, _sz, _i64p, _i64p)
    f("ace_host_automorphism_order", C.c_int, _vp, _i64p, C.c_uint32, C.c_int)
    f("ace_alloc", _vp, _vp, _sz)
    f("ace_free", None, _vp, _vp)
    f("ace_upload", C.c_int, _vp, _vp, _i64p, _sz)
    f("ace_download", C.c_int, _vp, _i64p, _vp, _sz)
    f("ace_copy", C.c_int, _vp, _vp, _vp, _sz)
    f("ace_zero", C.c_int, _vp, _vp, _sz)
    f("ace_sync", C.c_int, _vp)
    f("ace_sync_device", C.c_int, _vp)
    f("ace_memory_stats", None, _vp, C.POINTER(C.c_size_t))
    f("ace_ctx_share", _vp, _vp)
    f("ace_fork_release", C.c_int, _vp)
    f("ace_census_mark", None, C.c_char_p)
    f("ace_timer_start", C.c_int, _vp)
    f("ace_timer_stop_ms", C.c_float, _vp)
    f("ace_ntt", C.c_int, _vp, _vp, _vp, _i32p, _sz, _sz, _sz)
    f("ace_intt", C.c_int, _vp, _vp, _vp, _i32p, _sz, _sz, _sz)
    f("ace_ntt_pass", C.c_int, _vp, _vp, _vp, _i32p, _sz, _sz, _sz, C.c_int, C.c_int)
    for n in ("modadd", "modsub", "modmul", "modmuladd"):
        f("ace_hw_" + n, C.c_int, _vp, _vp, _vp, _vp, _sz, _sz)
        f("ace_hw_" + n + "_scalar", C.c_int, _vp, _vp, _vp, C.c_int64, _sz, _sz)
    f("ace_hw_rotate", C.c_int, _vp, _vp, _vp, _vp, _sz, _sz)
    f("ace_find_automorphism_index", C.c_uint32, _vp, C.c_int32)
    f("ace_automorphism_order", C.c_int, _vp, _vp, C.c_uint32, C.c_int)
    for n in ("add", "sub", "mul"):
        f("ace_poly_" + n, C.c_int, _vp, _vp, _vp, _vp, _sz, C.c_int)
    f("ace_poly_automorphism", C.c_int, _vp, _vp, _vp, _vp, _sz, C.c_int)
    f("ace_decomp_modup", C.c_int, _vp, _vp, _vp, _sz, _sz, C.c_int)
    f("ace_mod_up", C.c_int, _vp, _vp, _vp, _sz, _sz, C.c_int)
    f("ace_host_fft_tables", C.c_int, _vp, _vp, _vp)
    f("ace_embedding_inv", C.c_int, _vp, _vp, _vp, _sz)
    for n in ("ace_fork", "ace_fork_switch", "ace_join"):
        f(n, C.c_int, _vp)
    f("ace_decode", C.c_int, _vp, _vp, _vp, _sz, C.c_int, C.c_uint32, C.c_double)
    f("ace_encode", C.c_int, _vp, _vp, _vp, _sz, C.c_uint32, _sz, C.c_uint32, _sz)
    f("ace_ext_plain_mac_groups", C.c_int, _vp, _vp, _vp, _sz, _vp, _vp, _sz, _vp, _sz, _sz)
    f("ace_ext_rotate", C.c_int, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp, _sz, C.c_int)
    f("ace_encode_scaled", C.c_int, _vp, _vp, _vp, _sz, C.c_uint32, _sz, C.c_double, _sz)
    f("ace_encode_real_batch", C.c_int, _vp, _vp, _sz, _vp, C.c_int, _sz, _sz, C.c_uint32, _sz, C.c_uint32, _sz)
    f("ace_encode_real", C.c_int, _vp, _vp, _vp, C.c_int, _sz, C.c_uint32, _sz, C.c_uint32, _sz)
    f("ace_mod_down_rescale", C.c_int, _vp, _vp, _vp, _sz, C.c_int)
    f("ace_reduce_rescale_modup", C.c_int, _vp, _vp, _vp, _vp, _sz, C.c_int)
    f("ace_transform_from_level0", C.c_int, _vp, _vp, _vp, _sz)
    f("ace_precomp", C.c_int, _vp, _vp, _vp, _sz, C.c_int)
    f("ace_mod_down", C.c_int, _vp, _vp, _vp, _sz, C.c_int)
    f("ace_mod_down_noalloc", C.c_int, _vp, _vp, _vp, _sz, C.c_int)
    f("ace_precomp_batch", C.c_int, _vp, _vp, _sz, _vp, _sz, _sz, _sz, C.c_int)
    f("ace_mod_down_batch", C.c_int, _vp, _vp, _sz, _vp, _sz, _sz, _sz, C.c_int)
    f("ace_rescale", C.c_int, _vp, _vp, _vp, _sz, C.c_int)
    f("ace_extend", C.c_int, _vp, _vp, _vp, _sz)
    f("ace_dot_prod", C.c_int, _vp, _vp, _vp, _vp, _sz, _sz, _sz)
    f("ace_mul_ciph3", C.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz)
    f("ace_fast_switch_key", C.c_int, _vp, _vp, _vp, _vp, _vp, _sz)
    f("ace_relin", C.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz)
    f("ace_rescale_ciph", C.c_int, _vp, _vp, _vp, _vp, _vp, _sz)
    f("ace_mul_relin_rescale", C.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz)
    f("ace_mod_down_pair_rescale", C.c_int, _vp, _vp, _vp, _vp, _vp, _sz)
    f("ace_mul_relin_double_rescale", C.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz)
    f("ace_mul_relin_double_add_rescale", C.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64p, _sz)
    f("ace_mul_relin_rescale_batch", C.c_int, _vp, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _sz, _vp, _sz, _sz)
    f("ace_fast_rotate", C.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz)
    f("ace_rotate_batch", C.c_int, _vp, _vp, _vp, _vp, _vp, C.POINTER(_vp), C.POINTER(_vp), _sz, _sz)
    f("ace_poly_add_scalars", C.c_int, _vp, _vp, _vp, _i64p, _sz)
    f("ace_poly_mul_scalars", C.c_int, _vp, _vp, _vp, _i64p, _sz)
    f("ace_ciph_wsum", C.c_int, _vp, _vp, _vp, C.POINTER(_vp), C.POINTER(_vp), _i64p, _sz, _sz)
    f("ace_alloc_uninit", _vp, _vp, _sz)
    f("ace_set_batching", C.c_int, _vp, C.c_int)
    f("ace_sample_uniform", C.c_int, _vp, _vp, _sz, C.c_int, C.c_uint64, C.c_uint64)
    f("ace_expand_small", C.c_int, _vp, _vp, _i64p, _sz, C.c_int)
    f("ace_ext_plain_mac", C.c_int, _vp, _vp, _vp, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), _sz, _sz, _sz, C.c_int)


# every symbol include/ace_hip.h declares
EXPORTS = [
    "ace_mod_down_noalloc", "ace_precomp_batch", "ace_mod_down_batch", "ace_sample_uniform", "ace_expand_small", "ace_set_batching", "ace_ext_plain_mac", "ace_poly_add_scalars", "ace_poly_mul_scalars", "ace_ciph_wsum", "ace_alloc_uninit", "ace_ctx_create", "ace_ctx_create_with_primes", "ace_ctx_destroy", "ace_has_device", "ace_last_error",
    "ace_degree", "ace_num_q", "ace_num_p", "ace_num_parts", "ace_part_size", "ace_num_decomp", "ace_prime",
    "ace_root", "ace_modulus", "ace_host_twiddles", "ace_host_tbl_modup", "ace_host_tbl_moddown",
    "ace_host_tbl_rescale", "ace_host_automorphism_order", "ace_alloc", "ace_free", "ace_upload", "ace_download",
    "ace_copy", "ace_zero", "ace_sync", "ace_sync_device", "ace_memory_stats", "ace_ctx_share", "ace_fork_release", "ace_census_mark", "ace_timer_start", "ace_timer_stop_ms", "ace_ntt", "ace_intt", "ace_ntt_pass",
    "ace_hw_modadd", "ace_hw_modsub", "ace_hw_modmul", "ace_hw_modmuladd", "ace_hw_modadd_scalar",
    "ace_hw_modsub_scalar", "ace_hw_modmul_scalar", "ace_hw_modmuladd_scalar", "ace_hw_rotate",
    "ace_find_automorphism_index", "ace_automorphism_order", "ace_poly_add", "ace_poly_sub", "ace_poly_mul",
    "ace_poly_automorphism", "ace_decomp_modup", "ace_mod_up", "ace_mod_down_rescale",
    "ace_reduce_rescale_modup", "ace_transform_from_level0", "ace_host_fft_tables", "ace_embedding_inv", "ace_decode", "ace_fork", "ace_fork_switch", "ace_join", "ace_encode", "ace_encode_scaled", "ace_encode_real", "ace_encode_real_batch", "ace_ext_rotate", "ace_ext_plain_mac_groups", "ace_precomp", "ace_mod_down", "ace_rescale", "ace_extend",
    "ace_dot_prod", "ace_mul_ciph3", "ace_fast_switch_key", "ace_relin", "ace_rescale_ciph",
    "ace_mul_relin_rescale", "ace_mod_down_pair_rescale", "ace_mul_relin_double_rescale", "ace_mul_relin_double_add_rescale", "ace_mul_relin_rescale_batch", "ace_fast_rotate", "ace_rotate_batch",
]

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("libace_hip.so is not built: run `python -c 'import __graft_entry__ as g; g.build()'`")
        _lib = C.CDLL(LIB_PATH)
        _sig(_lib)
    return _lib


class DevBuf:
    """n int64 words of HBM owned by a context."""

    def __init__(self, ctx, n_words, ptr=None):
        self.ctx, self.n = ctx, int(n_words)
        self.own = ptr is None
        self.ptr = ctx.lib.ace_alloc(ctx.h, self.n) if ptr is None else ptr
        if not self.ptr:
            raise AceError(ctx.err())

    def get(self):
        out = np.empty(self.n, np.int64)
        self.ctx._chk(self.ctx.lib.ace_download(self.ctx.h, out.ctypes.data_as(_i64p), self.ptr, self.n))
        return out

    def set(self, arr):
        arr = np.ascontiguousarray(arr, dtype=np.int64).ravel()
        assert arr.size == self.n
        self.ctx._chk(self.ctx.lib.ace_upload(self.ctx.h, self.ptr, arr.ctypes.data_as(_i64p), self.n))
        return self

    def view(self, off_words, n_words):
        assert off_words + n_words <= self.n
        return DevBuf(self.ctx, n_words, ptr=self.ptr + 8 * off_words)

    def free(self):
        if self.own and self.ptr:
            self.ctx.lib.ace_free(self.ctx.h, self.ptr)
            self.ptr = None


class Context:
    """One CRT context (primes, tables in HBM, one HIP stream)."""

    def __init__(self, degree, num_q, q0_bits=0, sf_bits=0, parts=1, primes=None, share=None):
        self.lib = lib()
        if share is not None:  # a further context over `share`'s tables, for another host thread
            h = self.lib.ace_ctx_share(share.h)
        elif primes is None:
            h = self.lib.ace_ctx_create(degree, num_q, q0_bits, sf_bits, parts)
        else:
            p = np.ascontiguousarray(primes, dtype=np.int64)
            h = self.lib.ace_ctx_create_with_primes(degree, len(p), p.ctypes.data_as(_i64p), parts)
        if not h:
            raise AceError(self.err())
        self.h = _vp(h)
        self.N = self.lib.ace_degree(self.h)
        self.L = self.lib.ace_num_q(self.h)
        self.K = self.lib.ace_num_p(self.h)
        self.parts = self.lib.ace_num_parts(self.h)
        self.part_size = self.lib.ace_part_size(self.h)
        self.primes = [self.lib.ace_prime(self.h, i) for i in range(self.L + self.K)]
        self.roots = [self.lib.ace_root(self.h, i) for i in range(self.L + self.K)]
        self.has_device = bool(self.lib.ace_has_device(self.h))

    def share(self):
        """A context over the same tables with its own stream, arena and pool (close it before this one)."""
        return Context(0, 0, share=self)

    def err(self):
        return (self.lib.ace_last_error() or b"").decode()

    def _chk(self, rc):
        if rc != 0:
            raise AceError(self.err())

    def close(self):
        if self.h:
            self.lib.ace_ctx_destroy(self.h)
            self.h = None

    # ---- getters / host tables
    def num_decomp(self, level):
        return self.lib.ace_num_decomp(self.h, level)

    def modulus(self, i):
        out = (C.c_uint64 * 5)()
        self.lib.ace_modulus(self.h, i, out)
        return list(out)

    def limb_primes(self, level, with_p=True):
        return list(range(level)) + ([self.L + j for j in range(self.K)] if with_p else [])

    def twiddles(self, i, which):
        out = np.empty(self.N, np.uint64)
        self._chk(self.lib.ace_host_twiddles(self.h, i, which, out.ctypes.data_as(_u64p)))
        return out

    def tbl_modup(self, level, part):
        hat_inv = np.zeros(96, np.int64)
        hat = np.zeros(96 * 96, np.int64)
        cidx = np.zeros(96, np.int32)
        nd, nc = _sz(), _sz()
        self._chk(self.lib.ace_host_tbl_modup(self.h, level, part, hat_inv.ctypes.data_as(_i64p),
                                              hat.ctypes.data_as(_i64p), cidx.ctypes.data_as(_i32p),
                                              C.byref(nd), C.byref(nc)))
        nd, nc = nd.value, nc.value
        return hat_inv[:nd].copy(), hat[:nd * nc].reshape(nd, nc).copy(), cidx[:nc].copy()

    def tbl_moddown(self):
        a = np.zeros(self.K, np.int64)
        b = np.zeros(self.L * self.K, np.int64)
        c = np.zeros(self.L, np.int64)
        d = np.zeros(self.L, np.int64)
        self._chk(self.lib.ace_host_tbl_moddown(self.h, *[x.ctypes.data_as(_i64p) for x in (a, b, c, d)]))
        return a, b.reshape(self.L, self.K), c, d

    def tbl_rescale(self, level):
        a = np.zeros(level - 1, np.int64)
        b = np.zeros(level - 1, np.int64)
        self._chk(self.lib.ace_host_tbl_rescale(self.h, level, a.ctypes.data_as(_i64p), b.ctypes.data_as(_i64p)))
        return a, b

    def find_automorphism_index(self, rot):
        return self.lib.ace_find_automorphism_index(self.h, rot)

    def host_automorphism_order(self, k, is_ntt=True):
        out = np.zeros(self.N, np.int64)
        self._chk(self.lib.ace_host_automorphism_order(self.h, out.ctypes.data_as(_i64p), k, int(is_ntt)))
        return out

    # ---- memory
    def alloc(self, n_words):
        return DevBuf(self, n_words)

    def upload(self, arr):
        arr = np.ascontiguousarray(arr, dtype=np.int64).ravel()
        return DevBuf(self, arr.size).set(arr)

    def copy(self, dst, src, n_words=None):
        self._chk(self.lib.ace_copy(self.h, dst.ptr, src.ptr, src.n if n_words is None else n_words))

    def fork(self):
        self._chk(self.lib.ace_fork(self.h))

    def fork_switch(self):
        self._chk(self.lib.ace_fork_switch(self.h))

    def join(self):
        self._chk(self.lib.ace_join(self.h))

    def fork_release(self):
        self._chk(self.lib.ace_fork_release(self.h))

    def sync(self):
        self._chk(self.lib.ace_sync(self.h))

    def memory_stats(self):
        """(arena words, pooled words, live buffers, pooled buffers) of the context right now."""
        out = (C.c_size_t * 4)()
        self.lib.ace_memory_stats(self.h, out)
        return tuple(int(v) for v in out)

    def timer_start(self):
        self._chk(self.lib.ace_timer_start(self.h))

    def timer_stop_ms(self):
        ms = self.lib.ace_timer_stop_ms(self.h)
        if ms < 0:
            raise AceError(self.err())
        return ms

    # ---- NTT
    def ntt(self, dst, src, prime_idx, n_polys=1, poly_stride_limbs=0, inverse=False):
        idx = np.ascontiguousarray(prime_idx, dtype=np.int32)
        f = self.lib.ace_intt if inverse else self.lib.ace_ntt
        self._chk(f(self.h, dst.ptr, src.ptr, idx.ctypes.data_as(_i32p), len(idx), n_polys, poly_stride_limbs))

    def intt(self, dst, src, prime_idx, n_polys=1, poly_stride_limbs=0):
        self.ntt(dst, src, prime_idx, n_polys, poly_stride_limbs, inverse=True)

    def ntt_pass(self, dst, src, prime_idx, n_polys, poly_stride_limbs, inverse, which):
        idx = np.ascontiguousarray(prime_idx, dtype=np.int32)
        self._chk(self.lib.ace_ntt_pass(self.h, dst.ptr, src.ptr, idx.ctypes.data_as(_i32p), len(idx), n_polys,
                                        poly_stride_limbs, int(inverse), which))

    # ---- Hw_*
    def hw(self, name, r, a, b, prime_idx, n=None):
        n = a.n if n is None else n
        f = getattr(self.lib, "ace_hw_" + name)
        if name.endswith("_scalar"):
            self._chk(f(self.h, r.ptr, a.ptr, int(b), prime_idx, n))
        else:
            self._chk(f(self.h, r.ptr, a.ptr, b.ptr, prime_idx, n))

    def automorphism_order(self, k, is_ntt=True):
        buf = self.alloc(self.N)
        self._chk(self.lib.ace_automorphism_order(self.h, buf.ptr, k, int(is_ntt)))
        return buf

    # ---- polynomial ops
    def poly(self, name, r, a, b, level, with_p=False):
        self._chk(getattr(self.lib, "ace_poly_" + name)(self.h, r.ptr, a.ptr, b.ptr, level, int(with_p)))

    def decomp_modup(self, res, src, level, part, is_ntt=True):
        self._chk(self.lib.ace_decomp_modup(self.h, res.ptr, src.ptr, level, part, int(is_ntt)))

    def mod_down_rescale(self, res, poly, level, is_ntt=True):
        self._chk(self.lib.ace_mod_down_rescale(self.h, res.ptr, poly.ptr, level, int(is_ntt)))

    def reduce_rescale_modup(self, res, raised, poly, level, is_ntt=True):
        self._chk(self.lib.ace_reduce_rescale_modup(self.h, res.ptr, raised.ptr, poly.ptr, level, int(is_ntt)))

    def transform_from_level0(self, res, src, level):
        self._chk(self.lib.ace_transform_from_level0(self.h, res.ptr, src.ptr, level))

    def host_fft_tables(self):
        rou = np.zeros(4 * self.N, np.float64)
        rot = np.zeros(max(1, self.N // 2), np.uint32)
        self._chk(self.lib.ace_host_fft_tables(self.h, rou.ctypes.data_as(C.c_void_p), rot.ctypes.data_as(C.c_void_p)))
        return rou, rot

    def embedding_inv(self, values):
        v = np.ascontiguousarray(values, dtype=np.complex128)
        out = np.zeros_like(v)
        self._chk(self.lib.ace_embedding_inv(self.h, out.ctypes.data_as(C.c_void_p), v.ctypes.data_as(C.c_void_p), v.size))
        return out

    def decode(self, poly, level, slots, factor, is_ntt=True):
        out = np.zeros(slots or self.N // 2, np.complex128)
        self._chk(self.lib.ace_decode(self.h, out.ctypes.data_as(C.c_void_p), poly.ptr, level, int(is_ntt), slots,
                                      float(factor)))
        return out

    def encode(self, res, values, slots=0, level=0, sf_degree=1, p_cnt=0):
        v = np.ascontiguousarray(values, dtype=np.complex128)
        self._chk(self.lib.ace_encode(self.h, res.ptr, v.ctypes.data_as(C.c_void_p), v.size, slots, level, sf_degree,
                                      p_cnt))

    def encode_scaled(self, res, values, slots, level, scale, p_cnt=0):
        v = np.ascontiguousarray(values, dtype=np.complex128)
        self._chk(self.lib.ace_encode_scaled(self.h, res.ptr, v.ctypes.data_as(C.c_void_p), v.size, slots, level,
                                             float(scale), p_cnt))

    def encode_real(self, res, values, slots=0, level=0, sf_degree=1, p_cnt=0):
        """values: a float32 or float64 array of real numbers."""
        v = np.ascontiguousarray(values)
        assert v.dtype in (np.float32, np.float64)
        self._chk(self.lib.ace_encode_real(self.h, res.ptr, v.ctypes.data_as(C.c_void_p), int(v.dtype == np.float32), v.size,
                                           slots, level, sf_degree, p_cnt))

    def encode_real_batch(self, res, res_stride, vectors, slots=0, level=0, sf_degree=1, p_cnt=0):
        """vectors: equally long float32 or float64 arrays, one per polynomial."""
        vs = [np.ascontiguousarray(v) for v in vectors]
        assert vs and all(v.dtype == vs[0].dtype and v.size == vs[0].size for v in vs)
        ptrs = (C.c_void_p * len(vs))(*[v.ctypes.data for v in vs])
        self._chk(self.lib.ace_encode_real_batch(self.h, res.ptr, res_stride, ptrs, int(vs[0].dtype == np.float32),
                                                 vs[0].size, len(vs), slots, level, sf_degree, p_cnt))

    def mod_up(self, res, digit, level, part, is_ntt=True):
        self._chk(self.lib.ace_mod_up(self.h, res.ptr, digit.ptr, level, part, int(is_ntt)))

    def precomp(self, res, src, level, is_ntt=True):
        self._chk(self.lib.ace_precomp(self.h, res.ptr, src.ptr, level, int(is_ntt)))

    def mod_down(self, res, src, level, is_ntt=True):
        self._chk(self.lib.ace_mod_down(self.h, res.ptr, src.ptr, level, int(is_ntt)))

    def precomp_batch(self, res, res_stride, src, src_stride, count, level, is_ntt=True):
        self._chk(self.lib.ace_precomp_batch(self.h, res.ptr, res_stride, src.ptr, src_stride, count, level, int(is_ntt)))

    def mod_down_batch(self, res, res_stride, src, src_stride, count, level, is_ntt=True):
        self._chk(self.lib.ace_mod_down_batch(self.h, res.ptr, res_stride, src.ptr, src_stride, count, level, int(is_ntt)))

    def mod_down_noalloc(self, res, src, level, is_ntt=True):
        self._chk(self.lib.ace_mod_down_noalloc(self.h, res.ptr, src.ptr, level, int(is_ntt)))

    def rescale(self, res, src, level, is_ntt=True):
        self._chk(self.lib.ace_rescale(self.h, res.ptr, src.ptr, level, int(is_ntt)))

    def extend(self, res, src, level):
        self._chk(self.lib.ace_extend(self.h, res.ptr, src.ptr, level))

    def ext_rotate(self, out0, out1, digits, key, key_half_words, key_stride, n_parts, addend0, order, level,
                   accumulate=0):
        self._chk(self.lib.ace_ext_rotate(self.h, out0.ptr, out1.ptr, digits.ptr, key.ptr, key_half_words, key_stride,
                                          n_parts, addend0.ptr if addend0 is not None else None, order.ptr, level,
                                          accumulate))

    def dot_prod(self, res, digits, key, key_stride, n_parts, level):
        self._chk(self.lib.ace_dot_prod(self.h, res.ptr, digits.ptr, key.ptr, key_stride, n_parts, level))

    # ---- ciphertext level
    def mul_ciph3(self, d0, d1, d2, a0, a1, b0, b1, level):
        self._chk(self.lib.ace_mul_ciph3(self.h, d0.ptr, d1.ptr, d2.ptr, a0.ptr, a1.ptr, b0.ptr, b1.ptr, level))

    def fast_switch_key(self, o0, o1, digits, swk, level):
        self._chk(self.lib.ace_fast_switch_key(self.h, o0.ptr, o1.ptr, digits.ptr, swk.ptr, level))

    def relin(self, r0, r1, d0, d1, d2, swk, level):
        self._chk(self.lib.ace_relin(self.h, r0.ptr, r1.ptr, d0.ptr, d1.ptr, d2.ptr, swk.ptr, level))

    def rescale_ciph(self, r0, r1, c0, c1, level):
        self._chk(self.lib.ace_rescale_ciph(self.h, r0.ptr, r1.ptr, c0.ptr, c1.ptr, level))

    def mul_relin_rescale(self, r0, r1, a0, a1, b0, b1, swk, level):
        self._chk(self.lib.ace_mul_relin_rescale(self.h, r0.ptr, r1.ptr, a0.ptr, a1.ptr, b0.ptr, b1.ptr, swk.ptr, level))

    def mod_down_pair_rescale(self, r0, r1, e0, e1, level):
        self._chk(self.lib.ace_mod_down_pair_rescale(self.h, r0.ptr, r1.ptr, e0.ptr, e1.ptr, level))

    def mul_relin_double_rescale(self, r0, r1, a0, a1, b0, b1, swk, level):
        self._chk(self.lib.ace_mul_relin_double_rescale(self.h, r0.ptr, r1.ptr, a0.ptr, a1.ptr, b0.ptr, b1.ptr, swk.ptr,
                                                        level))

    def mul_relin_double_add_rescale(self, r0, r1, a0, a1, b0, b1, swk, constant, level):
        sc = np.ascontiguousarray(constant, dtype=np.int64)
        assert sc.size >= level
        self._chk(self.lib.ace_mul_relin_double_add_rescale(self.h, r0.ptr, r1.ptr, a0.ptr, a1.ptr, b0.ptr, b1.ptr,
                                                            swk.ptr, sc.ctypes.data_as(_i64p), level))

    def mul_relin_rescale_batch(self, r0, r1, out_stride, a0, a1, b0, b1, in_stride, swk, level, count):
        self._chk(self.lib.ace_mul_relin_rescale_batch(self.h, r0.ptr, r1.ptr, out_stride, a0.ptr, a1.ptr, b0.ptr,
                                                       b1.ptr, in_stride, swk.ptr, level, count))

    def fast_rotate(self, r0, r1, c0, digits, swk, order, level):
        self._chk(self.lib.ace_fast_rotate(self.h, r0.ptr, r1.ptr, c0.ptr, digits.ptr, swk.ptr, order.ptr, level))

    def poly_scalars(self, mul, r, a, scalars, level):
        sc = np.ascontiguousarray(scalars, dtype=np.int64)
        fn = self.lib.ace_poly_mul_scalars if mul else self.lib.ace_poly_add_scalars
        self._chk(fn(self.h, r.ptr, a.ptr, sc.ctypes.data_as(_i64p), level))

    def ciph_wsum(self, r0, r1, a0s, a1s, weights, level):
        n = len(a0s)
        w = np.ascontiguousarray(weights, dtype=np.int64).ravel()
        assert w.size == n * level
        p0 = (_vp * n)(*[a.ptr for a in a0s])
        p1 = (_vp * n)(*[a.ptr for a in a1s])
        self._chk(self.lib.ace_ciph_wsum(self.h, r0.ptr, r1.ptr, p0, p1, w.ctypes.data_as(_i64p), n, level))

    def sample_uniform(self, r, level, with_p, seed, stream):
        self._chk(self.lib.ace_sample_uniform(self.h, r.ptr, level, int(with_p), seed, stream))

    def expand_small(self, r, small, level, with_p):
        v = np.ascontiguousarray(small, dtype=np.int64)
        assert v.size == self.N
        self._chk(self.lib.ace_expand_small(self.h, r.ptr, v.ctypes.data_as(_i64p), level, int(with_p)))

    def set_batching(self, on):
        self._chk(self.lib.ace_set_batching(self.h, int(bool(on))))

    def ext_plain_mac(self, r0, r1, a0s, a1s, plains, level, plain_level, accumulate=False):
        n = len(plains)
        p0 = (_vp * n)(*[a.ptr for a in a0s])
        p1 = (_vp * n)(*[a.ptr for a in a1s])
        pp = (_vp * n)(*[a.ptr for a in plains])
        self._chk(self.lib.ace_ext_plain_mac(self.h, r0.ptr, r1.ptr, p0, p1, pp, C.c_size_t(n), C.c_size_t(level),
                                             C.c_size_t(plain_level), C.c_int(int(accumulate))))

    def ext_plain_mac_groups(self, r0s, r1s, a0s, a1s, plains, level, plain_level):
        """plains[g][j]: the plaintext of group g, operand j, or None."""
        ng, n = len(r0s), len(a0s)
        q0 = (_vp * ng)(*[r.ptr for r in r0s])
        q1 = (_vp * ng)(*[r.ptr for r in r1s])
        p0 = (_vp * n)(*[a.ptr for a in a0s])
        p1 = (_vp * n)(*[a.ptr for a in a1s])
        pp = (_vp * (ng * n))(*[(plains[g][j].ptr if plains[g][j] is not None else None) for g in range(ng) for j in range(n)])
        self._chk(self.lib.ace_ext_plain_mac_groups(self.h, q0, q1, C.c_size_t(ng), p0, p1, C.c_size_t(n), pp,
                                                    C.c_size_t(level), C.c_size_t(plain_level)))

    def rotate_batch(self, r0s, r1s, c0, c1, swks, orders, level):
        n = len(swks)
        ks = (_vp * n)(*[k.ptr for k in swks])
        os_ = (_vp * n)(*[o.ptr for o in orders])
        self._chk(self.lib.ace_rotate_batch(self.h, r0s.ptr, r1s.ptr, c0.ptr, c1.ptr, ks, os_, n, level))
