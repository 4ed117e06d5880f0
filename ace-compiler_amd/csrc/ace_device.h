// Device-side data structures and 64-bit modular arithmetic for gfx950.
//
// All residues are 64-bit words in [0, q), q < 2^61.  There is no 64x64->128
// VALU multiply on CDNA4; __umul64hi and `*` lower to v_mad_u64_u32 chains.
// Three reductions are used, each value-identical to the reference's because
// the canonical residue of an integer is unique:
//   shoup_*    multiply by a constant w with precomputed floor(w*2^64/q)
//              (Fast_mul_const_with_mod, include/util/modular.h:249-256)
//   mulmod     product of two residues, shifted Barrett with a 64-bit mu
//              (same result as Mul_int64_mod_barret, modular.h:231-241)
//   barrett128 any 128-bit value, mu = floor(2^128/q)
//              (Mod_barrett_128, modular.h:185-224)
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ace {

typedef uint64_t u64;
typedef int64_t  i64;
typedef uint32_t u32;

constexpr int kMaxPrimes = 96;

struct DevPrime {
  u64 q;
  u64 mu_lo, mu_hi;  // floor(2^128/q)
  u64 mu_sh;         // floor(2^(shift+64)/q)
  u32 shift;         // bitlen(q)-1
  u32 pad;
  u64 ninv, ninv_p;  // N^-1 mod q and its Shoup companion
};

// What every kernel needs to find primes and twiddles.
struct DevCtx {
  const DevPrime* primes;
  const u64 *rou, *rou_p, *irou, *irou_p;  // [num primes][N]
  // FP64 copies of rou / irou for the primes flagged in fp_ok
  const double *roud, *iroud;
  u32 N, logN;
  uint8_t fp_ok[kMaxPrimes];  // prime is small enough for the FP64 NTT back end
};

// largest prime the FP64 back end accepts: below 2^50.2, so that eight stages'
// worth of lazily accumulated magnitude stays under 2^53 (see ace_ntt.hip)
constexpr u64 kFpPrimeLimit = 1290000000000000ull;
// largest target prime of the FP64 base conversion (3 * 2^50): the halves of a cofactor stay below 2^26, so 48
// products with 21-bit pieces of the sources add up below 2^53, and 1.4 m < 2^53 in the final reduction
constexpr u64 kFpConvTargetLimit = (u64)3 << 50;

// limb t of a launch -> prime index
struct LimbMap {
  uint8_t prime[kMaxPrimes];
};

// A sequence of polynomials addressed as pairs: polynomial p lives at
// b[p & 1] + (p >> 1) * pair_stride words.  Covers a plain strided batch
// (b[1] = b[0] + stride, pair_stride = 2*stride) as well as the two halves
// (c0, c1) of a batch of ciphertexts held in separate buffers.
struct PolySeq {
  u64* b[2];
  u64 pair_stride;
  __host__ __device__ __forceinline__ u64* at(u32 p) const { return b[p & 1] + (u64)(p >> 1) * pair_stride; }
};
inline PolySeq seq_strided(const u64* base, u64 stride) {
  PolySeq s;
  s.b[0] = const_cast<u64*>(base);
  s.b[1] = const_cast<u64*>(base) + stride;
  s.pair_stride = 2 * stride;
  return s;
}
inline PolySeq seq_pair(const u64* c0, const u64* c1, u64 op_stride) {
  PolySeq s;
  s.b[0] = const_cast<u64*>(c0);
  s.b[1] = const_cast<u64*>(c1);
  s.pair_stride = op_stride;
  return s;
}

// where an inverse transform drops a copy of the words it reads: limb t of polynomial p goes to
// seq.at(p) + (t / part_size) * digit_stride + t * N (the digits' own limbs inside raised polynomials)
struct CopyThrough {
  PolySeq seq;
  u64 digit_stride;
  u32 part_size;
};

// base conversion: target j -> prime index and limb position in the output
struct ConvMap {
  uint8_t prime[kMaxPrimes];
  uint8_t out_limb[kMaxPrimes];
};

__device__ __forceinline__ u64 csub(u64 a, u64 q) { return a >= q ? a - q : a; }

// a*w mod q up to one extra q: result in [0, 2q) for any a < 2^64
__device__ __forceinline__ u64 shoup_lazy(u64 a, u64 w, u64 wp, u64 q) {
  return a * w - __umul64hi(a, wp) * q;
}
// The same with the quotient a*wp / 2^64 estimated from three of the four partial products (the low x low one and
// the carries of the middle sum are dropped): at most 2 too small, so the result is in [0, 4q).  Five instructions
// for the quotient instead of about ten; for the NTT butterflies, whose lazy ranges absorb the slack (q < 2^61).
__device__ __forceinline__ u64 shoup_lazier(u64 a, u64 w, u64 wp, u64 q) {
  const u32 ah = (u32)(a >> 32), al = (u32)a, ph = (u32)(wp >> 32), pl = (u32)wp;
  const u64 quot = (u64)ah * ph + __umulhi(ah, pl) + __umulhi(al, ph);
  return a * w - quot * q;
}
__device__ __forceinline__ u64 shoup_mul(u64 a, u64 w, u64 wp, u64 q) {
  return csub(shoup_lazy(a, w, wp, q), q);
}

// a*b mod q for a*b < 2^(2*(shift+1))
__device__ __forceinline__ u64 mulmod(u64 a, u64 b, const DevPrime& p) {
  u64 lo = a * b, hi = __umul64hi(a, b);
  u64 x1 = (hi << (64 - p.shift)) | (lo >> p.shift);
  u64 r  = lo - __umul64hi(x1, p.mu_sh) * p.q;  // < 3q
  return csub(csub(r, p.q), p.q);
}

// (hi:lo) mod q for a value below 2^(shift + 64), e.g. a sum of up to sum_terms(p) products of residues: the
// single-word Barrett step of mulmod, a third of barrett128's multiplies, and the same canonical residue
__device__ __forceinline__ u64 barrett_sum(u64 hi, u64 lo, const DevPrime& p) {
  u64 x1 = (hi << (64 - p.shift)) | (lo >> p.shift);
  u64 r  = lo - __umul64hi(x1, p.mu_sh) * p.q;  // < 3q
  return csub(csub(r, p.q), p.q);
}
// how many products of residues (each below 2^(2 shift + 2)) stay below 2^(shift + 64) when added up
__device__ __forceinline__ u32 sum_terms(const DevPrime& p) { return p.shift >= 60 ? 4u : p.shift == 59 ? 8u : 16u; }

// (hi:lo) mod q for any 128-bit value
__device__ __forceinline__ u64 barrett128(u64 hi, u64 lo, const DevPrime& p) {
  u64 ll_hi = __umul64hi(lo, p.mu_lo);
  u64 lh_lo = lo * p.mu_hi, lh_hi = __umul64hi(lo, p.mu_hi);
  u64 hl_lo = hi * p.mu_lo, hl_hi = __umul64hi(hi, p.mu_lo);
  u64 s1 = ll_hi + lh_lo;
  u64 c1 = s1 < ll_hi;
  u64 s2 = s1 + hl_lo;
  u64 c2 = s2 < s1;
  u64 qhat = lh_hi + hl_hi + c1 + c2 + hi * p.mu_hi;
  u64 r = lo - qhat * p.q;  // < 2q
  return csub(csub(r, p.q), p.q);
}

// Sub_mul_const_mod (modular.h:262-276), literally: ((v1 - v2) * w) mod q with the
// Shoup companion wp.  One +q after the subtraction; if the difference is still
// negative (v2 a residue of a larger prime) the reference's casts decide the
// value: the 128-bit product sees the sign-extended difference, i.e. the high
// word of s*wp taken as unsigned minus wp.
__device__ __forceinline__ u64 sub_mul_const(u64 v1, u64 v2, u64 w, u64 wp, u64 q) {
  i64 s = (i64)v1 - (i64)v2;
  if (s < 0) s += (i64)q;
  u64 qq = __umul64hi((u64)s, wp) - (s < 0 ? wp : 0);
  u64 y = (u64)s * w - qq * q;
  return y >= q ? y - q : y;
}

// acc += a*b over 128 bits
__device__ __forceinline__ void mac128(u64& hi, u64& lo, u64 a, u64 b) {
  u64 pl = a * b, ph = __umul64hi(a, b);
  lo += pl;
  hi += ph + (lo < pl);
}

// Add_int64_with_mod / Sub_int64_with_mod (modular.h:139-160), literally
__device__ __forceinline__ u64 add_mod(u64 a, u64 b, u64 q) {
  i64 s = (i64)(a + b);
  return (u64)(s >= (i64)q ? s - (i64)q : s);
}
__device__ __forceinline__ u64 sub_mod(u64 a, u64 b, u64 q) {
  i64 r = (i64)(a - b);
  if (r > (i64)a || r < 0) r += (i64)q;
  return (u64)r;
}


// ---- pieces of the base conversion on the matrix cores shared by its kernels (see baseconv_mx_kernel) ----
typedef int conv_v16i __attribute__((ext_vector_type(16)));
typedef int conv_v4i __attribute__((ext_vector_type(4)));
constexpr u64 kSignedBytes = 0x8080808080808080ull;
// a source word as the MFMA's B operand takes it: its eight signed bytes (the carries moved up), low half first
__device__ __forceinline__ void conv_mx_signed(u64 word, bool live, int& lo, int& hi) {
  const u64 e = live ? (word + kSignedBytes) ^ kSignedBytes : 0;
  lo = (int)(u32)e;
  hi = (int)(u32)(e >> 32);
}
// the canonical residue mod m of V = sum_p 2^(8p) S[8w + p], the eight byte sums of target w of a lane's pair
__device__ __forceinline__ u64 conv_mx_residue(const conv_v16i& S, int w, u64 m, double minv) {
  // byte sums are below 2^21 in size: two of them, one shifted by a byte, fit a 32-bit word
  const int u0 = S[8 * w + 0] + (S[8 * w + 1] << 8), v0 = S[8 * w + 2] + (S[8 * w + 3] << 8);
  const int u1 = S[8 * w + 4] + (S[8 * w + 5] << 8), v1 = S[8 * w + 6] + (S[8 * w + 7] << 8);
  const i64 t0 = (i64)u0 + ((i64)v0 << 16), t1 = (i64)u1 + ((i64)v1 << 16);
  const u64 v_lo = (u64)t0 + ((u64)t1 << 32);  // V mod 2^64
  const double d0 = __builtin_fma((double)v0, 65536.0, (double)u0);  // exact
  const double d1 = __builtin_fma((double)v1, 65536.0, (double)u1);
  const double vd = __builtin_fma(d1, 4294967296.0, d0);  // V to 53 bits
  // |V / m| < 2^14 and the estimate is off by far less than 1/2: V - Q m lies within (1/2 + 2^-30) m of zero
  const int quot = (int)__builtin_rint(vd * minv);
  const i64 r = (i64)(v_lo - (u64)(i64)quot * m);
  return (u64)(r < 0 ? r + (i64)m : r);
}

constexpr int kMaxBatchPtrs = 32;  // keys / index tables per batched launch
struct OrderSet {  // one automorphism table per rotation, or one shared (n == 1)
  const i64* p[kMaxBatchPtrs];
  u32 n;
};

// Work folded into a forward NTT of N > 4096 (launch_ntt): a prologue that forms
// the transform's input on the fly, and an epilogue that consumes its output
// instead of storing it.  Limb t of polynomial p is word offset pos[t]*N.
//   pro 1  Rescale's modulus switch (rns_poly.c:340-360): input word i of limb t =
//          Switch_modulus(last[p*last_stride + i], q_last -> q_t) * sw[3t] (Shoup sw[3t+1], sw[3t+2] = q_t - q_last mod q_t)
//   pro 2  Mod_down and Rescale sharing one forward transform (the transform is linear, so the two that
//          Mod_down and Rescale would run one after the other on the same limbs are one transform of a sum): with
//          y_t = -(P q_last)^-1 times the P part converted to prime t (the transform's source; the constant is part
//          of the conversion's matrix), ylast = P^-1 times the P part converted to the dropped prime, and z = the
//          inverse transform of the dropped limb of (polynomial + P * addend) scaled by P^-1,
//            last[i]   = z[p*z_stride + i] - ylast[p*ylast_stride + i]                (mod q_last)
//            input[i]  = Switch_modulus(last[i], q_last -> q_t) * sw[3t] + y_t[i]     (mod q_t)
//          `last` is the word Rescale's inverse transform of the Mod_down result's last limb would hold.
//   epi 1  Mod_down tail (rns_poly.c:292-303): out = (src - ntt) * cst[2t] (+ addend).  With index tables
//          (orders.n != 0; polynomials 2r and 2r+1 use table r) the automorphism that ends a rotation is applied
//          on the way out: out[i] = the value at orders[i].  The tables must be those of
//          Precompute_automorphism_order for the NTT form (number_theory.c:211-222): an affine map of the
//          evaluation index, which in bit-reversed order takes every aligned block of 2^s words onto one such
//          block, so a 4096-word chunk of the result comes from one chunk of the transform.
//   epi 2  Rescale tail (rns_poly.c:362-372):  out = src * cst[2t] + ntt
// addend_mode: 0 none, 1 every polynomial, 2 even polynomials only.
struct FwdFuse {
  int pro, epi;
  const u64* last;
  u64 last_stride;
  u32 last_prime;
  const u64* sw;
  const u64 *z, *ylast;  // pro 2
  u64 z_stride, ylast_stride;
  PolySeq out, src, addend;
  int addend_mode;
  const u64* cst;
  OrderSet orders;
  // pro 2 with epi 2 only: the Mod_down's result is doubled before the Rescale (Add_ciph of a product with itself
  // between Relinearize and Rescale_ciph): z - ylast, the converted words and the tail's product count twice
  u32 twice;
};

}  // namespace ace
