/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the CKKS polynomial hot path.
 *
 * A plain-C restatement of the reference runtime's algorithms (radix-2
 * negacyclic NTT with Shoup twiddles, Barrett-128 modular multiply, hybrid
 * key-switch base conversion, rescale, automorphism).  It exists to check the
 * HIP implementation bit for bit and to serve as the timed CPU baseline.
 * Only tests, the smoke check and the benchmark's cpu_baseline leg may link
 * or load it; the product library never does.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * fhe-cmplr/rtlib/ant in the reference tree).
 *
 * Pinning status (which independent evidence fixes each function's output):
 *   modular primitives      closed form (__int128 %) + ut_test_number_theory KATs
 *   prime / root generation reference-printed prime lists + Find_generator and
 *                           Root_of_unity KATs + compiled reference (_ref)
 *   NTT / INTT              ut_ntt.cxx vector, brute-force evaluation at odd
 *                           powers of psi, negacyclic product KAT, _ref
 *   elementwise, rotate     closed form, ut_poly.cxx rotate KAT, _ref
 *   Decomp_modup, Mod_down  exact big-integer formula on small rings,
 *                           fused == unfused, Extend->Mod_down identity, _ref
 *   Rescale                 big-integer centred division on small rings, _ref
 *   ciphertext-level ops    composition of the above; decrypt-level check with
 *                           a real key (evaluator.c itself is not buildable
 *                           here, so these are compared by composition only)
 */
#ifndef ACE_ORACLE_H
#define ACE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct orc_ctx orc_ctx;

/* context ---------------------------------------------------------------- */
/* util/src/crt.c:607-618 Init_crtcontext_with_prime_size */
orc_ctx* orc_ctx_create(uint32_t degree, size_t num_q, size_t q0_bits,
                        size_t sf_bits, size_t num_parts);
/* util/src/crt.c:596-605 Init_crtcontext, with the Q primes given */
orc_ctx* orc_ctx_create_with_primes(uint32_t degree, size_t num_q,
                                    const int64_t* q, size_t num_parts);
void     orc_ctx_destroy(orc_ctx* c);
uint32_t orc_degree(const orc_ctx* c);
size_t   orc_num_q(const orc_ctx* c);
size_t   orc_num_p(const orc_ctx* c);
size_t   orc_num_parts(const orc_ctx* c);
size_t   orc_part_size(const orc_ctx* c);
size_t   orc_num_decomp(const orc_ctx* c, size_t level);
/* prime index: 0..num_q-1 are Q primes, num_q.. are P primes */
int64_t  orc_prime(const orc_ctx* c, size_t idx);
int64_t  orc_root(const orc_ctx* c, size_t idx);
/* MODULUS fields of prime idx: out[0]=val out[1]=br_k out[2]=br_m
 * out[3]=prec128 low, out[4]=prec128 high */
void     orc_modulus(const orc_ctx* c, size_t idx, uint64_t out[5]);
/* twiddle tables of prime idx (each degree entries); which: 0 rou, 1 rou_prec,
 * 2 rou_inv, 3 rou_inv_prec */
const uint64_t* orc_twiddles(const orc_ctx* c, size_t idx, int which);
/* base-conversion tables, for table-level checks.
 *  orc_tbl_modup: hat_inv[part_len], hat[part_len * n_compl] row-major [i][j],
 *  compl_idx[n_compl] prime indices; returns n_compl, *part_len_out set */
size_t   orc_tbl_modup(const orc_ctx* c, size_t level, size_t part,
                       int64_t* hat_inv, int64_t* hat, int32_t* compl_idx,
                       size_t* part_len_out);
/*  orc_tbl_moddown: phat_inv[k], phat_modq[num_q*k] ([i][j]), pinv_modq[num_q],
 *  pmodq[num_q] */
void     orc_tbl_moddown(const orc_ctx* c, int64_t* phat_inv, int64_t* phat_modq,
                         int64_t* pinv_modq, int64_t* pmodq);
/*  orc_tbl_rescale at level (>=2): ql_inv[level-1], qlql[level-1] */
void     orc_tbl_rescale(const orc_ctx* c, size_t level, int64_t* ql_inv,
                         int64_t* qlql);

/* scalar primitives (include/util/modular.h) ------------------------------ */
int64_t  orc_add_mod(int64_t a, int64_t b, int64_t q);
int64_t  orc_sub_mod(int64_t a, int64_t b, int64_t q);
int64_t  orc_mul_mod_barrett(const orc_ctx* c, size_t idx, int64_t a, int64_t b);
uint64_t orc_precompute_const(uint64_t v, uint64_t q);
int64_t  orc_fast_mul_const(uint64_t a, uint64_t w, uint64_t w_prec, uint64_t q);
int64_t  orc_switch_modulus(int64_t v, int64_t old_q, int64_t new_q);
int64_t  orc_mod_exp(int64_t v, int64_t e, int64_t q);
int64_t  orc_mod_inv(int64_t v, int64_t m);
int      orc_is_prime(int64_t n);
int64_t  orc_find_generator(int64_t q);
int64_t  orc_root_of_unity(int64_t order, int64_t q);
void     orc_precompute_const_128(uint64_t q, uint64_t out[2]);

/* NTT: limb t (degree coefficients at dst + t*degree) uses prime prime_idx[t].
 * dst may equal src.  util/src/ntt.c:140-330 */
void orc_ntt(const orc_ctx* c, int64_t* dst, const int64_t* src,
             const int32_t* prime_idx, size_t n_limbs);
void orc_intt(const orc_ctx* c, int64_t* dst, const int64_t* src,
              const int32_t* prime_idx, size_t n_limbs);

/* per-limb vector ops, hal/src/hal.c:15-138.  n = number of coefficients */
void orc_hw_modadd(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t idx, size_t n);
void orc_hw_modsub(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t idx, size_t n);
void orc_hw_modmul(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t idx, size_t n);
void orc_hw_modmuladd(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t idx, size_t n);
void orc_hw_modadd_scalar(const orc_ctx* c, int64_t* r, const int64_t* a, int64_t s, size_t idx, size_t n);
void orc_hw_modsub_scalar(const orc_ctx* c, int64_t* r, const int64_t* a, int64_t s, size_t idx, size_t n);
void orc_hw_modmul_scalar(const orc_ctx* c, int64_t* r, const int64_t* a, int64_t s, size_t idx, size_t n);
void orc_hw_modmuladd_scalar(const orc_ctx* c, int64_t* r, const int64_t* a, int64_t s, size_t idx, size_t n);
void orc_hw_rotate(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* order, size_t idx, size_t n);

/* automorphism, util/src/number_theory.c:192-231 */
uint32_t orc_find_automorphism_index(int32_t rot_idx, uint32_t degree);
void     orc_automorphism_order(int64_t* order, uint32_t k, uint32_t degree, int is_ntt);

/* RNS polynomial ops; a polynomial at `level` with P part is level+num_p
 * contiguous limbs (Q limbs then P limbs).  poly/src/rns_poly.c */
/* :74-105 Decomp, out = digit limbs only; returns number of limbs written */
size_t orc_decomp(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level, size_t part);
/* :107-158 Mod_up: digit (coefficient or NTT form) -> level+num_p limbs */
void orc_mod_up(const orc_ctx* c, int64_t* out, const int64_t* digit, size_t digit_len, size_t level, size_t part, int is_ntt);
/* :160-258 Decomp_modup (fused) */
void orc_decomp_modup(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level, size_t part, int is_ntt);
/* :416-481 Precomp over all digits; out is num_decomp x (level+num_p) limbs */
void orc_precomp(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level, int is_ntt, int fused);
/* :260-308 Mod_down: in level+num_p limbs -> out level limbs */
void orc_mod_down(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level, int is_ntt);
/* :310-404 Rescale: in level limbs -> out level-1 limbs */
void orc_rescale(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level, int is_ntt);
/* :483-500 Extend: in level limbs -> out level+num_p limbs (P part zero) */
void orc_extend(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level);
/* Sub_mul_const_mod (include/util/modular.h:262-276) */
int64_t orc_sub_mul_const(uint64_t v1, uint64_t v2, uint64_t w, uint64_t wp, uint64_t q);
/* Mod_down_rescale (rns_poly.c:531-597): poly (level+K limbs) is converted to coefficient form in place */
void orc_mod_down_rescale(const orc_ctx* c, int64_t* out, int64_t* poly, size_t level, int is_ntt);
/* Reduce_and_rescale_modup (rns_poly_impl.c:521-620) */
void orc_reduce_rescale_modup(const orc_ctx* c, int64_t* res, int64_t* raised, int64_t* poly, size_t level, int is_ntt);
/* Transform_values_from_level0 (rns_poly.c:1101-1125) */
void orc_transform_from_level0(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level);
/* :502-529 Dot_prod / Fast_dot_prod.  digits: n_parts x (level+num_p) limbs.
 * key: n_parts polynomials of key_stride int64 each, laid out with all num_q
 * Q limbs followed by num_p P limbs; viewed at `level`. */
void orc_dot_prod(const orc_ctx* c, int64_t* out, const int64_t* digits, const int64_t* key, size_t key_stride, size_t n_parts, size_t level, int fast);
/* :852-1054 Add/Sub/Mul_poly over level Q limbs (+ num_p P limbs if with_p) */
void orc_poly_add(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p);
void orc_poly_sub(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p);
void orc_poly_mul(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p);
/* :1056-1099 Automorphism_transform */
void orc_poly_automorphism(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* order, size_t level, int with_p);

/* ciphertext level, ckks/src/evaluator.c.  A ciphertext at `level` is two
 * polynomials of level limbs.  A switch key is
 * [num_parts][2][(num_q+num_p) limbs] (b then a per digit). */
/* :142-175 Mul_ciphertext3 */
void orc_mul_ciph3(const orc_ctx* c, int64_t* d0, int64_t* d1, int64_t* d2, const int64_t* a0, const int64_t* a1, const int64_t* b0, const int64_t* b1, size_t level);
/* :411-462 Fast_switch_key on precomputed digits: out0,out1 level limbs */
void orc_fast_switch_key(const orc_ctx* c, int64_t* out0, int64_t* out1, const int64_t* digits, const int64_t* swk, size_t level);
/* :288-306 Relinearize_ciph3 */
void orc_relin(const orc_ctx* c, int64_t* r0, int64_t* r1, const int64_t* d0, const int64_t* d1, const int64_t* d2, const int64_t* swk, size_t level);
/* :342-362 Rescale_ciphertext */
void orc_rescale_ciph(const orc_ctx* c, int64_t* r0, int64_t* r1, const int64_t* c0, const int64_t* c1, size_t level);
/* :503-522 Fast_rotate with hoisted digits of c1 */
void orc_fast_rotate(const orc_ctx* c, int64_t* r0, int64_t* r1, const int64_t* c0, const int64_t* digits, const int64_t* swk, const int64_t* order, size_t level);
/* Mul_ciphertext + Rescale_ciphertext (:177-190, :342-362) */
void orc_mul_relin_rescale(const orc_ctx* c, int64_t* r0, int64_t* r1, const int64_t* a0, const int64_t* a1, const int64_t* b0, const int64_t* b1, const int64_t* swk, size_t level);

/* ---- encoder (ckks/src/encoder.c, util/src/ntt.c:598-675) ---- */
/* Embedding / Embedding_inv over `len` complex slots (re, im interleaved) */
/* the 2N (cos, sin) pairs of Precompute_fft */
const double* orc_fft_rou(const orc_ctx* c);
void orc_embedding(const orc_ctx* c, double* res, const double* coeffs, size_t len, int inverse);
/* Encode_impl (encoder.c:234-326): 1 on success, 0 where the reference asserts on range */
int orc_encode(const orc_ctx* c, int64_t* out, const double* values, size_t n_values, uint32_t slots, size_t level,
               uint32_t sf_degree, size_t p_cnt);
/* Encode_impl_with_scale (encoder.c:337-403) */
int orc_encode_scaled(const orc_ctx* c, int64_t* out, const double* values, size_t n_values, uint32_t slots,
                      size_t level, double scale, size_t p_cnt);
/* Decode (encoder.c:657-704) */
void orc_decode(const orc_ctx* c, double* res, const int64_t* poly, size_t level, uint32_t slots, double factor,
                int is_ntt);

#ifdef __cplusplus
}
#endif
#endif
