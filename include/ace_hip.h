/*
 * MI355X (gfx950) CKKS polynomial runtime -- device C-ABI.
 *
 * Plain C: opaque context handle, raw device pointers, sizes, prime indices.
 * Every polynomial is int64 limb-major (`data[limb * degree + i]`, values in
 * [0, q_limb)), exactly the reference's POLYNOMIAL::_data layout
 * (fhe-cmplr/rtlib/ant/include/poly/rns_poly.h:23-32,253-256), but resident in
 * HBM.  All calls are asynchronous on the context's HIP stream unless stated;
 * results are visible to the host after ace_sync() or a download.
 *
 * Each entry point names the reference function it replaces (paths relative
 * to fhe-cmplr/rtlib/ant).  Prime index convention: 0..num_q-1 are the Q
 * primes, num_q..num_q+num_p-1 the P (special) primes.
 *
 * Return convention: functions returning int give 0 on success, non-zero on a
 * rejected call (message via ace_last_error()); nothing is launched then.
 */
#ifndef ACE_HIP_H
#define ACE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ace_ctx ace_ctx;

/* ---- context -------------------------------------------------------------
 * Replaces Init_crtcontext_with_prime_size (util/src/crt.c:607-618): same
 * prime sequence, same 2N-th roots, same number of special primes, all NTT and
 * base-conversion tables built on the host and uploaded once. */
ace_ctx* ace_ctx_create(uint32_t degree, size_t num_q, size_t q0_bits,
                        size_t sf_bits, size_t num_parts);
/* Replaces Init_crtcontext (util/src/crt.c:596-605) with the Q primes given. */
ace_ctx* ace_ctx_create_with_primes(uint32_t degree, size_t num_q,
                                    const int64_t* q_primes, size_t num_parts);
/* Both return NULL on invalid parameters.  On a machine without a HIP device
 * the context still holds every host-side table (primes, roots, cofactors) and
 * answers the getters below, but each call that would touch the GPU is
 * rejected with an error: there is no CPU fallback. */
/* A further context over the same tables, for another host thread (the reference runs the images of a batch under
 * `#pragma omp parallel for` with the CRT context shared and the I/O, timing and generator state per thread:
 * dataset/resnet_cifar.main.inc:81-112, common/src/io_lib.c:24-27).  The new context shares the primes, twiddles and
 * conversion tables of `ctx` in HBM and has its own HIP stream, scratch arena, buffer pool and recorded calls, so
 * the two may be used from two threads at the same time; each context by itself is still used by one thread at a
 * time.  Buffers are plain device pointers: any context of the family may read and write them (the caller orders
 * uses on different contexts, e.g. with ace_sync) and ace_free accepts a buffer that a sibling's ace_alloc made.
 * The contexts made this way must be destroyed before `ctx` is.  NULL without a HIP device. */
ace_ctx*    ace_ctx_share(ace_ctx* ctx);
void        ace_ctx_destroy(ace_ctx* ctx);
int         ace_has_device(const ace_ctx* ctx);
const char* ace_last_error(void);
/* Degree / Get_q_cnt / Get_p_cnt / Get_q_parts (context/src/ckks_context.c:213-237) */
uint32_t ace_degree(const ace_ctx* ctx);
size_t   ace_num_q(const ace_ctx* ctx);
size_t   ace_num_p(const ace_ctx* ctx);
size_t   ace_num_parts(const ace_ctx* ctx);
size_t   ace_part_size(const ace_ctx* ctx);
/* Get_num_decomp (util/src/crt.c:1135-1144) */
size_t   ace_num_decomp(const ace_ctx* ctx, size_t level);
int64_t  ace_prime(const ace_ctx* ctx, size_t prime_idx);
int64_t  ace_root(const ace_ctx* ctx, size_t prime_idx);
/* MODULUS fields (include/util/modular.h:21-26): val, br_k, br_m, prec128 lo, hi */
void     ace_modulus(const ace_ctx* ctx, size_t prime_idx, uint64_t out[5]);

/* Host copies of the precomputed tables (what the kernels read from HBM), for
 * inspection and table-level parity checks.
 * ace_host_twiddles: which = 0 rou, 1 rou Shoup, 2 rou_inv, 3 rou_inv Shoup
 *   (Precompute_ntt, util/src/ntt.c:91-138), `degree` words.
 * ace_host_tbl_modup: _l_hat_inv_modq / _l_hat_modp of digit `part` at `level`
 *   (util/src/crt.c:459-566): hat_inv[n_digit], hat[n_digit][n_compl], and the
 *   prime index of each target limb in the reference's complement order.
 * ace_host_tbl_moddown: (P/p_j)^-1 mod p_j [num_p], (P/p_j) mod q_i [num_q][num_p],
 *   P^-1 mod q_i [num_q], P mod q_i [num_q] (crt.c:264-291,354-420).
 * ace_host_tbl_rescale: q_l^-1 mod q_i and the reference's second rescale
 *   constant (== -q_l^-1 mod q_i), i < level-1 (crt.c:299-349). */
int ace_host_twiddles(const ace_ctx* ctx, size_t prime_idx, int which, uint64_t* out);
/* Precompute_fft (util/src/ntt.c:559-587), fft_length 2N: rou = 2N (cos, sin) pairs, rot = N/2 powers of 5 */
int ace_host_fft_tables(const ace_ctx* ctx, double* rou, uint32_t* rot);
int ace_host_tbl_modup(const ace_ctx* ctx, size_t level, size_t part, int64_t* hat_inv, int64_t* hat,
                       int32_t* compl_idx, size_t* n_digit, size_t* n_compl);
int ace_host_tbl_moddown(const ace_ctx* ctx, int64_t* phat_inv, int64_t* phat_modq, int64_t* pinv_modq, int64_t* pmodq);
int ace_host_tbl_rescale(const ace_ctx* ctx, size_t level, int64_t* ql_inv, int64_t* neg_ql_inv);
/* Precompute_automorphism_order into host memory (`degree` words) */
int ace_host_automorphism_order(const ace_ctx* ctx, int64_t* host_order, uint32_t k, int is_ntt);

/* ---- device memory -------------------------------------------------------
 * Replaces the malloc+memset of Alloc_poly_data (include/poly/rns_poly.h:109-119):
 * zero-filled HBM, n int64 words.  ace_free keeps the buffer (up to a third of
 * the device's memory in total, or ACE_POOL_LIMIT_GB) for the next ace_alloc of
 * the same size on the same context, so alloc/free pairs inside a program's
 * loops cost a fill (recorded with the Hw_* calls around it, and dropped where
 * nothing reads the zeros), not a hipMalloc. */
int64_t* ace_alloc(ace_ctx* ctx, size_t n_words);
/* the same without the zero fill, for buffers that are written before they are read */
int64_t* ace_alloc_uninit(ace_ctx* ctx, size_t n_words);
void     ace_free(ace_ctx* ctx, int64_t* dev_ptr);
int      ace_upload(ace_ctx* ctx, int64_t* dev_dst, const int64_t* host_src, size_t n_words);
int      ace_download(ace_ctx* ctx, int64_t* host_dst, const int64_t* dev_src, size_t n_words); /* synchronises */
int      ace_copy(ace_ctx* ctx, int64_t* dev_dst, const int64_t* dev_src, size_t n_words);
int      ace_zero(ace_ctx* ctx, int64_t* dev_dst, size_t n_words);
int      ace_sync(ace_ctx* ctx);
/* Waits for every stream of the process on the context's GPU (the contexts of a family and their second lanes): for a
 * thread that is about to read what another thread's context may still be writing.  Touches no state of `ctx`. */
int      ace_sync_device(ace_ctx* ctx);
/* Two lanes.  No counterpart in the reference, whose runtime is synchronous: calls enqueue on one stream per context
 * and therefore run one after another on the GPU, although a single polynomial's kernels do not fill the machine.
 * Where a program has two independent pieces of work (the two sine evaluations of a fully packed bootstrap):
 *   ace_fork(ctx);         the calls that follow are issued on a second stream, which first waits for everything
 *                          issued so far;
 *   ace_fork_switch(ctx);  back to the first stream: the calls that follow may run at the same time as those issued
 *                          since ace_fork;
 *   ace_join(ctx);         the first stream waits for the second (ace_join straight after ace_fork works too).
 * Between ace_fork and ace_join the two sequences must not touch each other's buffers (what either reads may have
 * been written before the fork); results are those of issuing both sequences one after the other.  Buffers may be
 * allocated and freed on either lane. */
int      ace_fork(ace_ctx* ctx);
int      ace_fork_switch(ace_ctx* ctx);
int      ace_join(ace_ctx* ctx);
/* Gives back the second stream with its scratch arena and kept buffers (made by the first ace_fork; the next
 * ace_fork makes them again).  For a program that goes on with several contexts of a family on several threads:
 * the hardware serves a process's streams through a few queues, and a stream that is no longer used still holds
 * its place among them.  Rejected between ace_fork and ace_join. */
int      ace_fork_release(ace_ctx* ctx);
/* Device memory the context holds right now, in 64-bit words and buffers (no counterpart in the reference; for
 * tests that check that a call allocates nothing): out[0] = scratch arena of the current lane, out[1] = freed
 * buffers kept for reuse (words), out[2] = buffers handed out by ace_alloc and not yet freed, out[3] = freed buffers
 * kept for reuse (count). */
void     ace_memory_stats(const ace_ctx* ctx, size_t out[4]);
/* With ACE_HIP_CENSUS=<file> in the environment the library counts the calls of its entry points by size and writes
 * "<entry point> <level or limbs> <second size> <calls>" lines to <file> when the process ends (no counterpart in
 * the reference; the counts feed cost models of a whole program, such as the benchmark's estimate of the
 * reference's CPU time).  ace_census_mark writes the counts so far to <file>.<label> and starts again from zero, so
 * that a program's phases (key generation, images) can be told apart.  Without the variable: nothing. */
void     ace_census_mark(const char* label);
/* HIP-event stopwatch on the context's stream (for benchmarks) */
int      ace_timer_start(ace_ctx* ctx);
float    ace_timer_stop_ms(ace_ctx* ctx); /* synchronises; <0 on error */

/* ---- NTT -----------------------------------------------------------------
 * Replaces Ftt_fwd / Ftt_inv (util/src/ntt.c:140-164) as driven by
 * Conv_poly2ntt(_inplace)(_with_primes), Conv_ntt2poly* (poly/src/rns_poly.c:
 * 608-699, rns_poly_impl.c:164-285) and Hw_ntt / Hw_intt (hal/src/hal.c:140-153).
 * Polynomial p (0..n_polys-1) limb t (0..n_limbs-1) lives at
 * base + (p*poly_stride_limbs + t)*degree and uses prime prime_idx[t].
 * Forward: natural order in, bit-reversed out.  Inverse: the opposite, 1/N
 * included.  dst may equal src; otherwise the two must not overlap (polynomials of a batch are transformed in any
 * order, several at a time). */
int ace_ntt(ace_ctx* ctx, int64_t* dst, const int64_t* src, const int32_t* prime_idx,
            size_t n_limbs, size_t n_polys, size_t poly_stride_limbs);
int ace_intt(ace_ctx* ctx, int64_t* dst, const int64_t* src, const int32_t* prime_idx,
             size_t n_limbs, size_t n_polys, size_t poly_stride_limbs);

/* One of the two kernels a transform consists of when degree > 4096 (pass 1 then
 * pass 2 equals ace_ntt / ace_intt).  For profiling each kernel on its own; the
 * intermediate buffer holds lazily reduced values.  Both passes of a transform must be
 * called with the same n_limbs and n_polys: how the stages are divided between the two
 * kernels depends on the size of the launch (n_limbs * n_polys >= 192 moves one stage
 * of the inverse transform from pass 1 to pass 2), so passes issued with different
 * shapes run that stage twice or not at all. */
int ace_ntt_pass(ace_ctx* ctx, int64_t* dst, const int64_t* src, const int32_t* prime_idx,
                 size_t n_limbs, size_t n_polys, size_t poly_stride_limbs, int inverse, int pass);

/* ---- per-limb vector ops: Hw_* (hal/src/hal.c:15-138) ----------------------
 * n coefficients with the modulus of prime_idx. */
int ace_hw_modadd(ace_ctx* ctx, int64_t* res, const int64_t* a, const int64_t* b, size_t prime_idx, size_t n);
int ace_hw_modsub(ace_ctx* ctx, int64_t* res, const int64_t* a, const int64_t* b, size_t prime_idx, size_t n);
int ace_hw_modmul(ace_ctx* ctx, int64_t* res, const int64_t* a, const int64_t* b, size_t prime_idx, size_t n);
int ace_hw_modmuladd(ace_ctx* ctx, int64_t* res, const int64_t* a, const int64_t* b, size_t prime_idx, size_t n);
int ace_hw_modadd_scalar(ace_ctx* ctx, int64_t* res, const int64_t* a, int64_t s, size_t prime_idx, size_t n);
int ace_hw_modsub_scalar(ace_ctx* ctx, int64_t* res, const int64_t* a, int64_t s, size_t prime_idx, size_t n);
int ace_hw_modmul_scalar(ace_ctx* ctx, int64_t* res, const int64_t* a, int64_t s, size_t prime_idx, size_t n);
int ace_hw_modmuladd_scalar(ace_ctx* ctx, int64_t* res, const int64_t* a, int64_t s, size_t prime_idx, size_t n);
/* Consecutive ace_hw_* calls are recorded and launched together (one kernel for a run of calls instead of one
 * each: generated code issues them limb by limb); every other entry point launches what is pending first, so
 * results are those of issuing the calls one by one.  ace_set_batching(ctx, 0) launches each call on its own. */
int ace_set_batching(ace_ctx* ctx, int on);
/* Hw_rotate: res[i] = order[i] >= 0 ? a[order[i]] : q - a[-order[i]]; order is a device table */
int ace_hw_rotate(ace_ctx* ctx, int64_t* res, const int64_t* a, const int64_t* order, size_t prime_idx, size_t n);

/* ---- automorphism tables (util/src/number_theory.c:192-231) ---------------- */
uint32_t ace_find_automorphism_index(const ace_ctx* ctx, int32_t rot_idx);
/* Precompute_automorphism_order into a device table of `degree` words */
int ace_automorphism_order(ace_ctx* ctx, int64_t* dev_order, uint32_t k, int is_ntt);

/* ---- RNS polynomial ops (poly/src/rns_poly.c) -------------------------------
 * A polynomial "at level l" is l Q limbs; "extended" adds the num_p P limbs
 * right after them (l + num_p contiguous limbs). */
/* Add_poly / Sub_poly / Mul_poly (:852-1010), Automorphism_transform (:1056-1099) */
int ace_poly_add(ace_ctx* ctx, int64_t* res, const int64_t* a, const int64_t* b, size_t level, int with_p);
int ace_poly_sub(ace_ctx* ctx, int64_t* res, const int64_t* a, const int64_t* b, size_t level, int with_p);
int ace_poly_mul(ace_ctx* ctx, int64_t* res, const int64_t* a, const int64_t* b, size_t level, int with_p);
int ace_poly_automorphism(ace_ctx* ctx, int64_t* res, const int64_t* a, const int64_t* order, size_t level, int with_p);
/* Scalars_integer_add_poly / Scalars_integer_multiply_poly (poly/src/rns_poly.c; Add_scalars, Mul_scalars,
 * evaluator.c:113-125,218-235): limb t of res = limb t of a plus / times scalars[t] (a HOST array of `level`
 * residues).  res may equal a. */
int ace_poly_add_scalars(ace_ctx* ctx, int64_t* res, const int64_t* a, const int64_t* scalars, size_t level);
int ace_poly_mul_scalars(ace_ctx* ctx, int64_t* res, const int64_t* a, const int64_t* scalars, size_t level);
/* Eval_linear_wsum (ckks/src/chebyshev_impl.c:276-318) without its rescale: (r0, r1) = sum_j weights[j] *
 * (a0[j], a1[j]) at `level`; weights is a HOST array of count x level residues (the encoded constants of
 * Mul_const), a0/a1 host arrays of `count` (<= 32) device pointers.  The result may alias an operand. */
int ace_ciph_wsum(ace_ctx* ctx, int64_t* r0, int64_t* r1, const int64_t* const* a0, const int64_t* const* a1,
                  const int64_t* weights, size_t count, size_t level);
/* Key-generation helpers (the polynomials of ckks/src/key_gen.c:127-200 are drawn limb by limb on the host in the
 * reference; its generator cannot be reproduced, so these have no bit-level counterpart).
 * ace_sample_uniform: level Q limbs (+ the P limbs) of residues uniform on [0, q_t), a pure function of
 *   (seed, stream, limb, position) through a 64-bit mixing hash: reproducible, NOT a cryptographic generator.
 * ace_expand_small: a HOST array of N small signed coefficients (|v| <= 2^30) as residues of every limb. */
int ace_sample_uniform(ace_ctx* ctx, int64_t* res, size_t level, int with_p, uint64_t seed, uint64_t stream);
int ace_expand_small(ace_ctx* ctx, int64_t* res, const int64_t* small_host, size_t level, int with_p);
/* The inner sum of a baby-step group of the bootstrap's linear transforms (Mul_plaintext + Add_ciphertext,
 * ckks/src/bootstrap.c:1291-1311): (r0, r1) = sum_j (a0[j], a1[j]) * plain[j], or += when `accumulate`.
 * Operands and result are extended polynomials at `level`; a plaintext holds plain_level >= level Q limbs
 * before its P limbs (Derive_plain, include/ckks/plaintext.h:107-114).  a0/a1/plain: host arrays of `count`
 * device pointers; no operand may alias the result. */
int ace_ext_plain_mac(ace_ctx* ctx, int64_t* r0, int64_t* r1, const int64_t* const* a0, const int64_t* const* a1,
                      const int64_t* const* plain, size_t count, size_t level, size_t plain_level, int accumulate);
/* The same for n_groups baby-step groups over the same operands: (r0[g], r1[g]) = sum_j (a0[j], a1[j]) *
 * plain[g * count + j]; a NULL plaintext means group g has no term j.  The operands are read once for up to four
 * groups.  No result may share a buffer with an operand or with another result. */
int ace_ext_plain_mac_groups(ace_ctx* ctx, int64_t* const* r0, int64_t* const* r1, size_t n_groups,
                             const int64_t* const* a0, const int64_t* const* a1, size_t count,
                             const int64_t* const* plain, size_t level, size_t plain_level);
/* Decomp_modup (:160-258) (== Decomp :74-105 + Mod_up :107-158): digit `part`
 * of src (level limbs) raised to level+num_p limbs. */
int ace_decomp_modup(ace_ctx* ctx, int64_t* res, const int64_t* src, size_t level, size_t part, int is_ntt);
/* Mod_up (:107-158) alone: `digit` holds only the limbs of digit `part` (what
 * Decomp :74-105 produced), res as for ace_decomp_modup. */
int ace_mod_up(ace_ctx* ctx, int64_t* res, const int64_t* digit, size_t level, size_t part, int is_ntt);
/* Precomp / Alloc_precomp (:416-481): all digits, res = num_decomp x (level+num_p) limbs */
int ace_precomp(ace_ctx* ctx, int64_t* res, const int64_t* src, size_t level, int is_ntt);
/* Mod_down (:260-308): src level+num_p limbs -> res level limbs */
int ace_mod_down(ace_ctx* ctx, int64_t* res, const int64_t* src, size_t level, int is_ntt);
/* Precomp (:416-481) / Mod_down (:260-308) of `count` polynomials in one set of launches: polynomial o is read at
 * src + o * src_stride and written at res + o * res_stride (strides in words, at least the size of one operand /
 * result; results and operands must not overlap).  The words are those of `count` single calls; the batch exists
 * because one polynomial's kernels leave most of the machine idle (the rotated inner sums of a bootstrap level). */
int ace_precomp_batch(ace_ctx* ctx, int64_t* res, size_t res_stride, const int64_t* src, size_t src_stride,
                      size_t count, size_t level, int is_ntt);
int ace_mod_down_batch(ace_ctx* ctx, int64_t* res, size_t res_stride, const int64_t* src, size_t src_stride,
                       size_t count, size_t level, int is_ntt);
/* Mod_down for callers that cannot allocate device memory (tight serving loops, harnesses that forbid hipMalloc,
 * code that prepares a HIP graph -- capture itself is not exercised by this library's tests).  No counterpart in the reference.  Same operands and result as ace_mod_down;
 * the intermediates live in a 16 MiB device array that is part of the library image (one copy per GPU, held until
 * the process ends), so the call performs no hipMalloc / hipFree and takes nothing from the context's arena.
 * Rejected when (level + num_p) * degree exceeds 2^21 words, and while more than 96 recorded ace_hw_* calls or a
 * paired Mod_down / Rescale are pending (their launch may allocate: ace_sync first; up to 96 recorded calls are
 * launched first, as kernel arguments).  Every call on one GPU shares that array: calls that overlap in time on one GPU (two
 * contexts, two streams) race; calls on one context are ordered by its stream, and the call is rejected between
 * ace_fork and ace_join, when the context issues on two streams.  Nothing in the array needs to
 * start at zero: each call writes every word it later reads. */
int ace_mod_down_noalloc(ace_ctx* ctx, int64_t* res, const int64_t* src, size_t level, int is_ntt);
/* Rescale (:310-404): src level limbs -> res level-1 limbs */
int ace_rescale(ace_ctx* ctx, int64_t* res, const int64_t* src, size_t level, int is_ntt);
/* Mod_down_rescale (:531-597): Mod_down and rescale in one pass over the coefficient
 * form.  `poly` (level + num_p limbs) is converted to coefficient form IN PLACE, as the
 * reference does to its argument; res receives level-1 limbs in NTT form. */
int ace_mod_down_rescale(ace_ctx* ctx, int64_t* res, int64_t* poly, size_t level, int is_ntt);
/* Reduce_and_rescale_modup (poly/src/rns_poly_impl.c:521-620): the same value, left in
 * coefficient form and raised digit by digit: `raised` = num_decomp(level-1) polynomials of
 * (level-1 + num_p) limbs, coefficient form.  `res` (level limbs) is left as the reference
 * leaves it: the converted P part in limbs 0..level-2, the reduced last limb in limb level-1.
 * `poly` is converted to coefficient form in place. */
int ace_reduce_rescale_modup(ace_ctx* ctx, int64_t* res, int64_t* raised, int64_t* poly, size_t level, int is_ntt);
/* Transform_values_from_level0 (:1101-1125): limb 0 of src copied, limb i of res =
 * Switch_modulus(limb 0, q_0 -> q_i), i < level. */
int ace_transform_from_level0(ace_ctx* ctx, int64_t* res, const int64_t* src, size_t level);
/* Embedding_inv (util/src/ntt.c:631-675) on `len` complex numbers, host to host through the device */
int ace_embedding_inv(ace_ctx* ctx, double* host_out, const double* host_in, size_t len);
/* Decode (ckks/src/encoder.c:657-704): the message of a plaintext polynomial at `level` (NTT or coefficient form,
 * left unchanged): Reconstruct (util/src/crt.c:1247-1275) of the coefficients the slots use to centred integers, their
 * conversion to double as mpz_get_d truncates, division by `factor` (the plaintext's scale) and Embedding
 * (util/src/ntt.c:598-629), all on the device.  host_out receives `slots` complex numbers (re, im interleaved);
 * slots = 0 means N/2.  Synchronises.  At most 64 limbs. */
int ace_decode(ace_ctx* ctx, double* host_out, const int64_t* poly, size_t level, int is_ntt, uint32_t slots,
               double factor);
/* Encode_impl (ckks/src/encoder.c:234-326; Encode_at_level_with_sf, Encode_ext_at_level): `values` is a
 * HOST array of n_values complex numbers (re, im interleaved), zero-padded to `slots` (0: N/2); the
 * plaintext polynomial lands in res: level (0: all) Q limbs followed by p_cnt (0 or num_p) P limbs, NTT
 * form, scale 2^(sf_bits * sf_degree).  The inverse embedding, rounding and residues are computed on the
 * device with the reference's floating-point operations in the reference's order.  Where the
 * reference asserts on a value out of range for the level, a flag is raised inside the kernel and
 * reported by the next ace_sync / ace_download. */
int ace_encode(ace_ctx* ctx, int64_t* res, const double* values, size_t n_values, uint32_t slots, size_t level,
               uint32_t sf_degree, size_t p_cnt);
/* The same for real-valued messages (Encode_float / Encode_double, ckks/src/plain.c:29-63, and the weight
 * plaintexts of Pt_from_msg, pt_mgr.c): `values` is a HOST array of n_values doubles (is_f32 = 0) or floats
 * (is_f32 = 1), widened to complex numbers with zero imaginary part on the device. */
int ace_encode_real(ace_ctx* ctx, int64_t* res, const void* values, int is_f32, size_t n_values, uint32_t slots,
                    size_t level, uint32_t sf_degree, size_t p_cnt);
/* The same for `n_vec` vectors of `n_values` values each (values[v] points to vector v) in one set of launches:
 * vector v is encoded into res + v * res_stride words, bit for bit as ace_encode_real would.  For weight files, whose
 * entries a program asks for one after the other. */
int ace_encode_real_batch(ace_ctx* ctx, int64_t* res, size_t res_stride, const void* const* values, int is_f32,
                          size_t n_values, size_t n_vec, uint32_t slots, size_t level, uint32_t sf_degree,
                          size_t p_cnt);
/* Encode_at_level_with_scale (ckks/src/encoder.c:337-420): complex values at an explicit scale (any positive
 * double below the level's modulus): one multiplication by `scale`, rounded to nearest. */
int ace_encode_scaled(ace_ctx* ctx, int64_t* res, const double* values, size_t n_values, uint32_t slots, size_t level,
                      double scale, size_t p_cnt);
/* Extend (:483-500): src level limbs -> res level+num_p limbs (P limbs zero) */
int ace_extend(ace_ctx* ctx, int64_t* res, const int64_t* src, size_t level);
/* Dot_prod / Fast_dot_prod (:502-529): digits = n_parts x (level+num_p) limbs;
 * key = n_parts polynomials, key_stride words apart, each laid out as all num_q
 * Q limbs followed by num_p P limbs and viewed at `level` (Derive_poly :701-707).
 * Digits and key words must be residues (below the prime of their limb), as everything the library writes is: the
 * products are summed in 128 bits and reduced once, which relies on that bound. */
int ace_dot_prod(ace_ctx* ctx, int64_t* res, const int64_t* digits, const int64_t* key,
                 size_t key_stride, size_t n_parts, size_t level);
/* Fast_rotate_ext without its Mod_down (evaluator.c:503-566, as Rotate_iteration of bootstrap.c:1233-1373 uses it):
 * out0 = sigma(sum_d digit_d * key_d.b + addend0), out1 = sigma(sum_d digit_d * key_d.a), level + num_p limbs each,
 * NTT form; sigma is the automorphism given by `order` (ace_automorphism_order, NTT form).  key points at digit 0's b
 * half, its a half lies key_half_words further, digit d's pair key_stride words further; addend0 may be NULL.
 * accumulate: bit 0 adds the first result to what out0 holds, bit 1 the second to out1 (the running sums of the
 * giant steps).  The results must not overlap the operands. */
int ace_ext_rotate(ace_ctx* ctx, int64_t* out0, int64_t* out1, const int64_t* digits, const int64_t* key,
                   size_t key_half_words, size_t key_stride, size_t n_parts, const int64_t* addend0,
                   const int64_t* order, size_t level, int accumulate);

/* ---- ciphertext level (ckks/src/evaluator.c, ckks/src/cipher.c) ------------
 * A ciphertext at level l is two polynomials (c0, c1) of l limbs.  A switch
 * key is [num_parts][2][(num_q+num_p) limbs]: per digit the b polynomial then
 * the a polynomial (include/ckks/switch_key.h:27-29, public_key.h:24-27). */
/* Mul_ciphertext3 (evaluator.c:142-175) */
int ace_mul_ciph3(ace_ctx* ctx, int64_t* d0, int64_t* d1, int64_t* d2, const int64_t* a0, const int64_t* a1,
                  const int64_t* b0, const int64_t* b1, size_t level);
/* Fast_switch_key (evaluator.c:411-462) on hoisted digits: out0/out1 level limbs */
int ace_fast_switch_key(ace_ctx* ctx, int64_t* out0, int64_t* out1, const int64_t* digits, const int64_t* swk, size_t level);
/* Relinearize_ciph3 (evaluator.c:288-306) */
int ace_relin(ace_ctx* ctx, int64_t* r0, int64_t* r1, const int64_t* d0, const int64_t* d1, const int64_t* d2,
              const int64_t* swk, size_t level);
/* Rescale_ciphertext (evaluator.c:342-362): level -> level-1 limbs */
int ace_rescale_ciph(ace_ctx* ctx, int64_t* r0, int64_t* r1, const int64_t* c0, const int64_t* c1, size_t level);
/* Mul_ciphertext + Rescale_ciphertext (evaluator.c:177-190, 342-362): r0/r1 level-1 limbs */
int ace_mul_relin_rescale(ace_ctx* ctx, int64_t* r0, int64_t* r1, const int64_t* a0, const int64_t* a1,
                          const int64_t* b0, const int64_t* b1, const int64_t* swk, size_t level);
/* Mod_down (rns_poly.c:260-308) of two polynomials of the extended basis (level + num_p limbs, NTT form) followed by
 * Rescale (rns_poly.c:310-404) of both: what ends a linear transform carried out in the extended basis when a
 * Rescale_ciphertext follows.  r0/r1: level - 1 limbs, apart from the operands and from each other.  The words of
 * ace_mod_down twice and ace_rescale_ciph. */
int ace_mod_down_pair_rescale(ace_ctx* ctx, int64_t* r0, int64_t* r1, const int64_t* e0, const int64_t* e1, size_t level);
/* Mul_ciphertext, Add_ciphertext of the product with itself, Rescale_ciphertext (evaluator.c:177-190, 47-76, 342-362):
 * 2ab one level down, the step of the Chebyshev product rule as Eval_chebyshev_ps issues it
 * (chebyshev_impl.c:563-565, 581-583, 597-599).  The words of the three calls one after the other. */
int ace_mul_relin_double_rescale(ace_ctx* ctx, int64_t* r0, int64_t* r1, const int64_t* a0, const int64_t* a1,
                                 const int64_t* b0, const int64_t* b1, const int64_t* swk, size_t level);
/* Mul_ciphertext, Add_ciphertext(prod, prod), Add_const and Rescale_ciphertext (evaluator.c:177-190, 47-76, 127-140
 * with Add_scalars :113-124, 342-362): a double-angle step of the bootstrap's sine
 * evaluation (bootstrap.c:1504-1516).  constant: host array of `level` residues, one per limb, of the integer that is
 * added to every word of c0 (NTT form) between the sum and the Rescale.  r0/r1 level-1 limbs.  The words of
 * ace_mul_ciph3, ace_relin, two elementwise sums, ace_poly_add_scalars and ace_rescale_ciph. */
int ace_mul_relin_double_add_rescale(ace_ctx* ctx, int64_t* r0, int64_t* r1, const int64_t* a0, const int64_t* a1,
                                     const int64_t* b0, const int64_t* b1, const int64_t* swk, const int64_t* constant,
                                     size_t level);
/* ace_mul_relin_rescale for `count` independent ciphertext pairs that share the relinearisation key: pair i reads
 * a0 + i*in_stride (likewise a1, b0, b1) and writes r0 + i*out_stride, r1 + i*out_stride (strides in
 * words).  Equivalent to `count` calls of ace_mul_relin_rescale; every kernel launch covers the batch. */
int ace_mul_relin_rescale_batch(ace_ctx* ctx, int64_t* r0, int64_t* r1, size_t out_stride, const int64_t* a0,
                                const int64_t* a1, const int64_t* b0, const int64_t* b1, size_t in_stride,
                                const int64_t* swk, size_t level, size_t count);
/* Fast_rotate (evaluator.c:503-522) with the digits of c1 hoisted (Alloc_precomp).
 * order: a device table of `degree` entries, result[i] = value at order[i] (what Auto_order hands out; made by
 * ace_automorphism_order or uploaded by the caller).  Tables of Precompute_automorphism_order's NTT form
 * (number_theory.c:211-222) are applied inside the last kernel of the Mod_down transform; any other table
 * (examined on the device the first time a rotation uses it, one stream synchronisation) goes through a separate
 * pass and gives the same words more slowly.  A table must not be rewritten other than through ace_upload,
 * ace_copy, ace_zero, ace_free or ace_automorphism_order while the context is alive.
 * r0 and r1 must not overlap c0, the digits or each other: the result is permuted on the way out. */
int ace_fast_rotate(ace_ctx* ctx, int64_t* r0, int64_t* r1, const int64_t* c0, const int64_t* digits,
                    const int64_t* swk, const int64_t* order, size_t level);
/* Rotate_batch_ciph (cipher.c:459-479): one ModUp of c1, then `count` rotations.
 * r0s/r1s: count x level limbs; swks/orders: host arrays of `count` device pointers (tables as for
 * ace_fast_rotate).  The result slabs must not overlap c0 or each other (c1 is consumed before they are written). */
int ace_rotate_batch(ace_ctx* ctx, int64_t* r0s, int64_t* r1s, const int64_t* c0, const int64_t* c1,
                     const int64_t* const* swks, const int64_t* const* orders, size_t count, size_t level);

#ifdef __cplusplus
}
#endif
#endif /* ACE_HIP_H */
