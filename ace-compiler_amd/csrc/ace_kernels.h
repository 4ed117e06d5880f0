// Launchers of the gfx950 kernels (definitions in ace_ntt.hip, ace_poly.hip).
// Every launcher enqueues on the given stream and returns immediately.
#pragma once
#include "ace_device.h"

namespace ace {

enum EwOp { EW_ADD, EW_SUB, EW_MUL, EW_MULADD, EW_ADD_S, EW_SUB_S, EW_MUL_S, EW_MULADD_S };

constexpr int kMaxConvJobs = 4;   // digits converted per base-conversion launch
// (kMaxBatchPtrs, the number of keys / index tables per batched launch, and OrderSet live in ace_device.h)

// one digit's base conversion: out[map.out_limb[j]][i] = (sum_k t[k][i] * hat[k*hat_stride + j]) mod prime map.prime[j]
// Targets below kFpConvTargetLimit take the conversion in exact double arithmetic when the job has tables (fw):
// a source word is cut into three 21-bit pieces, row 3k+i of fw belongs to piece i of source k:
// fw: [3 nd][fw_stride][2] = the halves above and below bit 26 of hat * 2^(21 i) mod m_j as doubles (plus a margin of
//     four entries); fq: [nc][2] = (m_j, 1 / m_j);
// fp_target[j] says whether target j uses them.
// mx: operands of the conversion on the matrix cores (null: not available for this job), [quad][kMxSteps][64 lanes]
//     of 16 bytes each, a quad being four consecutive targets and a step four source limbs; mt: [4 quads] for each
//     target its modulus, the reciprocal as a double and the word offset of its limb in the output polynomial.
constexpr u32 kMxSteps = 4;
struct ConvTarget {
  u64 m;
  double minv;
  u64 out_off;
  u64 pad;
};
struct ConvJob {
  const u64* hat;
  u32 hat_stride, nd, nc;
  const uint4* mx;
  const ConvTarget* mt;
  u64 t_off, out_off;  // word offsets of this job's source limbs / output polynomial inside one operand
  ConvMap map;
  const double* fw;
  const double* fq;
  u32 fw_stride;
  uint8_t fp_target[kMaxPrimes];
};
struct ConvBatch {
  ConvJob job[kMaxConvJobs];
  u32 n_jobs;
  u32 matrix;                // take the matrix-core kernel where the jobs have its tables
  u64 t_stride, out_stride;  // word strides between operands
};
struct KeySet {   // one switch key per operand, or one shared by all (n == 1)
  const u64* p[kMaxBatchPtrs];
  u32 n;
};

// NTT / INTT over n_polys x n_limbs limbs; polynomial p of dst/src is seq.at(p),
// limb t sits pos[t] limbs into it (t itself when pos is null).
// scale: optional device array of 2*n_limbs words (constant, Shoup companion)
// replacing 1/N in the inverse.
// passes: for N > 4096 the transform is two kernels; bit 0 / bit 1 select them
// (both by default; single passes exist so a benchmark can time each kernel).
// fuse: optional prologue / epilogue of a whole forward transform of N > 4096 (FwdFuse); with an epilogue dst
// only holds the intermediate between the two kernels.  Returns false when the request cannot be served.
// times: the inverse transform of the limb-wise product src * times (canonical words, modulo each limb's prime)
// instead of src; served only by the kernel for large launches of FP64-capable limbs at N > 4096 -- false, and
// nothing launched, otherwise (the caller then forms the product itself).
bool launch_ntt(hipStream_t st, const DevCtx& c, const PolySeq& dst, const PolySeq& src, const LimbMap& lm,
                const LimbMap* pos, u32 n_limbs, u32 n_polys, bool inverse, const u64* scale, int passes = 3,
                const FwdFuse* fuse = nullptr, const CopyThrough* copy_src_to = nullptr,
                const PolySeq* times = nullptr);

constexpr u32 kMaxMacOps = 32;
struct MacSet { // operands of one multiply-accumulate launch
  const u64* a0[kMaxMacOps];
  const u64* a1[kMaxMacOps];
  const u64* p[kMaxMacOps];
  u32 n;
};
// (r0, r1) (+)= sum_j (a0_j, a1_j) * p_j over n_limbs limbs; limb t of p_j sits at limb t below `level`,
// at plain_level + (t - level) above it
void launch_plain_mac(hipStream_t st, const DevCtx& c, u64* r0, u64* r1, const MacSet& ops, const LimbMap& lm,
                      u32 n_limbs, u32 level, u32 plain_level, bool accumulate, u64 n);
// The same for up to kMacGroups groups that share the operands (a0_j, a1_j) and differ in their plaintexts: the
// operands, two thirds of the traffic of a single group, are read once.  p[g][j] == nullptr: group g has no term j.
constexpr int kMacGroups = 4, kMacGroupOps = 16;
struct MacGroups {
  u64* r0[kMacGroups];
  u64* r1[kMacGroups];
  const u64* a0[kMacGroupOps];
  const u64* a1[kMacGroupOps];
  const u64* p[kMacGroups][kMacGroupOps];
  u32 n_groups, n_ops;
};
void launch_plain_mac_groups(hipStream_t st, const DevCtx& c, const MacGroups& ops, const LimbMap& lm, u32 n_limbs,
                             u32 level, u32 plain_level, bool accumulate, u64 n);
// a run of Hw_* calls executed as one launch: thread i carries out every entry for element i, in order
enum BatchKind : u32 { BATCH_ROTATE = 100, BATCH_COPY = 101, BATCH_ZERO = 102 };
// flag on BatchOp::op: the result is handed to the next entry of the chain in a register and overwritten later in
// the run, so it need not be stored (the scratch limb between an Hw_modmul and the Hw_modadd that consumes it)
constexpr u32 kBatchDeadStore = 0x80000000u;
struct BatchOp {
  u64* r;
  const u64* a;
  const u64* b;  // second operand, or the index table of a rotate
  u64 scalar;
  u32 op;        // an EwOp, or BATCH_ROTATE
  u32 prime;
};
// an entry as the kernels read it: b is the second operand, the index table of a rotate, or the scalar
struct BatchOpDev {
  u64* r;
  const u64* a;
  u64 b;
  u32 op, prime;
};
constexpr u32 kSmallRun = 96;  // runs up to this many entries travel as kernel arguments (3.3 KB), no copy
struct SmallRun {
  BatchOpDev ops[kSmallRun];
  uint16_t chain_start[kSmallRun + 1];
};
void launch_ew_batch_small(hipStream_t st, const DevCtx& c, const SmallRun& run, u32 n_chains, u64 n, bool pairs);
// chain y (blockIdx.y) is the entries [chain_start[y], chain_start[y+1]): chains share no written range, so they run side by side
void launch_ew_batch(hipStream_t st, const DevCtx& c, const BatchOpDev* dev_ops, const u32* dev_chain_start, u32 n_chains,
                     u64 n, bool pairs);
void launch_sample_uniform(hipStream_t st, const DevCtx& c, u64* r, u64 seed, u64 stream, const LimbMap& lm,
                           u32 n_limbs, u64 n);
void launch_expand_small(hipStream_t st, const DevCtx& c, u64* r, const i64* v, const LimbMap& lm, u32 n_limbs, u64 n);
struct LimbScalars { // one residue per limb
  u64 v[kMaxPrimes];
};
// r[t] = a[t] + s.v[t] (mul == false) or a[t] * s.v[t] (mul == true) modulo prime lm.prime[t]
void launch_limb_scalars(hipStream_t st, const DevCtx& c, bool mul, u64* r, const u64* a, const LimbScalars& s,
                         const LimbMap& lm, u32 n_limbs, u64 n);
// (r0, r1) = sum_j w[j*n_limbs + t] * (a0_j, a1_j)[t]; w is a device array
void launch_wsum(hipStream_t st, const DevCtx& c, u64* r0, u64* r1, const MacSet& ops, const u64* w,
                 const LimbMap& lm, u32 n_limbs, u64 n);
// elementwise over n_limbs limbs of n words each (limb t uses lm.prime[t]);
// scalar ops take the same scalar for every limb.
void launch_ew(hipStream_t st, const DevCtx& c, EwOp op, u64* r, const u64* a, const u64* b, u64 scalar,
               const LimbMap& lm, u32 n_limbs, u64 n);
// r[t][i] = order[i] >= 0 ? a[t][order[i]] : q_t - a[t][-order[i]]
void launch_gather(hipStream_t st, const DevCtx& c, u64* r, const u64* a, const i64* order, const LimbMap& lm,
                   u32 n_limbs, u64 n);
// n_rot rotations: rotation z gathers (a0,a1) + z*a_stride into (r0,r1) + z*r_stride with table orders.p[z]
void launch_gather2(hipStream_t st, const DevCtx& c, u64* r0, u64* r1, u64 r_stride, const u64* a0, const u64* a1,
                    u64 a_stride, const OrderSet& orders, const LimbMap& lm, u32 n_limbs, u32 n_rot);
// tensor product of n_ops ciphertext pairs: d0 = a0*b0, d1 = a0*b1 + a1*b0, d2 = a1*b1; d0 == null: d2 only
void launch_tensor(hipStream_t st, const DevCtx& c, u64* d0, u64* d1, u64* d2, const u64* a0, const u64* a1,
                   const u64* b0, const u64* b1, const LimbMap& lm, u32 n_limbs, u32 n_ops, u64 d01_stride,
                   u64 d2_stride, u64 in_stride);
// fast base conversion of b.n_jobs digits for each of n_ops operands
void launch_baseconv(hipStream_t st, const DevCtx& c, u64* out, const u64* t, const ConvBatch& b, u32 n_ops);
// The same conversion followed, in the same kernel, by the strided pass of the forward transform of every converted
// limb (in place where the conversion would have put it): the caller then runs launch_ntt with passes = 2.  Returns
// false, having launched nothing, where the two kernels serve better or the shape is not covered (N != 2^16, more
// than eight source limbs, a job without matrix tables, a launch too small to fill the machine).
// rescale: the FwdFuse of a transform whose prologue is pro 2 (a Mod_down and a Rescale sharing it): the prologue is
// then carried out here as well, on the conversion's last target (`ylast`, which stays out of the transform).
bool launch_baseconv_fwd_strided(hipStream_t st, const DevCtx& c, u64* out, const u64* t, const ConvBatch& b, u32 n_ops,
                                 const FwdFuse* rescale = nullptr);
// digit limbs of src copied into the raised polynomials (see digit_copy_kernel)
void launch_digit_copy(hipStream_t st, const DevCtx& c, u64* res, const u64* src, u32 level, u32 part_size,
                       u32 n_digits, u64 digit_stride, u64 res_stride, u64 src_stride, u32 n_ops);
// inner product with a switch key for n_ops operands: out0/out1 (n_limbs limbs, out_stride apart) =
// sum_d digits[op][d] * key[d][0/1]; key limb of launch limb t is key_limb[t]; out1 may be null.
// Where the raised digits do not hold the digits' own limbs (the Q limbs of the polynomial that was decomposed,
// which Mod_up only passes through): limb t < level of digit t / part_size is read from src + op * op_stride + t * N.
struct OwnLimbs {
  const u64* src;  // null with `product`: the own limbs are Lift's a1 * b1, formed where they are used
  u64 op_stride;
  u32 part_size, level;
  u32 product;
};
// An addend lifted to the extended basis on the way out (what Extend, rns_poly.c:483-500, would add before a
// Mod_down): limb t < level of operand op's results gains addend.at(2 op) [t] * cst[2t] and addend.at(2 op + 1) [t] *
// cst[2t] (cst: P mod q_t and its Shoup companion).  The Mod_down of such a sum is Mod_down(sum) + addend.
// With a0 set the addend is the tensor product of operand op's ciphertexts, formed on the way instead of being read:
// (a0 b0, a0 b1 + a1 b0) at a0 + op * in_stride etc. (only the kernel that shares one key among the operands).
struct Lift {
  PolySeq addend;
  const u64* cst;
  u32 level;
  const u64 *a0, *a1, *b0, *b1;
  u64 in_stride;
};
// whether launch_dotprod with these arguments reads own limbs from OwnLimbs (only the kernel that shares a key does)
bool dotprod_reads_own(u32 n_keys, u32 n_ops, bool two_halves, u32 n_parts);
void launch_dotprod(hipStream_t st, const DevCtx& c, u64* out0, u64* out1, u64 out_stride, const u64* digits,
                    u64 digit_stride, u64 digits_op_stride, const KeySet& keys, u64 key1_off, u64 key_stride,
                    u32 n_parts, const LimbMap& lm, const LimbMap& key_limb, u32 n_limbs, u32 n_ops, const OwnLimbs* own = nullptr,
                    const Lift* lift = nullptr);  // lift: only with both halves (out1 != null) and keys.n == 1 or n_ops == 1
// out0[i] (+)= (sum_d digit_d * key0_d)[order[i]] (+ addend0[order[i]]), out1[i] (+)= (sum_d digit_d * key1_d)[order[i]];
// accumulate bit 0 / 1: add to what out0 / out1 holds
void launch_ext_rotate(hipStream_t st, const DevCtx& c, u64* out0, u64* out1, const u64* digits, u64 digit_stride,
                       const u64* key0, u64 key1_off, u64 key_stride, u32 n_parts, const u64* addend0, const i64* order,
                       int accumulate, const LimbMap& lm, const LimbMap& key_limb, u32 n_limbs);
// Mod_down tail for n_polys polynomials: out = (src - y) * pinv (+ addend), per limb constants cst[2t], cst[2t+1];
// addend_mode 0 none, 1 every polynomial, 2 even polynomials only.  With `orders` the result is permuted on the
// way out: out[i] = value at orders[p / 2][i] (the automorphism closing a rotation; out must not alias an input).
void launch_moddown_tail(hipStream_t st, const DevCtx& c, const PolySeq& out, const PolySeq& src, const u64* y,
                         u64 y_stride, const PolySeq* addend, int addend_mode, const u64* cst, const LimbMap& lm,
                         u32 n_limbs, u32 n_polys, const OrderSet* orders = nullptr);
// Rescale: u[p][t][i] = switch_modulus(last[p][i], q_l -> q_t) * K_t ;  cst per limb: K, K', diff
void launch_rescale_switch(hipStream_t st, const DevCtx& c, u64* u, u64 u_stride, const u64* last, u64 last_stride,
                           u32 last_prime, const u64* cst, const LimbMap& lm, u32 n_limbs, u32 n_polys);
// out = src * qlinv + u  (NTT form)   cst per limb: qlinv, qlinv'
void launch_rescale_tail(hipStream_t st, const DevCtx& c, const PolySeq& out, const PolySeq& src, const u64* u,
                         u64 u_stride, const u64* cst, const LimbMap& lm, u32 n_limbs, u32 n_polys);
// coefficient-form rescale: out = (src - (last mod q_t)) * qlinv
void launch_rescale_coef(hipStream_t st, const DevCtx& c, u64* out, const u64* src, const u64* last,
                         const u64* cst, const LimbMap& lm, u32 n_limbs);
// fused Mod_down + rescale tail in coefficient form (see moddown_rescale_kernel); out: level-1 limbs
void launch_moddown_rescale(hipStream_t st, const DevCtx& c, u64* out, const u64* poly, const u64* y, u64* last_out,
                            const u64* pinv, const u64* qlinv, u32 level);
// out[0] = src, out[i] = Switch_modulus(src, q_0 -> q_i) for i < level
void launch_from_level0(hipStream_t st, const DevCtx& c, u64* out, const u64* src, u32 level);
// out[t] = src[t] * cst[2t] (Shoup constant per limb)
void launch_mul_const(hipStream_t st, const DevCtx& c, u64* out, const u64* src, const u64* cst, const LimbMap& lm,
                      u32 n_limbs);
void launch_fill_zero(hipStream_t st, u64* p, u64 n);
// What the forward chunk pass needs of an index table before it can apply it on the way out (FwdFuse, epi 1):
// report[0] = 1 if an entry lies outside [0, N) or a 4096-word block of the table draws on more than one block of
// the source; report[1 + b] = the source block of block b.  report: 1 + N / 4096 words, zeroed by the kernel's caller.
void launch_order_check(hipStream_t st, const DevCtx& c, const i64* order, u32* report);
// Embedding_inv (util/src/ntt.c:631-675) over len complex values: out = result, r = input (overwritten)
void launch_embedding_inv(hipStream_t st, const DevCtx& c, double2* out, double2* r, const double2* rou,
                          const u32* rot, u32 len);
// Encode_impl up to the residues (coefficient form): r holds `slots` complex values on entry (zero-padded
// message) and is used as scratch; rou = exp(2 pi i k / 2N), k < 2N; rot = 5^k mod 2N, k < N/2.
// out: n_limbs limbs of N words (limb t uses lm.prime[t]).  *err is set to 1 where the reference asserts.
// z[i] = (raw[i], 0) for i < n_values, (0, 0) up to slots; raw holds doubles or floats
void launch_widen_real(hipStream_t st, double2* z, const void* raw, bool is_f32, u32 n_values, u32 slots,
                       u32 n_vec = 1);  // n_vec vectors of n_values back to back in raw, of slots in z
void launch_encode(hipStream_t st, const DevCtx& c, u64* out, double2* r, const double2* rou, const u32* rot,
                   u32 slots, double scaling_factor, double scale, double round_add, double range_bound,
                   const LimbMap& lm, u32 n_limbs, int* err, u32 n_vec = 1, u64 out_stride = 0);
constexpr int kDecodeWords = 64;  // most limbs of a polynomial the decoder reconstructs
// Decode (ckks/src/encoder.c:657-704) of a polynomial in coefficient form: r receives the `slots` complex values
void launch_decode(hipStream_t st, const DevCtx& c, double2* r, const u64* poly, u32 level, u32 slots, double factor,
                   const u64* inv, const u64* garner, u32 stride, const u64* big_q, const double2* rou,
                   const u32* rot);

}  // namespace ace
