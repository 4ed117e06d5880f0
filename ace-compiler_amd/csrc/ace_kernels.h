// Launchers of the gfx950 kernels (definitions in ace_ntt.hip, ace_poly.hip).
// Every launcher enqueues on the given stream and returns immediately.
#pragma once
#include "ace_device.h"

namespace ace {

enum EwOp { EW_ADD, EW_SUB, EW_MUL, EW_MULADD, EW_ADD_S, EW_SUB_S, EW_MUL_S, EW_MULADD_S };

// NTT / INTT over n_polys x n_limbs limbs (limb t of poly p at
// base + p*poly_stride + t*N words).  scale: optional device array of
// 2*n_limbs words (constant, Shoup companion) replacing 1/N in the inverse.
// pos: optional limb positions (limb t at pos->prime[t]*N instead of t*N).
// passes: for N > 4096 the transform is two kernels; bit 0 / bit 1 select them
// (both by default; single passes exist so a benchmark can time each kernel).
bool launch_ntt(hipStream_t st, const DevCtx& c, u64* dst, const u64* src, const LimbMap& lm, const LimbMap* pos,
                u32 n_limbs, u32 n_polys, u64 poly_stride, bool inverse, const u64* scale, int passes = 3);

// elementwise over n_limbs limbs of n words each (limb t uses lm.prime[t]);
// scalar ops take the same scalar for every limb.
void launch_ew(hipStream_t st, const DevCtx& c, EwOp op, u64* r, const u64* a, const u64* b, u64 scalar,
               const LimbMap& lm, u32 n_limbs, u64 n);
// r[t][i] = order[i] >= 0 ? a[t][order[i]] : q_t - a[t][-order[i]]
void launch_gather(hipStream_t st, const DevCtx& c, u64* r, const u64* a, const i64* order, const LimbMap& lm,
                   u32 n_limbs, u64 n);
// two polynomials gathered with one table (rotation of c0 and c1)
void launch_gather2(hipStream_t st, const DevCtx& c, u64* r0, u64* r1, const u64* a0, const u64* a1,
                    const i64* order, const LimbMap& lm, u32 n_limbs, u64 n);
// tensor product of two ciphertexts: d0 = a0*b0, d1 = a0*b1 + a1*b0, d2 = a1*b1
void launch_tensor(hipStream_t st, const DevCtx& c, u64* d0, u64* d1, u64* d2, const u64* a0, const u64* a1,
                   const u64* b0, const u64* b1, const LimbMap& lm, u32 n_limbs);
// fast base conversion: out[map.out_limb[j]][i] = (sum_k t[k][i] * hat[k*hat_stride + j]) mod prime map.prime[j]
// t: nd limbs of canonical residues, already multiplied by the inverse cofactors.
void launch_baseconv(hipStream_t st, const DevCtx& c, u64* out, const u64* t, const u64* hat, u32 hat_stride,
                     u32 nd, u32 nc, const ConvMap& map);
// inner product with a switch key: out0/out1 (n_limbs limbs) = sum_d digits[d] * key[d][0/1]
// key limb of launch limb t is key_limb[t]; out1/key1 may be null (single polynomial).
void launch_dotprod(hipStream_t st, const DevCtx& c, u64* out0, u64* out1, const u64* digits, u64 digit_stride,
                    const u64* key0, const u64* key1, u64 key_stride, u32 n_parts, const LimbMap& lm,
                    const LimbMap& key_limb, u32 n_limbs);
// Mod_down tail: out = (src - y) * pinv (+ addend if given), per limb constants cst[2t], cst[2t+1]
void launch_moddown_tail(hipStream_t st, const DevCtx& c, u64* out, const u64* src, const u64* y,
                         const u64* addend, const u64* cst, const LimbMap& lm, u32 n_limbs);
// Rescale: u[t][i] = switch_modulus(last[i], q_l -> q_t) * K_t ;  cst per limb: K, K', diff
void launch_rescale_switch(hipStream_t st, const DevCtx& c, u64* u, const u64* last, u32 last_prime,
                           const u64* cst, const LimbMap& lm, u32 n_limbs);
// out = src * qlinv + u  (NTT form)   cst per limb: qlinv, qlinv'
void launch_rescale_tail(hipStream_t st, const DevCtx& c, u64* out, const u64* src, const u64* u, const u64* cst,
                         const LimbMap& lm, u32 n_limbs);
// coefficient-form rescale: out = (src - (last mod q_t)) * qlinv
void launch_rescale_coef(hipStream_t st, const DevCtx& c, u64* out, const u64* src, const u64* last,
                         const u64* cst, const LimbMap& lm, u32 n_limbs);
// out[t] = src[t] * cst[2t] (Shoup constant per limb)
void launch_mul_const(hipStream_t st, const DevCtx& c, u64* out, const u64* src, const u64* cst, const LimbMap& lm,
                      u32 n_limbs);
void launch_fill_zero(hipStream_t st, u64* p, u64 n);

}  // namespace ace
