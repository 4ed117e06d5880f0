/*
 * TEST INFRASTRUCTURE ONLY -- driver that runs the *reference's own* compiled
 * hot-path functions on inputs supplied by the test harness, so the oracle
 * (ace_oracle.c) can be compared with the real thing limb by limb.
 *
 * It is linked against the reference sources where they lie (see Makefile);
 * the context is created with the reference's Prepare_context_for_cmplr
 * (context/src/cmplr_context.c:22-45), so every getter the poly layer calls is
 * the reference's own.  No reference code is copied here: this file only
 * calls public functions declared in the reference headers.
 *
 * usage: ref_driver <request.bin> <response.bin>
 * request  (int64 words): N num_q q0_bits sf_bits parts n_ops, then per op
 *          opcode a1 a2 a3 a4 n_in  in[n_in]
 * response (int64 words): L K part_size  prime[L+K] root[L+K]
 *          modulus[5*(L+K)], then per op  n_out out[n_out]
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "common/cmplr_api.h"
#include "common/rt_config.h"
#include "context/ckks_context.h"
#include "crt_impl.h"
#include "hal/hal.h"
#include "ntt_impl.h"
#include "number_theory_impl.h"
#include "poly/rns_poly.h"
#include "ckks/encoder.h"
#include "ckks/plaintext.h"
#include "context/ckks_context.h"
#include "rns_poly_impl.h"
#include "type_impl.h"
#include "util/crt.h"
#include "util/ntt.h"
#include "util/number_theory.h"

enum {
  OP_NTT = 1, OP_INTT, OP_HW, OP_DECOMP_MODUP, OP_PRECOMP, OP_MOD_DOWN,
  OP_RESCALE, OP_DOT_PROD, OP_AUTO_ORDER, OP_AUTO_INDEX, OP_AUTOMORPHISM,
  OP_EXTEND, OP_TBL_MODUP, OP_TBL_MODDOWN, OP_TBL_RESCALE, OP_POLY, OP_TWIDDLES,
  OP_MOD_UP, OP_MOD_DOWN_RESCALE, OP_REDUCE_RESCALE_MODUP, OP_FROM_LEVEL0, OP_ENCODE, OP_DECODE, OP_EMBEDDING, OP_TIME_NTT, OP_ENCODE_SCALED, OP_TIME_KEYSWITCH, OP_TIME_PRIMITIVES
};

static int64_t* in_buf;
static size_t   in_pos;
static FILE*    out_f;

static int64_t rd(void) { return in_buf[in_pos++]; }
static void wr(const int64_t* p, size_t n) { fwrite(p, sizeof(int64_t), n, out_f); }
static void wr1(int64_t v) { wr(&v, 1); }

static size_t L, K, N;

static CRT_PRIME* prime_at(size_t idx) {
  CRT_CONTEXT* crt = Get_crt_context();
  return idx < L ? Get_prime_at(Get_q(crt), idx) : Get_prime_at(Get_p(crt), idx - L);
}

/* wrap caller memory as a POLYNOMIAL with num_q + num_p limbs allocated */
static void wrap_poly(POLYNOMIAL* p, int64_t* data, size_t num_q, size_t num_p, bool ntt) {
  memset(p, 0, sizeof(*p));
  p->_num_alloc_primes = num_q + num_p;
  Init_poly_data(p, (uint32_t)N, num_q, num_p, data);
  Set_is_ntt(p, ntt);
}

int main(int argc, char** argv) {
  if (argc != 3) { fprintf(stderr, "usage: %s req resp\n", argv[0]); return 2; }
  FILE* f = fopen(argv[1], "rb");
  if (!f) { perror("request"); return 2; }
  fseek(f, 0, SEEK_END);
  long sz = ftell(f);
  fseek(f, 0, SEEK_SET);
  in_buf = (int64_t*)malloc((size_t)sz + 8);
  if (fread(in_buf, 1, (size_t)sz, f) != (size_t)sz) { perror("read"); return 2; }
  fclose(f);
  out_f = fopen(argv[2], "wb");
  if (!out_f) { perror("response"); return 2; }

  N = (size_t)rd();
  size_t num_q = (size_t)rd(), q0 = (size_t)rd(), sf = (size_t)rd(), parts = (size_t)rd();
  size_t n_ops = (size_t)rd();
  Prepare_context_for_cmplr((uint32_t)N, 0, (uint32_t)(num_q - 1), (uint32_t)num_q,
                            (uint32_t)q0, (uint32_t)sf, (uint32_t)parts, 0);
  CRT_CONTEXT* crt = Get_crt_context();
  L = Get_q_cnt();
  K = Get_p_cnt();
  wr1((int64_t)L);
  wr1((int64_t)K);
  wr1((int64_t)Get_per_part_size(Get_qpart(crt)));
  for (size_t i = 0; i < L + K; i++) wr1(Get_modulus_val(prime_at(i)));
  for (size_t i = 0; i < L + K; i++)
    wr1(Get_i64_value_at(Get_ntt(prime_at(i))->_rou, N / 2)); /* rou[bitrev(1)] = psi */
  for (size_t i = 0; i < L + K; i++) {
    MODULUS* m = Get_modulus(prime_at(i));
    wr1(m->_val); wr1(m->_br_k); wr1(m->_br_m);
    wr1((int64_t)(uint64_t)m->_prec128);
    wr1((int64_t)(uint64_t)(m->_prec128 >> 64));
  }

  for (size_t op = 0; op < n_ops; op++) {
    int64_t code = rd(), a1 = rd(), a2 = rd(), a3 = rd(), a4 = rd();
    size_t  n_in = (size_t)rd();
    int64_t* in = in_buf + in_pos;
    in_pos += n_in;
    (void)a4;
    switch (code) {
      case OP_NTT:
      case OP_INTT: { /* a1 = n_limbs; in = prime_idx[n_limbs] data[n_limbs*N] */
        size_t nl = (size_t)a1;
        int64_t* data = in + nl;
        for (size_t t = 0; t < nl; t++) {
          VALUE_LIST vl;
          Init_i64_value_list_no_copy(&vl, N, data + t * N);
          NTT_CONTEXT* ntt = Get_ntt(prime_at((size_t)in[t]));
          if (code == OP_NTT) Ftt_fwd(&vl, ntt, &vl);
          else                Ftt_inv(&vl, ntt, &vl);
        }
        wr1((int64_t)(nl * N));
        wr(data, nl * N);
        break;
      }
      case OP_TIME_NTT: { /* a1 = n_limbs, a2 = milliseconds; in = prime_idx[n_limbs] data[n_limbs*N];
                             forward + inverse of every limb, again and again; out = round trips, ns, data */
        size_t nl = (size_t)a1;
        int64_t* data = in + nl;
        struct timespec t0, t1;
        int64_t trips = 0, ns = 0;
        clock_gettime(CLOCK_MONOTONIC, &t0);
        do {
          for (size_t t = 0; t < nl; t++) {
            VALUE_LIST vl;
            Init_i64_value_list_no_copy(&vl, N, data + t * N);
            NTT_CONTEXT* ntt = Get_ntt(prime_at((size_t)in[t]));
            Ftt_fwd(&vl, ntt, &vl);
            Ftt_inv(&vl, ntt, &vl);
          }
          trips++;
          clock_gettime(CLOCK_MONOTONIC, &t1);
          ns = (int64_t)(t1.tv_sec - t0.tv_sec) * 1000000000 + (t1.tv_nsec - t0.tv_nsec);
        } while (ns < a2 * 1000000);
        wr1((int64_t)(2 + nl * N));
        wr1(trips);
        wr1(ns);
        wr(data, nl * N);
        break;
      }
      case OP_TIME_PRIMITIVES: { /* a1 = level, a2 = seed; no input.  The functions a compiled program and the
                                    bootstrap are made of, each run once at `level` on uniform residues and timed on
                                    its own.  out = nanoseconds of: Hw_modadd, Hw_modmul, Hw_modmuladd,
                                    Hw_modmul_scalar, Hw_rotate, Hw_ntt, Hw_intt (each per limb: the mean over the
                                    level's limbs), Decomp_modup of digit 0, Mod_down, Rescale (level >= 3, else 0),
                                    one Dot_prod over all digits, Encode_at_level_with_sf of N/2 values */
        size_t lv = (size_t)a1, nd = Get_num_decomp(Get_crt_context(), lv), T = lv + K;
        uint64_t st = (uint64_t)a2 * 0x9E3779B97F4A7C15ull + 1;
        int64_t *x = (int64_t*)malloc(T * N * sizeof(int64_t)), *y = (int64_t*)malloc(T * N * sizeof(int64_t));
        int64_t* r = (int64_t*)malloc(T * N * sizeof(int64_t));
        for (size_t t = 0; t < T; t++) {
          uint64_t q = (uint64_t)Get_modulus_val(prime_at(t < lv ? t : L + (t - lv)));
          for (size_t i = 0; i < N; i++) {
            st = st * 6364136223846793005ull + 1442695040888963407ull;
            x[t * N + i] = (int64_t)((st >> 3) % q);
            st = st * 6364136223846793005ull + 1442695040888963407ull;
            y[t * N + i] = (int64_t)((st >> 3) % q);
          }
        }
        struct timespec t0, t1;
        int64_t ns[12] = {0};
#define P_TICK() clock_gettime(CLOCK_MONOTONIC, &t0)
#define P_TOCK(k, div) (clock_gettime(CLOCK_MONOTONIC, &t1), ns[k] = ((int64_t)(t1.tv_sec - t0.tv_sec) * 1000000000 + (t1.tv_nsec - t0.tv_nsec)) / (int64_t)(div))
        VALUE_LIST* order = Alloc_value_list(I64_TYPE, N);
        Precompute_automorphism_order(order, 5, (uint32_t)N, true);
        memset(r, 0, T * N * sizeof(int64_t)); /* the pages of the result are there before the first timed loop */
        P_TICK();
        for (size_t t = 0; t < lv; t++) Hw_modadd(r + t * N, x + t * N, y + t * N, Get_modulus(prime_at(t)), N);
        P_TOCK(0, lv);
        P_TICK();
        for (size_t t = 0; t < lv; t++) Hw_modmul(r + t * N, x + t * N, y + t * N, Get_modulus(prime_at(t)), N);
        P_TOCK(1, lv);
        P_TICK();
        for (size_t t = 0; t < lv; t++) Hw_modmuladd(r + t * N, x + t * N, y + t * N, Get_modulus(prime_at(t)), N);
        P_TOCK(2, lv);
        P_TICK();
        for (size_t t = 0; t < lv; t++) Hw_modmul_scalar(r + t * N, x + t * N, 12345, Get_modulus(prime_at(t)), N);
        P_TOCK(3, lv);
        P_TICK();
        for (size_t t = 0; t < lv; t++) Hw_rotate(r + t * N, x + t * N, Get_i64_values(order), Get_modulus(prime_at(t)), N);
        P_TOCK(4, lv);
        P_TICK();
        for (size_t t = 0; t < lv; t++) {
          VALUE_LIST vl;
          Init_i64_value_list_no_copy(&vl, N, r + t * N);
          Ftt_fwd(&vl, Get_ntt(prime_at(t)), &vl);
        }
        P_TOCK(5, lv);
        P_TICK();
        for (size_t t = 0; t < lv; t++) {
          VALUE_LIST vl;
          Init_i64_value_list_no_copy(&vl, N, r + t * N);
          Ftt_inv(&vl, Get_ntt(prime_at(t)), &vl);
        }
        P_TOCK(6, lv);
        POLYNOMIAL src, ext, down, low, kb[16], dg[16], acc;
        wrap_poly(&src, x, lv, 0, true);
        wrap_poly(&ext, r, lv, K, true);
        P_TICK();
        Decomp_modup(&ext, &src, 0);
        P_TOCK(7, 1);
        memset(&down, 0, sizeof(down)), memset(&low, 0, sizeof(low)), memset(&acc, 0, sizeof(acc));
        Alloc_poly_data(&down, (uint32_t)N, lv, 0);
        Set_is_ntt(&down, true);
        wrap_poly(&ext, y, lv, K, true);
        P_TICK();
        Mod_down(&down, &ext);
        P_TOCK(8, 1);
        if (lv >= 3) { /* (the reference's Rescale drops the limb through Modswitch, which wants two limbs left) */
          Alloc_poly_data(&low, (uint32_t)N, lv - 1, 0);
          Set_is_ntt(&low, true);
          P_TICK();
          Rescale(&low, &down);
          P_TOCK(9, 1);
          Free_poly_data(&low);
        }
        /* the digits and the key halves of one inner product: the same limbs seen nd times (what is timed is the
         * arithmetic; a key is viewed at `level`, as Derive_poly does) */
        for (size_t d = 0; d < nd && d < 16; d++) {
          wrap_poly(&dg[d], x, lv, K, true);
          wrap_poly(&kb[d], y, lv, K, true);
        }
        P_TICK();
        Dot_prod(&acc, dg, kb, (uint32_t)nd);
        P_TOCK(10, 1);
        Free_poly_data(&acc);
        Free_poly_data(&down);
        {
          CKKS_ENCODER* enc = (CKKS_ENCODER*)Context->_encoder;
          size_t        nv  = N / 2;
          VALUE_LIST*   vals = Alloc_value_list(DCMPLX_TYPE, nv);
          for (size_t i = 0; i < nv; i++) {
            st = st * 6364136223846793005ull + 1442695040888963407ull;
            DCMPLX_VALUE_AT(vals, i) = (double)(int64_t)(st >> 11) / (double)(1ull << 52) - 1.0;
          }
          PLAINTEXT pt;
          memset(&pt, 0, sizeof(pt));
          P_TICK();
          Encode_at_level_with_sf(&pt, enc, vals, (uint32_t)lv, (uint32_t)nv, 1);
          P_TOCK(11, 1);
          Free_poly_data(Get_plain_poly(&pt));
          Free_value_list(vals);
        }
        Free_value_list(order);
        free(x), free(y), free(r);
        wr1(12);
        wr(ns, 12);
        break;
      }
      case OP_TIME_KEYSWITCH: { /* a1 = level, a2 = seed; no input.  The pieces of one key switch at `level`, each run
                                   once on uniform residues and timed on its own: Alloc_precomp, two Dot_prod (the two
                                   halves of a key), two Mod_down, two Rescale, two Automorphism_transform.
                                   out = nanoseconds of the five, in that order */
        size_t lv = (size_t)a1, nd = Get_num_decomp(Get_crt_context(), lv);
        uint64_t st = (uint64_t)a2 * 0x9E3779B97F4A7C15ull + 1;
        int64_t* c2 = (int64_t*)malloc(lv * N * sizeof(int64_t));
        int64_t* key = (int64_t*)malloc(2 * nd * (L + K) * N * sizeof(int64_t));
        for (size_t t = 0; t < lv; t++) {
          uint64_t q = (uint64_t)Get_modulus_val(prime_at(t));
          for (size_t i = 0; i < N; i++) {
            st = st * 6364136223846793005ull + 1442695040888963407ull;
            c2[t * N + i] = (int64_t)((st >> 3) % q);
          }
        }
        for (size_t h = 0; h < 2 * nd; h++)
          for (size_t t = 0; t < L + K; t++) {
            uint64_t q = (uint64_t)Get_modulus_val(prime_at(t));
            for (size_t i = 0; i < N; i++) {
              st = st * 6364136223846793005ull + 1442695040888963407ull;
              key[(h * (L + K) + t) * N + i] = (int64_t)((st >> 3) % q);
            }
          }
        struct timespec t0, t1;
        int64_t ns[5];
#define TICK() clock_gettime(CLOCK_MONOTONIC, &t0)
#define TOCK(k) (clock_gettime(CLOCK_MONOTONIC, &t1), ns[k] = (int64_t)(t1.tv_sec - t0.tv_sec) * 1000000000 + (t1.tv_nsec - t0.tv_nsec))
        POLYNOMIAL src, kb[16], ka[16], dg[16], ext[2], down[2], low[2], rot[2];
        wrap_poly(&src, c2, lv, 0, true);
        TICK();
        VALUE_LIST* pl = Alloc_precomp(&src);
        TOCK(0);
        for (size_t d = 0; d < nd; d++) {
          dg[d] = *(POLYNOMIAL*)Get_ptr_value_at(pl, d);
          wrap_poly(&kb[d], key + (2 * d) * (L + K) * N, L, K, true);
          wrap_poly(&ka[d], key + (2 * d + 1) * (L + K) * N, L, K, true);
        }
        memset(ext, 0, sizeof(ext)), memset(down, 0, sizeof(down)), memset(low, 0, sizeof(low)), memset(rot, 0, sizeof(rot));
        TICK();
        Dot_prod(&ext[0], dg, kb, (uint32_t)nd);
        Dot_prod(&ext[1], dg, ka, (uint32_t)nd);
        TOCK(1);
        for (int h = 0; h < 2; h++) {
          Alloc_poly_data(&down[h], (uint32_t)N, lv, 0);
          Alloc_poly_data(&low[h], (uint32_t)N, lv - 1, 0);
          Alloc_poly_data(&rot[h], (uint32_t)N, lv, 0);
          Set_is_ntt(&down[h], true), Set_is_ntt(&low[h], true), Set_is_ntt(&rot[h], true);
        }
        TICK();
        Mod_down(&down[0], &ext[0]);
        Mod_down(&down[1], &ext[1]);
        TOCK(2);
        VALUE_LIST* order = Alloc_value_list(I64_TYPE, N);
        Precompute_automorphism_order(order, 5, (uint32_t)N, true);
        TICK();
        Automorphism_transform(&rot[0], &down[0], order);
        Automorphism_transform(&rot[1], &down[1], order);
        TOCK(4);
        TICK();
        Rescale(&low[0], &down[0]);
        Rescale(&low[1], &down[1]);
        TOCK(3);
#undef TICK
#undef TOCK
        wr1(5);
        wr(ns, 5);
        for (int h = 0; h < 2; h++) {
          Free_poly_data(&ext[h]), Free_poly_data(&down[h]), Free_poly_data(&low[h]), Free_poly_data(&rot[h]);
        }
        Free_value_list(order);
        Free_precomp(pl);
        free(c2), free(key);
        break;
      }
      case OP_HW: { /* a1 = which, a2 = prime idx, a3 = n; in = r[n] a[n] b[n] */
        size_t n = (size_t)a3;
        int64_t *r = in, *a = in + n, *b = in + 2 * n;
        MODULUS* m = Get_modulus(prime_at((size_t)a2));
        switch (a1) {
          case 0: Hw_modadd(r, a, b, m, n); break;
          case 1: Hw_modsub(r, a, b, m, n); break;
          case 2: Hw_modmul(r, a, b, m, n); break;
          case 3: Hw_modmuladd(r, a, b, m, n); break;
          case 4: Hw_modadd_scalar(r, a, b[0], m, n); break;
          case 5: Hw_modsub_scalar(r, a, b[0], m, n); break;
          case 6: Hw_modmul_scalar(r, a, b[0], m, n); break;
          case 7: Hw_modmuladd_scalar(r, a, b[0], m, n); break;
          case 8: Hw_rotate(r, a, b, m, n); break;
          default: fprintf(stderr, "bad hw op\n"); return 2;
        }
        wr1((int64_t)n);
        wr(r, n);
        break;
      }
      case OP_DECOMP_MODUP: { /* a1 level, a2 part, a3 is_ntt; in = level*N */
        size_t lv = (size_t)a1;
        POLYNOMIAL src, res;
        wrap_poly(&src, in, lv, 0, a3 != 0);
        int64_t* out = (int64_t*)calloc((lv + K) * N, sizeof(int64_t));
        wrap_poly(&res, out, lv, K, a3 != 0);
        Decomp_modup(&res, &src, (uint32_t)a2);
        wr1((int64_t)((lv + K) * N));
        wr(out, (lv + K) * N);
        free(out);
        break;
      }
      case OP_MOD_UP: { /* a1 level, a2 part, a3 is_ntt, in = level*N (Decomp then Mod_up) */
        size_t lv = (size_t)a1;
        POLYNOMIAL src, res, dig;
        wrap_poly(&src, in, lv, 0, a3 != 0);
        int64_t* out = (int64_t*)calloc((lv + K) * N, sizeof(int64_t));
        wrap_poly(&res, out, lv, K, a3 != 0);
        memset(&dig, 0, sizeof(dig));
        Alloc_poly_data(&dig, (uint32_t)N, lv + K, 0);
        Decomp(&dig, &src, (uint32_t)a2);
        Mod_up(&res, &dig, (uint32_t)a2);
        wr1((int64_t)((lv + K) * N));
        wr(out, (lv + K) * N);
        free(out);
        Free_poly_data(&dig);
        break;
      }
      case OP_PRECOMP: { /* a1 level, a2 is_ntt, a3 fused */
        size_t lv = (size_t)a1;
        POLYNOMIAL src;
        wrap_poly(&src, in, lv, 0, a2 != 0);
        Set_rtlib_config(CONF_OP_FUSION_DECOMP_MODUP, a3 ? 1 : 0);
        VALUE_LIST* pl = Alloc_precomp(&src);
        size_t nd = LIST_LEN(pl);
        wr1((int64_t)(nd * (lv + K) * N));
        for (size_t d = 0; d < nd; d++) {
          POLYNOMIAL* p = (POLYNOMIAL*)Get_ptr_value_at(pl, d);
          wr(Get_poly_coeffs(p), (lv + K) * N);
        }
        Free_precomp(pl);
        break;
      }
      case OP_MOD_DOWN: { /* a1 level, a2 is_ntt; in = (level+K)*N */
        size_t lv = (size_t)a1;
        POLYNOMIAL src, res;
        wrap_poly(&src, in, lv, K, a2 != 0);
        int64_t* out = (int64_t*)calloc(lv * N, sizeof(int64_t));
        wrap_poly(&res, out, lv, 0, a2 != 0);
        Mod_down(&res, &src);
        wr1((int64_t)(lv * N));
        wr(out, lv * N);
        free(out);
        break;
      }
      case OP_MOD_DOWN_RESCALE: { /* a1 level, a2 is_ntt; in = (level+K)*N; out = result, input as left */
        size_t lv = (size_t)a1;
        POLYNOMIAL src, res;
        wrap_poly(&src, in, lv, K, a2 != 0);
        int64_t* out = (int64_t*)calloc(lv * N, sizeof(int64_t));
        wrap_poly(&res, out, lv, 0, a2 != 0);
        Mod_down_rescale(&res, &src);
        wr1((int64_t)((lv - 1) * N + (lv + K) * N + 1));
        wr(out, (lv - 1) * N);
        wr(in, (lv + K) * N);
        wr1((int64_t)Is_ntt(&res));
        free(out);
        break;
      }
      case OP_REDUCE_RESCALE_MODUP: { /* a1 level, a2 is_ntt; in = (level+K)*N; out = res[level], raised, input */
        size_t lv = (size_t)a1;
        POLYNOMIAL src, res;
        wrap_poly(&src, in, lv, K, a2 != 0);
        int64_t* out = (int64_t*)calloc(lv * N, sizeof(int64_t));
        wrap_poly(&res, out, lv, 0, a2 != 0);
        VALUE_LIST* raised = Reduce_and_rescale_modup(&res, &src);
        size_t nd = LIST_LEN(raised), each = (lv - 1 + K) * N;
        wr1((int64_t)(lv * N + nd * each + (lv + K) * N));
        wr(out, lv * N);
        for (size_t d = 0; d < nd; d++) wr(Get_poly_coeffs((POLYNOMIAL*)Get_ptr_value_at(raised, d)), each);
        wr(in, (lv + K) * N);
        Free_precomp(raised);
        free(out);
        break;
      }
      case OP_FROM_LEVEL0: { /* a1 level; in = N words (limb 0) */
        size_t lv = (size_t)a1;
        POLYNOMIAL src, res;
        wrap_poly(&src, in, 1, 0, false);
        int64_t* out = (int64_t*)calloc(lv * N, sizeof(int64_t));
        wrap_poly(&res, out, lv, 0, false);
        Transform_values_from_level0(&res, &src);
        wr1((int64_t)(lv * N));
        wr(out, lv * N);
        free(out);
        break;
      }
      case OP_ENCODE: { /* a1 level, a2 slots, a3 sf_degree, a4 p_cnt; in = n_values complex doubles (raw bits) */
        size_t lv = (size_t)a1, pc = (size_t)a4, nv = n_in / 2;
        CKKS_ENCODER* enc = (CKKS_ENCODER*)Context->_encoder;
        VALUE_LIST* vals = Alloc_value_list(DCMPLX_TYPE, nv);
        memcpy(DCMPLX_VALUES(vals), in, nv * sizeof(DCMPLX));
        PLAINTEXT pt;
        memset(&pt, 0, sizeof(pt));
        if (pc) Encode_ext_at_level(&pt, enc, vals, (uint32_t)lv, (uint32_t)a2, (uint32_t)pc);
        else Encode_at_level_with_sf(&pt, enc, vals, (uint32_t)lv, (uint32_t)a2, (uint32_t)a3);
        POLYNOMIAL* poly = Get_plain_poly(&pt);
        size_t n = (Poly_level(poly) + Num_p(poly)) * N;
        wr1((int64_t)(n + 3));
        wr(Get_poly_coeffs(poly), Poly_level(poly) * N);
        if (Num_p(poly)) wr(Get_p_coeffs(poly), Num_p(poly) * N);
        wr1((int64_t)pt._slots);
        wr1((int64_t)pt._sf_degree);
        { double sf = pt._scaling_factor; int64_t bits; memcpy(&bits, &sf, 8); wr1(bits); }
        Free_poly_data(poly);
        Free_value_list(vals);
        break;
      }
      case OP_ENCODE_SCALED: { /* a1 level, a2 slots, a3 raw bits of the scale, a4 p_cnt; in = complex doubles */
        size_t lv = (size_t)a1, nv = n_in / 2;
        double scale;
        memcpy(&scale, &a3, 8);
        CKKS_ENCODER* enc = (CKKS_ENCODER*)Context->_encoder;
        VALUE_LIST* vals = Alloc_value_list(DCMPLX_TYPE, nv);
        memcpy(DCMPLX_VALUES(vals), in, nv * sizeof(DCMPLX));
        PLAINTEXT pt;
        memset(&pt, 0, sizeof(pt));
        Encode_at_level_with_scale(&pt, enc, vals, (uint32_t)lv, (uint32_t)a2, scale, (uint32_t)a4);
        POLYNOMIAL* poly = Get_plain_poly(&pt);
        size_t n = (Poly_level(poly) + Num_p(poly)) * N;
        wr1((int64_t)(n + 3));
        wr(Get_poly_coeffs(poly), Poly_level(poly) * N);
        if (Num_p(poly)) wr(Get_p_coeffs(poly), Num_p(poly) * N);
        wr1((int64_t)pt._slots);
        wr1((int64_t)pt._sf_degree);
        { double sf = pt._scaling_factor; int64_t bits; memcpy(&bits, &sf, 8); wr1(bits); }
        Free_poly_data(poly);
        Free_value_list(vals);
        break;
      }
      case OP_DECODE: { /* a1 level, a2 slots, a3 is_ntt, a4 raw bits of the scaling factor; in = level*N */
        size_t lv = (size_t)a1;
        CKKS_ENCODER* enc = (CKKS_ENCODER*)Context->_encoder;
        PLAINTEXT pt;
        memset(&pt, 0, sizeof(pt));
        wrap_poly(Get_plain_poly(&pt), in, lv, 0, a3 != 0);
        pt._slots = (uint32_t)a2;
        memcpy(&pt._scaling_factor, &a4, 8);
        pt._sf_degree = 1;
        VALUE_LIST* res = Alloc_value_list(DCMPLX_TYPE, (size_t)a2);
        Decode(res, enc, &pt);
        wr1((int64_t)(2 * a2));
        wr((int64_t*)DCMPLX_VALUES(res), 2 * (size_t)a2);
        Free_value_list(res);
        break;
      }
      case OP_EMBEDDING: { /* a1 inverse; in = len complex doubles */
        size_t len = n_in / 2;
        CKKS_ENCODER* enc = (CKKS_ENCODER*)Context->_encoder;
        VALUE_LIST* vals = Alloc_value_list(DCMPLX_TYPE, len);
        VALUE_LIST* res  = Alloc_value_list(DCMPLX_TYPE, len);
        memcpy(DCMPLX_VALUES(vals), in, len * sizeof(DCMPLX));
        if (a1) Embedding_inv(res, enc->_fft, vals);
        else Embedding(res, enc->_fft, vals);
        wr1((int64_t)(2 * len));
        wr((int64_t*)DCMPLX_VALUES(res), 2 * len);
        Free_value_list(vals);
        Free_value_list(res);
        break;
      }
      case OP_RESCALE: { /* a1 level, a2 is_ntt; in = level*N */
        size_t lv = (size_t)a1;
        POLYNOMIAL src, res;
        wrap_poly(&src, in, lv, 0, a2 != 0);
        int64_t* out = (int64_t*)calloc(lv * N, sizeof(int64_t));
        wrap_poly(&res, out, lv, 0, a2 != 0);
        Rescale(&res, &src);
        wr1((int64_t)((lv - 1) * N));
        wr(out, (lv - 1) * N);
        free(out);
        break;
      }
      case OP_DOT_PROD: { /* a1 level, a2 n_parts, a3 fast; in = digits, keys */
        size_t lv = (size_t)a1, np = (size_t)a2;
        POLYNOMIAL dg[16], ky[16], res;
        int64_t* digits = in;
        int64_t* keys   = in + np * (lv + K) * N;
        for (size_t d = 0; d < np; d++) {
          wrap_poly(&dg[d], digits + d * (lv + K) * N, lv, K, true);
          wrap_poly(&ky[d], keys + d * (L + K) * N, L, K, true);
        }
        Set_rtlib_config(CONF_FAST_DOT_PROD, a3 ? 1 : 0);
        memset(&res, 0, sizeof(res));
        Dot_prod(&res, dg, ky, (uint32_t)np);
        wr1((int64_t)((lv + K) * N));
        wr(Get_poly_coeffs(&res), (lv + K) * N);
        Free_poly_data(&res);
        break;
      }
      case OP_AUTO_ORDER: { /* a1 k, a2 is_ntt */
        VALUE_LIST* vl = Alloc_value_list(I64_TYPE, N);
        Precompute_automorphism_order(vl, (uint32_t)a1, (uint32_t)N, a2 != 0);
        wr1((int64_t)N);
        wr(Get_i64_values(vl), N);
        Free_value_list(vl);
        break;
      }
      case OP_AUTO_INDEX: { /* a1 rot_idx */
        MODULUS m;
        Init_modulus(&m, 2 * (int64_t)N);
        wr1(1);
        wr1((int64_t)Find_automorphism_index((int32_t)a1, &m));
        break;
      }
      case OP_AUTOMORPHISM: { /* a1 level, a2 with_p, a3 is_ntt; in = poly, order[N] */
        size_t lv = (size_t)a1, T = lv + (a2 ? K : 0);
        POLYNOMIAL src, res;
        wrap_poly(&src, in, lv, a2 ? K : 0, a3 != 0);
        int64_t* out = (int64_t*)calloc(T * N, sizeof(int64_t));
        wrap_poly(&res, out, lv, a2 ? K : 0, a3 != 0);
        VALUE_LIST ord;
        Init_i64_value_list_no_copy(&ord, N, in + T * N);
        Automorphism_transform(&res, &src, &ord);
        wr1((int64_t)(T * N));
        wr(out, T * N);
        free(out);
        break;
      }
      case OP_EXTEND: { /* a1 level */
        size_t lv = (size_t)a1;
        POLYNOMIAL src, res;
        wrap_poly(&src, in, lv, 0, true);
        int64_t* out = (int64_t*)calloc((lv + K) * N, sizeof(int64_t));
        wrap_poly(&res, out, lv, K, true);
        Extend(&res, &src);
        wr1((int64_t)((lv + K) * N));
        wr(out, (lv + K) * N);
        free(out);
        break;
      }
      case OP_TBL_MODUP: { /* a1 level, a2 part: hat_inv[nd], hat[nd][nc], compl primes[nc] */
        size_t lv = (size_t)a1, part = (size_t)a2;
        CRT_PRIMES* qp = Get_qpart(crt);
        size_t ps = Get_per_part_size(qp), ndec = Get_num_decomp(crt, lv);
        size_t nd = (part == ndec - 1) ? lv - ps * part
                                       : LIST_LEN(Get_qpart_prime_at_l1(qp, part));
        VALUE_LIST* hinv = VL_L2_VALUE_AT(Get_qlhatinvmodq(qp), part, nd - 1);
        VL_VL_I64*  hat  = VL_L2_VALUE_AT(Get_qlhatmodp(qp), lv - 1, part);
        VL_CRTPRIME* cp  = Get_qpart_compl_at(Get_qpart_compl(crt), lv - 1, part);
        size_t nc = LIST_LEN(cp);
        wr1((int64_t)(2 + nd + nd * nc + nc));
        wr1((int64_t)nd);
        wr1((int64_t)nc);
        wr(Get_i64_values(hinv), nd);
        for (size_t i = 0; i < nd; i++) wr(Get_i64_values(VL_VALUE_AT(hat, i)), nc);
        for (size_t j = 0; j < nc; j++) wr1(Get_modulus_val(Get_vlprime_at(cp, j)));
        break;
      }
      case OP_TBL_MODDOWN: { /* phat_inv[K], phat_modq[L][K], pinv_modq[L], pmodq[L] */
        CRT_PRIMES* p = Get_p(crt);
        wr1((int64_t)(K + L * K + 2 * L));
        wr(Get_i64_values(Get_phatinvmodp(p)), K);
        for (size_t i = 0; i < L; i++) wr(Get_i64_values(Get_phatmodq_at(p, i)), K);
        wr(Get_i64_values(Get_pinvmodq(p)), L);
        wr(Get_i64_values(Get_pmodq(p)), L);
        break;
      }
      case OP_TBL_RESCALE: { /* a1 level: ql_inv[level-1], qlql[level-1] */
        size_t lv = (size_t)a1;
        CRT_PRIMES* q = Get_q(crt);
        wr1((int64_t)(2 * (lv - 1)));
        wr(Get_i64_values(Get_ql_inv_mod_qi_at(q, lv - 2)), lv - 1);
        wr(Get_i64_values(Get_ql_ql_inv_mod_ql_div_ql_mod_qi_at(q, lv - 2)), lv - 1);
        break;
      }
      case OP_POLY: { /* a1 which (0 add 1 sub 2 mul), a2 level, a3 with_p; in = a, b */
        size_t lv = (size_t)a2, T = lv + (a3 ? K : 0);
        POLYNOMIAL pa, pb, res;
        wrap_poly(&pa, in, lv, a3 ? K : 0, true);
        wrap_poly(&pb, in + T * N, lv, a3 ? K : 0, true);
        int64_t* out = (int64_t*)calloc(T * N, sizeof(int64_t));
        wrap_poly(&res, out, lv, a3 ? K : 0, true);
        if (a1 == 0) Add_poly(&res, &pa, &pb);
        else if (a1 == 1) Sub_poly(&res, &pa, &pb);
        else Mul_poly(&res, &pa, &pb);
        wr1((int64_t)(T * N));
        wr(out, T * N);
        free(out);
        break;
      }
      case OP_TWIDDLES: { /* a1 prime idx: rou, rou_prec, rou_inv, rou_inv_prec, ninv, ninv_prec */
        NTT_CONTEXT* ntt = Get_ntt(prime_at((size_t)a1));
        wr1((int64_t)(4 * N + 2));
        wr(Get_i64_values(ntt->_rou), N);
        wr((int64_t*)Get_ui64_values(ntt->_rou_prec), N);
        wr(Get_i64_values(ntt->_rou_inv), N);
        wr((int64_t*)Get_ui64_values(ntt->_rou_inv_prec), N);
        wr1((int64_t)ntt->_degree_inv);
        wr1((int64_t)ntt->_degree_inv_prec);
        break;
      }
      default:
        fprintf(stderr, "unknown opcode %ld\n", (long)code);
        return 2;
    }
  }
  fclose(out_f);
  return 0;
}
