/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle (see ace_oracle.h for the contract
 * and the pinning status of every function).  Plain C, one thread, no
 * dependencies beyond libc/libm.  Reference paths are relative to
 * fhe-cmplr/rtlib/ant.
 */
#include "ace_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

typedef unsigned __int128 u128;
typedef __int128          i128;
typedef uint64_t          u64;
typedef int64_t           i64;

#define ORC_ASSERT(c, msg)                                          \
  do {                                                              \
    if (!(c)) {                                                     \
      fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, msg);      \
      abort();                                                      \
    }                                                               \
  } while (0)

/* include/util/modular.h:21-26 */
typedef struct {
  i64  val;
  i64  br_k;
  i64  br_m;
  u128 prec128;
} modulus_t;

struct orc_ctx {
  uint32_t   N, logN;
  size_t     L, K, parts, part_size;
  modulus_t* mod;  /* [L+K] */
  i64*       root; /* [L+K] */
  u64 *      rou, *rou_prec, *rou_inv, *rou_inv_prec; /* [(L+K)*N] */
  u64 *      ninv, *ninv_prec;                        /* [L+K] */
  size_t     q0_bits, sf_bits;                        /* 0 when the primes were given explicitly */
  double*    fft_rou;   /* [2N][2]: cos, sin of 2 pi i / 2N (util/src/ntt.c:561-570) */
  i64*       rot_group; /* [N/2]: 5^i mod 2N           (util/src/ntt.c:580-586) */
};

/* ---------------------------------------------------------------------- */
/* scalar modular arithmetic, include/util/modular.h                      */
/* ---------------------------------------------------------------------- */

/* modular.h:139-145 */
int64_t orc_add_mod(int64_t a, int64_t b, int64_t q) {
  a += b;
  return a >= q ? a - q : a;
}

/* modular.h:153-160 (keeps the "res > val1" wrap test) */
int64_t orc_sub_mod(int64_t a, int64_t b, int64_t q) {
  i64 r = (i64)((u64)a - (u64)b);
  if (r > a || r < 0) r += q;
  return r;
}

/* modular.h:48-64: floor(2^128 / q) */
static u128 prec128_of(u64 q) {
  /* 2^128 = (2^128 - 1) + 1; floor((2^128-1)/q) differs from floor(2^128/q)
   * only when q divides 2^128, impossible for odd q > 1 */
  u128 all = ~(u128)0;
  u128 d   = all / q;
  if (all - d * q == (u128)q - 1) d += 1;
  return d;
}

void orc_precompute_const_128(uint64_t q, uint64_t out[2]) {
  u128 p = prec128_of(q);
  out[0] = (u64)p;
  out[1] = (u64)(p >> 64);
}

/* modular.h:67-72 */
static void init_modulus(modulus_t* m, i64 val) {
  m->val     = val;
  m->br_k    = 2 * ((i64)log2((double)val) + 1);
  m->br_m    = (i64)(((i128)1 << m->br_k) / val);
  m->prec128 = prec128_of((u64)val);
}

/* modular.h:185-224: low word of floor(x*mu/2^128), one multiply-subtract,
 * then subtract q while needed */
static inline i64 barrett128(u128 x, const modulus_t* m) {
  u64  xl = (u64)x, xh = (u64)(x >> 64);
  u64  ml = (u64)m->prec128, mh = (u64)(m->prec128 >> 64);
  u128 ll  = (u128)xl * ml;
  u128 lh  = (u128)xl * mh;
  u128 hl  = (u128)xh * ml;
  u128 mid = (ll >> 64) + (u64)lh + (u64)hl;
  u64  qhat = (u64)(lh >> 64) + (u64)(hl >> 64) + (u64)(mid >> 64) + xh * mh;
  u64  q = (u64)m->val;
  u64  r = xl - qhat * q;
  while (r >= q) r -= q;
  return (i64)r;
}

/* modular.h:166-183 */
static inline i64 barrett64(i64 val, const modulus_t* m) {
  u128 tmp = (u128)(u64)val * (u64)m->br_m;
  tmp >>= m->br_k;
  tmp *= (u64)m->val;
  i64 r = (i64)((u128)(u64)val - tmp);
  return r >= m->val ? r - m->val : r;
}

/* modular.h:231-241 (value of the Barrett branch) */
static inline i64 mul_mod_barrett(i64 a, i64 b, const modulus_t* m) {
  return barrett128((u128)(u64)a * (u64)b, m);
}

int64_t orc_mul_mod_barrett(const orc_ctx* c, size_t idx, int64_t a, int64_t b) {
  return mul_mod_barrett(a, b, &c->mod[idx]);
}

/* modular.h:325-329 */
uint64_t orc_precompute_const(uint64_t v, uint64_t q) {
  return (u64)(((u128)v << 64) / q);
}

/* modular.h:249-256 */
static inline i64 shoup_mul(u64 a, u64 w, u64 wp, u64 q) {
  u64 t = (u64)(((u128)a * wp) >> 64);
  u64 y = a * w - t * q;
  return (i64)(y >= q ? y - q : y);
}
int64_t orc_fast_mul_const(uint64_t a, uint64_t w, uint64_t wp, uint64_t q) {
  return shoup_mul(a, w, wp, q);
}

/* modular.h:296-322 */
int64_t orc_switch_modulus(int64_t v, int64_t old_q, int64_t new_q) {
  i64 res = v, half = old_q >> 1;
  if (new_q > old_q) {
    if (res > half) res += new_q - old_q;
  } else {
    i64 diff = new_q - (old_q % new_q);
    if (res > half) res += diff;
    if (res >= new_q) res %= new_q;
  }
  return res;
}

/* modular.h:124-131 (exact product mod q; used for set-up tables only) */
static inline i64 mul_mod_exact(i64 a, i64 b, i64 q) {
  i128 r = ((i128)a * b) % q;
  if (r < 0) r += q;
  return (i64)r;
}

/* util/src/number_theory.c:33-49 */
int64_t orc_mod_exp(int64_t v, int64_t e, int64_t q) {
  i64 result = 1, base = v % q;
  while (e > 0) {
    if (e & 1) result = mul_mod_exact(result, base, q);
    base = mul_mod_exact(base, base, q);
    e >>= 1;
  }
  if (result < 0) result += q;
  return result;
}

/* number_theory.c:57-79: extended Euclid, any modulus */
int64_t orc_mod_inv(int64_t v, int64_t m) {
  i64 mv = m, a = v % m;
  ORC_ASSERT(a != 0, "val does not have Mod_inv");
  if (m == 1) return 0;
  i64 y = 0, x = 1;
  while (a > 1) {
    i64 t = mv, q = a / t;
    mv = a % t;
    a  = t;
    t  = y;
    y  = x - q * y;
    x  = t;
  }
  if (x < 0) x += m;
  return x;
}

static i64 inv_prime(i64 v, i64 q) { return orc_mod_exp(v, q - 2, q); }

/* number_theory.c:164-189 decides primality with 200 random Miller-Rabin
 * rounds; the deterministic base set below gives the same verdict for every
 * 64-bit input */
int orc_is_prime(int64_t n) {
  if (n < 2) return 0;
  static const i64 small[] = {2, 3, 5, 7, 11, 13, 17, 19, 23, 29, 31, 37};
  for (size_t i = 0; i < 12; i++) {
    if (n == small[i]) return 1;
    if (n % small[i] == 0) return 0;
  }
  i64 d = n - 1;
  int s = 0;
  while ((d & 1) == 0) { d >>= 1; s++; }
  for (size_t i = 0; i < 12; i++) {
    i64 x = orc_mod_exp(small[i], d, n);
    if (x == 1 || x == n - 1) continue;
    int comp = 1;
    for (int r = 1; r < s; r++) {
      x = mul_mod_exact(x, x, n);
      if (x == n - 1) { comp = 0; break; }
    }
    if (comp) return 0;
  }
  return 1;
}

/* number_theory.c:97-139: smallest primitive root of a prime */
int64_t orc_find_generator(int64_t q) {
  i64 phi = q - 1, number = phi;
  i64 fac[64];
  size_t nf = 0;
  for (i64 i = 2; i <= (i64)sqrt((double)number); i++) {
    if (number % i == 0) {
      fac[nf++] = i;
      while (number % i == 0) number /= i;
    }
  }
  if (number > 1) fac[nf++] = number;
  for (i64 r = 2; r <= phi; r++) {
    int bad = 0;
    for (size_t i = 0; i < nf; i++) {
      if (orc_mod_exp(r, phi / fac[i], q) == 1) { bad = 1; break; }
    }
    if (!bad) return r;
  }
  return -1;
}

/* util/src/std_param.c:229-300: (order, prime, root) overrides consulted by
 * Root_of_unity before it computes anything (orders 32 and 32768 only) */
typedef struct { i64 order, prime, rou; } rou_entry;
static const rou_entry Rou_tbl[] = {
#include "rou_table.inc"
};

/* number_theory.c:141-162 */
int64_t orc_root_of_unity(int64_t order, int64_t q) {
  ORC_ASSERT((q - 1) % order == 0, "modulus - 1 not divisible by order");
  for (size_t i = 0; i < sizeof(Rou_tbl) / sizeof(Rou_tbl[0]); i++)
    if (Rou_tbl[i].order == order && Rou_tbl[i].prime == q) return Rou_tbl[i].rou;
  i64 g = orc_find_generator(q);
  return orc_mod_exp(g, (q - 1) / order, q);
}

/* ---------------------------------------------------------------------- */
/* prime generation, util/src/crt.c:42-148                                */
/* ---------------------------------------------------------------------- */

/* crt.c:42-50 */
static i64 gen_first_prime(uint32_t N, size_t bits) {
  i64 order = 2 * (i64)N;
  i64 p     = ((i64)1 << bits) + order + 1;
  while (!orc_is_prime(p)) p += order;
  return p;
}
/* crt.c:52-58 */
static i64 gen_previous_prime(i64 mod, i64 order) {
  i64 p = mod - order;
  while (!orc_is_prime(p)) p -= order;
  return p;
}
/* crt.c:60-67: the first candidate tried is mod + 2*order */
static i64 gen_next_prime(i64 mod, i64 order) {
  i64 p = mod + order;
  do { p += order; } while (!orc_is_prime(p));
  return p;
}

/* crt.c:112-148 */
static void generate_q_primes(i64* primes, size_t n, size_t first_bits,
                              size_t sf_bits, uint32_t N) {
  i64 order = 2 * (i64)N;
  i64 p     = gen_first_prime(N, sf_bits);
  primes[n - 1] = p;
  i64 q_next = p, q_prev = p;
  if (n > 1) {
    uint32_t cnt = 0;
    for (size_t i = n - 2; i >= 1; i--) {
      if ((cnt % 2) == 0) {
        q_prev = gen_previous_prime(q_prev, order);
        p      = q_prev;
      } else {
        q_next = gen_next_prime(q_next, order);
        p      = q_next;
      }
      primes[i] = p;
      cnt++;
    }
  }
  if (first_bits == sf_bits) {
    primes[0] = gen_previous_prime(q_prev, order);
  } else {
    primes[0] = gen_previous_prime(gen_first_prime(N, first_bits), order);
  }
}

/* crt.c:71-103 */
static void generate_p_primes(i64* p, size_t n, size_t bits, uint32_t N,
                              const i64* base, size_t nbase) {
  i64 order = 2 * (i64)N;
  i64 prev  = gen_first_prime(N, bits);
  for (size_t i = 0; i < n; i++) {
    i64 cand;
    int found;
    do {
      cand  = gen_previous_prime(prev, order);
      found = 0;
      for (size_t j = 0; j < nbase; j++)
        if (cand == base[j]) { found = 1; break; }
      prev = cand;
    } while (found);
    p[i] = cand;
  }
}

/* bit length of a product of primes (crt.c:445-450 BI_SIZE_INBASE) */
static size_t product_bits(const i64* primes, size_t n) {
  u64    w[64];
  size_t len = 1;
  w[0] = 1;
  for (size_t i = 0; i < n; i++) {
    u64 carry = 0;
    for (size_t j = 0; j < len; j++) {
      u128 t = (u128)w[j] * (u64)primes[i] + carry;
      w[j]   = (u64)t;
      carry  = (u64)(t >> 64);
    }
    if (carry) w[len++] = carry;
  }
  size_t bits = (len - 1) * 64;
  u64    top  = w[len - 1];
  while (top) { bits++; top >>= 1; }
  return bits;
}

/* Reverse_bits, util/include/bit_operation_impl.h:22-29 */
static inline u64 reverse_bits(u64 v, unsigned width) {
  u64 r = 0;
  for (unsigned i = 0; i < width; i++) { r = (r << 1) | (v & 1); v >>= 1; }
  return r;
}

/* util/src/ntt.c:34-138 Init_nttcontext + Precompute_ntt */
static void build_ntt_tables(orc_ctx* c, size_t idx) {
  uint32_t N = c->N;
  const modulus_t* m = &c->mod[idx];
  i64 q = m->val;
  c->ninv[idx]      = (u64)inv_prime(N, q);
  c->ninv_prec[idx] = orc_precompute_const(c->ninv[idx], q);
  i64 root     = orc_root_of_unity(2 * (i64)N, q);
  c->root[idx] = root;
  u64* rou  = c->rou + idx * N;
  u64* roui = c->rou_inv + idx * N;
  rou[0] = 1;
  i64 power = root;
  for (uint32_t i = 1; i < N; i++) {
    rou[reverse_bits(i, c->logN)] = (u64)power;
    power = mul_mod_barrett(power, root, m);
  }
  i64 root_inv = inv_prime(root, q);
  roui[0] = 1;
  power   = root_inv;
  for (uint32_t i = 1; i < N; i++) {
    roui[reverse_bits(i, c->logN)] = (u64)power;
    power = mul_mod_barrett(power, root_inv, m);
  }
  u64* roup  = c->rou_prec + idx * N;
  u64* rouip = c->rou_inv_prec + idx * N;
  for (uint32_t i = 0; i < N; i++) {
    roup[i]  = orc_precompute_const(rou[i], q);
    rouip[i] = orc_precompute_const(roui[i], q);
  }
}

static orc_ctx* ctx_finish(uint32_t N, size_t L, i64* q, size_t parts) {
  ORC_ASSERT(N >= 2 && (N & (N - 1)) == 0, "invalid poly degree");
  orc_ctx* c = (orc_ctx*)calloc(1, sizeof(orc_ctx));
  c->N = N;
  c->logN = 0;
  while ((1u << c->logN) < N) c->logN++;
  c->L = L;
  c->parts = parts;
  /* crt.c:422-457 Precompute_qpart */
  c->part_size = (L + parts - 1) / parts;
  ORC_ASSERT(L > c->part_size * (parts - 1), "invalid number of q parts");
  size_t max_bits = 0;
  for (size_t j = 0; j < parts; j++) {
    size_t lo = j * c->part_size, hi = lo + c->part_size;
    if (hi > L) hi = L;
    size_t bits = product_bits(q + lo, hi - lo);
    if (bits > max_bits) max_bits = bits;
  }
  c->K = (max_bits + 59) / 60; /* AUXBITS = 60, include/util/type.h:26-28 */
  size_t T = L + c->K;
  i64* all = (i64*)malloc(sizeof(i64) * T);
  memcpy(all, q, sizeof(i64) * L);
  generate_p_primes(all + L, c->K, 60, N, q, L);
  c->mod  = (modulus_t*)calloc(T, sizeof(modulus_t));
  c->root = (i64*)calloc(T, sizeof(i64));
  c->rou  = (u64*)malloc(sizeof(u64) * T * N);
  c->rou_prec     = (u64*)malloc(sizeof(u64) * T * N);
  c->rou_inv      = (u64*)malloc(sizeof(u64) * T * N);
  c->rou_inv_prec = (u64*)malloc(sizeof(u64) * T * N);
  c->ninv      = (u64*)calloc(T, sizeof(u64));
  c->ninv_prec = (u64*)calloc(T, sizeof(u64));
  for (size_t i = 0; i < T; i++) {
    init_modulus(&c->mod[i], all[i]);
    build_ntt_tables(c, i);
  }
  free(all);
  /* Precompute_fft (util/src/ntt.c:559-587) for fft_length = 2N */
  size_t M = 2 * (size_t)N;
  c->fft_rou = (double*)malloc(sizeof(double) * 2 * M);
  for (size_t i = 0; i < M; i++) {
    double angle = 2 * M_PI * i / M;
    c->fft_rou[2 * i] = cos(angle);
    c->fft_rou[2 * i + 1] = sin(angle);
  }
  size_t ns = M / 4;
  c->rot_group = (i64*)malloc(sizeof(i64) * (ns ? ns : 1));
  c->rot_group[0] = 1;
  for (size_t i = 1; i < ns; i++) c->rot_group[i] = (5 * c->rot_group[i - 1]) % (i64)M;
  return c;
}

orc_ctx* orc_ctx_create(uint32_t degree, size_t num_q, size_t q0_bits,
                        size_t sf_bits, size_t num_parts) {
  i64* q = (i64*)malloc(sizeof(i64) * num_q);
  generate_q_primes(q, num_q, q0_bits, sf_bits, degree);
  orc_ctx* c = ctx_finish(degree, num_q, q, num_parts);
  c->q0_bits = q0_bits;
  c->sf_bits = sf_bits;
  free(q);
  return c;
}

orc_ctx* orc_ctx_create_with_primes(uint32_t degree, size_t num_q,
                                    const int64_t* q, size_t num_parts) {
  i64* qq = (i64*)malloc(sizeof(i64) * num_q);
  memcpy(qq, q, sizeof(i64) * num_q);
  orc_ctx* c = ctx_finish(degree, num_q, qq, num_parts);
  free(qq);
  return c;
}

void orc_ctx_destroy(orc_ctx* c) {
  if (!c) return;
  free(c->mod); free(c->root); free(c->rou); free(c->rou_prec);
  free(c->rou_inv); free(c->rou_inv_prec); free(c->ninv); free(c->ninv_prec);
  free(c->fft_rou); free(c->rot_group);
  free(c);
}

uint32_t orc_degree(const orc_ctx* c) { return c->N; }
size_t   orc_num_q(const orc_ctx* c) { return c->L; }
size_t   orc_num_p(const orc_ctx* c) { return c->K; }
size_t   orc_num_parts(const orc_ctx* c) { return c->parts; }
size_t   orc_part_size(const orc_ctx* c) { return c->part_size; }
int64_t  orc_prime(const orc_ctx* c, size_t i) { return c->mod[i].val; }
int64_t  orc_root(const orc_ctx* c, size_t i) { return c->root[i]; }
void     orc_modulus(const orc_ctx* c, size_t i, uint64_t out[5]) {
  out[0] = (u64)c->mod[i].val;
  out[1] = (u64)c->mod[i].br_k;
  out[2] = (u64)c->mod[i].br_m;
  out[3] = (u64)c->mod[i].prec128;
  out[4] = (u64)(c->mod[i].prec128 >> 64);
}
const uint64_t* orc_twiddles(const orc_ctx* c, size_t i, int which) {
  const u64* t[4] = {c->rou, c->rou_prec, c->rou_inv, c->rou_inv_prec};
  return t[which] + i * c->N;
}

/* crt.c:1135-1144 */
size_t orc_num_decomp(const orc_ctx* c, size_t level) {
  size_t n = (level + c->part_size - 1) / c->part_size;
  return n > c->parts ? c->parts : n;
}

/* ---------------------------------------------------------------------- */
/* base-conversion tables                                                 */
/* ---------------------------------------------------------------------- */

/* product of primes[idx[t]] for t != skip, reduced mod m */
static i64 hat_mod(const orc_ctx* c, const size_t* idx, size_t n, size_t skip, i64 m) {
  i64 v = 1;
  for (size_t t = 0; t < n; t++) {
    if (t == skip) continue;
    v = mul_mod_exact(v, c->mod[idx[t]].val % m, m);
  }
  return v;
}

/* digit and complement prime indices at (level, part):
 * crt.c:503-533 (complement order) and rns_poly.c:173-183 (digit length) */
static void digit_layout(const orc_ctx* c, size_t level, size_t part,
                         size_t* dig, size_t* ndig, size_t* cmp, size_t* ncmp) {
  size_t nd = orc_num_decomp(c, level);
  ORC_ASSERT(part < nd, "digit index out of range");
  size_t start = c->part_size * part;
  size_t len   = (part == nd - 1) ? level - start : c->part_size;
  for (size_t i = 0; i < len; i++) dig[i] = start + i;
  size_t n = 0;
  for (size_t i = 0; i < level; i++)
    if (i < start || i >= start + len) cmp[n++] = i;
  for (size_t j = 0; j < c->K; j++) cmp[n++] = c->L + j;
  *ndig = len;
  *ncmp = n;
}

/* crt.c:470-497 (_l_hat_inv_modq) and :535-565 (_l_hat_modp) */
size_t orc_tbl_modup(const orc_ctx* c, size_t level, size_t part, int64_t* hat_inv,
                     int64_t* hat, int32_t* compl_idx, size_t* part_len_out) {
  size_t dig[64], cmp[128], nd, nc;
  digit_layout(c, level, part, dig, &nd, cmp, &nc);
  for (size_t i = 0; i < nd; i++) {
    i64 qi = c->mod[dig[i]].val;
    hat_inv[i] = inv_prime(hat_mod(c, dig, nd, i, qi), qi);
    for (size_t j = 0; j < nc; j++)
      hat[i * nc + j] = hat_mod(c, dig, nd, i, c->mod[cmp[j]].val);
  }
  for (size_t j = 0; j < nc; j++) compl_idx[j] = (int32_t)cmp[j];
  *part_len_out = nd;
  return nc;
}

/* crt.c:264-291 (P: _hat_inv_mod_self) and :354-420 (P -> Q tables) */
void orc_tbl_moddown(const orc_ctx* c, int64_t* phat_inv, int64_t* phat_modq,
                     int64_t* pinv_modq, int64_t* pmodq) {
  size_t pidx[64];
  for (size_t j = 0; j < c->K; j++) pidx[j] = c->L + j;
  for (size_t j = 0; j < c->K; j++) {
    i64 pj = c->mod[pidx[j]].val;
    phat_inv[j] = inv_prime(hat_mod(c, pidx, c->K, j, pj), pj);
  }
  for (size_t i = 0; i < c->L; i++) {
    i64 qi = c->mod[i].val;
    for (size_t j = 0; j < c->K; j++)
      phat_modq[i * c->K + j] = hat_mod(c, pidx, c->K, j, qi);
    i64 pm = hat_mod(c, pidx, c->K, (size_t)-1, qi);
    pmodq[i]     = pm;
    pinv_modq[i] = inv_prime(pm, qi);
  }
}

/* crt.c:299-349.  The reference value floor(H*(H^-1 mod q_l)/q_l) mod q_i,
 * H = (product of all Q primes)/q_l, equals -q_l^-1 mod q_i because q_i | H. */
void orc_tbl_rescale(const orc_ctx* c, size_t level, int64_t* ql_inv, int64_t* qlql) {
  ORC_ASSERT(level >= 2 && level <= c->L, "invalid rescale level");
  i64 ql = c->mod[level - 1].val;
  for (size_t i = 0; i + 1 < level; i++) {
    i64 qi = c->mod[i].val;
    i64 v  = inv_prime(ql % qi, qi);
    ql_inv[i] = v;
    qlql[i]   = qi - v;
  }
}

/* ---------------------------------------------------------------------- */
/* NTT, util/src/ntt.c                                                    */
/* ---------------------------------------------------------------------- */

/* ntt.c:167-241 Forward_transform: Cooley-Tukey, natural in, bit-reversed out */
static void forward_transform(const orc_ctx* c, size_t pi, u64* a) {
  const u64 q = (u64)c->mod[pi].val;
  const u64* rou  = c->rou + pi * c->N;
  const u64* roup = c->rou_prec + pi * c->N;
  uint32_t n = c->N >> 1, t = n;
  for (uint32_t m = 1; m < n; m <<= 1, t >>= 1) {
    for (uint32_t i = 0; i < m; i++) {
      u64 w = rou[i + m], wp = roup[i + m];
      uint32_t j1 = i * 2 * t, j2 = j1 + t;
      for (; j1 < j2; j1++) {
        u64 f  = (u64)shoup_mul(a[j1 + t], w, wp, q);
        u64 lo = a[j1];
        u64 hi = lo + f;
        if (hi >= q) hi -= q;
        if (lo < f) lo += q;
        a[j1]     = hi;
        a[j1 + t] = lo - f;
      }
    }
  }
  for (uint32_t i = 0; i < (n << 1); i += 2) {
    u64 w = rou[(i >> 1) + n], wp = roup[(i >> 1) + n];
    u64 f  = (u64)shoup_mul(a[i + 1], w, wp, q);
    u64 lo = a[i];
    u64 hi = lo + f;
    if (hi >= q) hi -= q;
    if (lo < f) lo += q;
    a[i]     = hi;
    a[i + 1] = lo - f;
  }
}

/* ntt.c:245-330 Inverse_transform: Gentleman-Sande, bit-reversed in, natural
 * out, 1/N applied to both outputs of the first stage */
static void inverse_transform(const orc_ctx* c, size_t pi, u64* a) {
  const u64 q = (u64)c->mod[pi].val;
  const u64* rou  = c->rou_inv + pi * c->N;
  const u64* roup = c->rou_inv_prec + pi * c->N;
  const u64 ni = c->ninv[pi], nip = c->ninv_prec[pi];
  uint32_t n = c->N;
  for (uint32_t i = 0; i < n; i += 2) {
    u64 w = rou[(i + n) >> 1], wp = roup[(i + n) >> 1];
    u64 hi = a[i + 1], lo = a[i];
    u64 f = lo;
    if (f < hi) f += q;
    f -= hi;
    lo += hi;
    if (lo >= q) lo -= q;
    lo = (u64)shoup_mul(lo, ni, nip, q);
    f  = (u64)shoup_mul(f, w, wp, q);
    f  = (u64)shoup_mul(f, ni, nip, q);
    a[i]     = lo;
    a[i + 1] = f;
  }
  uint32_t t = 2;
  for (uint32_t m = n >> 2; m >= 1; m >>= 1, t <<= 1) {
    for (uint32_t i = 0; i < m; i++) {
      u64 w = rou[i + m], wp = roup[i + m];
      uint32_t j1 = i * 2 * t, j2 = j1 + t;
      for (; j1 < j2; j1++) {
        u64 hi = a[j1 + t], lo = a[j1];
        u64 f = lo;
        if (f < hi) f += q;
        f -= hi;
        lo += hi;
        if (lo >= q) lo -= q;
        a[j1]     = lo;
        a[j1 + t] = (u64)shoup_mul(f, w, wp, q);
      }
    }
  }
}

void orc_ntt(const orc_ctx* c, int64_t* dst, const int64_t* src,
             const int32_t* prime_idx, size_t n_limbs) {
  for (size_t t = 0; t < n_limbs; t++) {
    if (dst != src) memcpy(dst + t * c->N, src + t * c->N, sizeof(i64) * c->N);
    forward_transform(c, (size_t)prime_idx[t], (u64*)dst + t * c->N);
  }
}
void orc_intt(const orc_ctx* c, int64_t* dst, const int64_t* src,
              const int32_t* prime_idx, size_t n_limbs) {
  for (size_t t = 0; t < n_limbs; t++) {
    if (dst != src) memcpy(dst + t * c->N, src + t * c->N, sizeof(i64) * c->N);
    inverse_transform(c, (size_t)prime_idx[t], (u64*)dst + t * c->N);
  }
}

/* ---------------------------------------------------------------------- */
/* per-limb vector ops, hal/src/hal.c                                     */
/* ---------------------------------------------------------------------- */

void orc_hw_modadd(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t idx, size_t n) {
  i64 q = c->mod[idx].val;
  for (size_t i = 0; i < n; i++) r[i] = orc_add_mod(a[i], b[i], q);
}
void orc_hw_modsub(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t idx, size_t n) {
  i64 q = c->mod[idx].val;
  for (size_t i = 0; i < n; i++) r[i] = orc_sub_mod(a[i], b[i], q);
}
void orc_hw_modmul(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t idx, size_t n) {
  const modulus_t* m = &c->mod[idx];
  for (size_t i = 0; i < n; i++) r[i] = mul_mod_barrett(a[i], b[i], m);
}
void orc_hw_modmuladd(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t idx, size_t n) {
  const modulus_t* m = &c->mod[idx];
  for (size_t i = 0; i < n; i++) r[i] = orc_add_mod(r[i], mul_mod_barrett(a[i], b[i], m), m->val);
}
void orc_hw_modadd_scalar(const orc_ctx* c, int64_t* r, const int64_t* a, int64_t s, size_t idx, size_t n) {
  i64 q = c->mod[idx].val;
  for (size_t i = 0; i < n; i++) r[i] = orc_add_mod(a[i], s, q);
}
void orc_hw_modsub_scalar(const orc_ctx* c, int64_t* r, const int64_t* a, int64_t s, size_t idx, size_t n) {
  i64 q = c->mod[idx].val;
  for (size_t i = 0; i < n; i++) r[i] = orc_sub_mod(a[i], s, q);
}
void orc_hw_modmul_scalar(const orc_ctx* c, int64_t* r, const int64_t* a, int64_t s, size_t idx, size_t n) {
  const modulus_t* m = &c->mod[idx];
  for (size_t i = 0; i < n; i++) r[i] = mul_mod_barrett(a[i], s, m);
}
void orc_hw_modmuladd_scalar(const orc_ctx* c, int64_t* r, const int64_t* a, int64_t s, size_t idx, size_t n) {
  const modulus_t* m = &c->mod[idx];
  for (size_t i = 0; i < n; i++) r[i] = orc_add_mod(r[i], mul_mod_barrett(a[i], s, m), m->val);
}
/* hal.c:123-138: a negative table entry means "negate the coefficient" */
void orc_hw_rotate(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* order, size_t idx, size_t n) {
  i64 q = c->mod[idx].val;
  for (size_t i = 0; i < n; i++) {
    i64 k = order[i];
    r[i] = k >= 0 ? a[k] : q - a[-k];
  }
}

/* ---------------------------------------------------------------------- */
/* automorphism tables, util/src/number_theory.c:192-231                  */
/* ---------------------------------------------------------------------- */

uint32_t orc_find_automorphism_index(int32_t rot_idx, uint32_t degree) {
  i64 m = 2 * (i64)degree;
  if (rot_idx == 0) return 1;
  if (rot_idx == (int32_t)(m - 1)) return (uint32_t)rot_idx;
  i64 gen = 5;
  if (rot_idx < 0) gen = orc_mod_inv(5, m);
  return (uint32_t)orc_mod_exp(gen, rot_idx < 0 ? -(i64)rot_idx : rot_idx, m);
}

void orc_automorphism_order(int64_t* order, uint32_t k, uint32_t n, int is_ntt) {
  u64 m = (u64)n << 1;
  unsigned logn = 0;
  while ((1u << logn) < n) logn++;
  if (is_ntt) {
    for (u64 j = 0; j < n; j++) {
      u64 jt  = (j << 1) + 1;
      u64 idx = ((jt * k) % m) >> 1;
      order[reverse_bits(j, logn)] = (i64)reverse_bits(idx, logn);
    }
  } else {
    for (u64 j = 0; j < n; j++) {
      u64 shift = (j * k) % m;
      if (shift < n) order[shift] = (i64)j;
      else           order[shift - n] = -(i64)j;
    }
  }
}

/* ---------------------------------------------------------------------- */
/* RNS polynomial ops, poly/src/rns_poly.c + rns_poly_impl.c              */
/* ---------------------------------------------------------------------- */

/* prime index of limb t of a polynomial at `level` with optional P part */
static inline size_t limb_prime(const orc_ctx* c, size_t level, size_t t) {
  return t < level ? t : c->L + (t - level);
}

/* rns_poly.c:74-105 */
size_t orc_decomp(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level, size_t part) {
  size_t nd = orc_num_decomp(c, level);
  ORC_ASSERT(part < nd, "digit index out of range");
  size_t start = c->part_size * part;
  size_t len   = (part == nd - 1) ? level - start : c->part_size;
  memcpy(out, in + start * c->N, sizeof(i64) * len * c->N);
  return len;
}

/* rns_poly_impl.c:341-378 Fast_base_conv_with_parts: src is the digit in
 * coefficient form, dst receives n_compl limbs */
static void base_conv_parts(const orc_ctx* c, i64* dst, const i64* src, size_t level, size_t part) {
  size_t N = c->N, nd, nc;
  i64 hat_inv[64];
  i64* hat = (i64*)malloc(sizeof(i64) * 64 * 128);
  int32_t cmp[128];
  nc = orc_tbl_modup(c, level, part, hat_inv, hat, cmp, &nd);
  size_t start = c->part_size * part;
  i128 sum[128];
  for (size_t n = 0; n < N; n++) {
    for (size_t j = 0; j < nc; j++) sum[j] = 0;
    for (size_t i = 0; i < nd; i++) {
      i64 t = mul_mod_barrett(src[i * N + n], hat_inv[i], &c->mod[start + i]);
      for (size_t j = 0; j < nc; j++) sum[j] += (i128)t * hat[i * nc + j];
    }
    for (size_t j = 0; j < nc; j++)
      dst[j * N + n] = barrett128((u128)sum[j], &c->mod[cmp[j]]);
  }
  free(hat);
}

/* rns_poly.c:107-158 Mod_up: INTT the digit (if NTT), convert, NTT the
 * converted limbs, then assemble [lower Q | digit | upper Q + P] */
void orc_mod_up(const orc_ctx* c, int64_t* out, const int64_t* digit, size_t digit_len, size_t level, size_t part, int is_ntt) {
  size_t N = c->N, dig[64], cmp[128], nd, nc;
  digit_layout(c, level, part, dig, &nd, cmp, &nc);
  ORC_ASSERT(nd == digit_len, "digit length does not match level/part");
  i64* coef = (i64*)malloc(sizeof(i64) * nd * N);
  i64* ext  = (i64*)malloc(sizeof(i64) * nc * N);
  int32_t pidx[128];
  memcpy(coef, digit, sizeof(i64) * nd * N);
  if (is_ntt) {
    for (size_t i = 0; i < nd; i++) pidx[i] = (int32_t)dig[i];
    orc_intt(c, coef, coef, pidx, nd);
  }
  base_conv_parts(c, ext, coef, level, part);
  if (is_ntt) {
    for (size_t j = 0; j < nc; j++) pidx[j] = (int32_t)cmp[j];
    orc_ntt(c, ext, ext, pidx, nc);
  }
  size_t start = c->part_size * part, end = start + nd;
  memcpy(out, ext, sizeof(i64) * N * start);
  memcpy(out + start * N, digit, sizeof(i64) * N * nd);
  memcpy(out + end * N, ext + start * N, sizeof(i64) * N * (level + c->K - end));
  free(coef);
  free(ext);
}

/* rns_poly.c:160-258 Decomp_modup: same result written in place, the
 * per-coefficient accumulation order of the reference is kept */
void orc_decomp_modup(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level, size_t part, int is_ntt) {
  size_t N = c->N, dig[64], cmp[128], nd, nc;
  digit_layout(c, level, part, dig, &nd, cmp, &nc);
  size_t n1 = c->part_size * part, p3 = n1 + nd, n3 = level + c->K - p3;
  memcpy(out + n1 * N, in + n1 * N, sizeof(i64) * nd * N);
  i64* coef = (i64*)malloc(sizeof(i64) * nd * N);
  int32_t pidx[128];
  memcpy(coef, in + n1 * N, sizeof(i64) * nd * N);
  if (is_ntt) {
    for (size_t i = 0; i < nd; i++) pidx[i] = (int32_t)dig[i];
    orc_intt(c, coef, coef, pidx, nd);
  }
  i64 hat_inv[64];
  i64* hat = (i64*)malloc(sizeof(i64) * 64 * 128);
  int32_t ci[128];
  size_t nd2;
  orc_tbl_modup(c, level, part, hat_inv, hat, ci, &nd2);
  i128 sum[128];
  for (size_t n = 0; n < N; n++) {
    for (size_t j = 0; j < nc; j++) sum[j] = 0;
    for (size_t i = 0; i < nd; i++) {
      i64 t = mul_mod_barrett(coef[i * N + n], hat_inv[i], &c->mod[dig[i]]);
      for (size_t j = 0; j < nc; j++) sum[j] += (i128)t * hat[i * nc + j];
    }
    for (size_t j = 0; j < n1; j++)
      out[j * N + n] = barrett128((u128)sum[j], &c->mod[cmp[j]]);
    for (size_t j1 = 0, j2 = n1; j1 < n3; j1++, j2++)
      out[(j1 + p3) * N + n] = barrett128((u128)sum[j2], &c->mod[cmp[j2]]);
  }
  if (is_ntt) {
    for (size_t j = 0; j < n1; j++) pidx[j] = (int32_t)cmp[j];
    orc_ntt(c, out, out, pidx, n1);
    for (size_t j = 0; j < n3; j++) pidx[j] = (int32_t)cmp[n1 + j];
    orc_ntt(c, out + p3 * N, out + p3 * N, pidx, n3);
  }
  free(coef);
  free(hat);
}

/* rns_poly.c:416-481 Precomp / Alloc_precomp */
void orc_precomp(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level, int is_ntt, int fused) {
  size_t nd = orc_num_decomp(c, level), stride = (level + c->K) * c->N;
  i64* tmp = fused ? NULL : (i64*)malloc(sizeof(i64) * c->part_size * c->N);
  for (size_t part = 0; part < nd; part++) {
    if (fused) {
      orc_decomp_modup(c, out + part * stride, in, level, part, is_ntt);
    } else {
      size_t len = orc_decomp(c, tmp, in, level, part);
      orc_mod_up(c, out + part * stride, tmp, len, level, part, is_ntt);
    }
  }
  free(tmp);
}

/* rns_poly_impl.c:287-339 Fast_base_conv, P -> Q (src: K limbs, coefficient
 * form; dst: level limbs) */
static void base_conv_p2q(const orc_ctx* c, i64* dst, const i64* src, size_t level) {
  size_t N = c->N, K = c->K;
  i64* phat_inv = (i64*)malloc(sizeof(i64) * K);
  i64* phat     = (i64*)malloc(sizeof(i64) * c->L * K);
  i64* pinv     = (i64*)malloc(sizeof(i64) * c->L);
  i64* pmod     = (i64*)malloc(sizeof(i64) * c->L);
  orc_tbl_moddown(c, phat_inv, phat, pinv, pmod);
  i64* t = (i64*)malloc(sizeof(i64) * K * N);
  for (size_t j = 0; j < K; j++) {
    u64 pj = (u64)c->mod[c->L + j].val;
    u64 w = (u64)phat_inv[j], wp = orc_precompute_const(w, pj);
    for (size_t n = 0; n < N; n++) t[j * N + n] = shoup_mul((u64)src[j * N + n], w, wp, pj);
  }
  for (size_t i = 0; i < level; i++) {
    for (size_t n = 0; n < N; n++) {
      i128 sum = 0;
      for (size_t j = 0; j < K; j++) sum += (i128)t[j * N + n] * phat[i * K + j];
      dst[i * N + n] = barrett128((u128)sum, &c->mod[i]);
    }
  }
  free(phat_inv); free(phat); free(pinv); free(pmod); free(t);
}

/* rns_poly.c:260-308 */
void orc_mod_down(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level, int is_ntt) {
  size_t N = c->N, K = c->K;
  i64* p = (i64*)malloc(sizeof(i64) * K * N);
  memcpy(p, in + level * N, sizeof(i64) * K * N);
  int32_t pidx[128];
  if (is_ntt) {
    for (size_t j = 0; j < K; j++) pidx[j] = (int32_t)(c->L + j);
    orc_intt(c, p, p, pidx, K);
  }
  base_conv_p2q(c, out, p, level);
  if (is_ntt) {
    for (size_t i = 0; i < level; i++) pidx[i] = (int32_t)i;
    orc_ntt(c, out, out, pidx, level);
  }
  i64* phat_inv = (i64*)malloc(sizeof(i64) * K);
  i64* phat     = (i64*)malloc(sizeof(i64) * c->L * K);
  i64* pinv     = (i64*)malloc(sizeof(i64) * c->L);
  i64* pmod     = (i64*)malloc(sizeof(i64) * c->L);
  orc_tbl_moddown(c, phat_inv, phat, pinv, pmod);
  for (size_t i = 0; i < level; i++) {
    const modulus_t* m = &c->mod[i];
    for (size_t n = 0; n < N; n++) {
      i64 v = orc_sub_mod(in[i * N + n], out[i * N + n], m->val);
      out[i * N + n] = mul_mod_barrett(v, pinv[i], m);
    }
  }
  free(p); free(phat_inv); free(phat); free(pinv); free(pmod);
}

/* rns_poly.c:310-404 */
void orc_rescale(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level, int is_ntt) {
  ORC_ASSERT(level >= 2, "Level of rescale opnd is too small");
  size_t N = c->N;
  i64 ql_inv[64], qlql[64];
  orc_tbl_rescale(c, level, ql_inv, qlql);
  i64 last_mod = c->mod[level - 1].val;
  if (is_ntt) {
    i64* last = (i64*)malloc(sizeof(i64) * N);
    i64* tmp  = (i64*)malloc(sizeof(i64) * N);
    int32_t pi = (int32_t)(level - 1);
    orc_intt(c, last, in + (level - 1) * N, &pi, 1);
    for (size_t i = 0; i + 1 < level; i++) {
      u64 q = (u64)c->mod[i].val;
      u64 kq = (u64)qlql[i], kqp = orc_precompute_const(kq, q);
      u64 iv = (u64)ql_inv[i], ivp = orc_precompute_const(iv, q);
      for (size_t n = 0; n < N; n++)
        tmp[n] = shoup_mul((u64)orc_switch_modulus(last[n], last_mod, (i64)q), kq, kqp, q);
      pi = (int32_t)i;
      orc_ntt(c, tmp, tmp, &pi, 1);
      for (size_t n = 0; n < N; n++) {
        i64 v = shoup_mul((u64)in[i * N + n], iv, ivp, q);
        out[i * N + n] = orc_add_mod(v, tmp[n], (i64)q);
      }
    }
    free(last);
    free(tmp);
  } else {
    const i64* last = in + (level - 1) * N;
    for (size_t i = 0; i + 1 < level; i++) {
      const modulus_t* m = &c->mod[i];
      u64 q = (u64)m->val;
      u64 iv = (u64)ql_inv[i], ivp = orc_precompute_const(iv, q);
      for (size_t n = 0; n < N; n++) {
        i64 lc = barrett64(last[n], m);
        i64 v  = orc_sub_mod(in[i * N + n], lc, m->val);
        out[i * N + n] = shoup_mul((u64)v, iv, ivp, q);
      }
    }
  }
}

/* modular.h:262-276 Sub_mul_const_mod, literally: ((v1 - v2) * w) mod q with a
 * Shoup constant, one conditional +q after the subtraction.  When v2 exceeds
 * v1 + q (possible where v2 is a residue of a LARGER prime, as in
 * Mod_down_rescale) the difference stays negative and the reference's casts
 * decide the value; they are reproduced here: (UINT128_T)int64 sign-extends,
 * int64 * uint64 wraps modulo 2^64. */
static inline i64 sub_mul_const(u64 v1, u64 v2, u64 w, u64 wp, u64 q) {
  i64 s = (i64)v1 - (i64)v2;
  if (s < 0) s += (i64)q;
  u64 qq = (u64)(((u128)(i128)s * wp) >> 64);
  u64 y  = ((u64)s * w) - qq * q;
  return (i64)(y >= q ? y - q : y);
}
int64_t orc_sub_mul_const(uint64_t v1, uint64_t v2, uint64_t w, uint64_t wp, uint64_t q) {
  return sub_mul_const(v1, v2, w, wp, q);
}

/* shared front of Mod_down_rescale (rns_poly.c:531-597) and
 * Reduce_and_rescale_modup (rns_poly_impl.c:521-620): the input is brought to
 * coefficient form IN PLACE (all level+K limbs), its P part is converted to the
 * Q basis into y, and limb level-1 of y becomes (old - y) * P^-1 mod q_last. */
static void moddown_rescale_front(const orc_ctx* c, i64* y, i64* poly, size_t level, int is_ntt) {
  size_t N = c->N, K = c->K;
  int32_t idx[128];
  if (is_ntt) {
    for (size_t i = 0; i < level; i++) idx[i] = (int32_t)i;
    for (size_t j = 0; j < K; j++) idx[level + j] = (int32_t)(c->L + j);
    orc_intt(c, poly, poly, idx, level + K);
  }
  base_conv_p2q(c, y, poly + level * N, level);
  i64* phat_inv = (i64*)malloc(sizeof(i64) * K);
  i64* phat     = (i64*)malloc(sizeof(i64) * c->L * K);
  i64* pinv     = (i64*)malloc(sizeof(i64) * c->L);
  i64* pmod     = (i64*)malloc(sizeof(i64) * c->L);
  orc_tbl_moddown(c, phat_inv, phat, pinv, pmod);
  size_t last = level - 1;
  u64 ql = (u64)c->mod[last].val, w = (u64)pinv[last], wp = orc_precompute_const(w, ql);
  for (size_t n = 0; n < N; n++)
    y[last * N + n] = sub_mul_const((u64)poly[last * N + n], (u64)y[last * N + n], w, wp, ql);
  free(phat_inv); free(phat); free(pinv); free(pmod);
}

/* value of limb i < level-1 after the fused Mod_down and rescale */
static void moddown_rescale_limb(const orc_ctx* c, i64* dst, const i64* poly, const i64* y, size_t level, size_t i) {
  size_t N = c->N, last = level - 1;
  i64 ql_inv[64], qlql[64];
  orc_tbl_rescale(c, level, ql_inv, qlql);
  i64* phat_inv = (i64*)malloc(sizeof(i64) * c->K);
  i64* phat     = (i64*)malloc(sizeof(i64) * c->L * c->K);
  i64* pinv     = (i64*)malloc(sizeof(i64) * c->L);
  i64* pmod     = (i64*)malloc(sizeof(i64) * c->L);
  orc_tbl_moddown(c, phat_inv, phat, pinv, pmod);
  u64 q = (u64)c->mod[i].val;
  u64 w = (u64)pinv[i], wp = orc_precompute_const(w, q);
  u64 v = (u64)ql_inv[i], vp = orc_precompute_const(v, q);
  for (size_t n = 0; n < N; n++) {
    i64 t = sub_mul_const((u64)poly[i * N + n], (u64)y[i * N + n], w, wp, q);
    dst[n] = sub_mul_const((u64)t, (u64)y[last * N + n], v, vp, q);
  }
  free(phat_inv); free(phat); free(pinv); free(pmod);
}

/* rns_poly.c:531-597.  poly: (level+K) limbs, converted to coefficient form in
 * place (the reference does the same to its argument); out: level-1 limbs, NTT form. */
void orc_mod_down_rescale(const orc_ctx* c, int64_t* out, int64_t* poly, size_t level, int is_ntt) {
  ORC_ASSERT(level >= 2, "Mod_down_rescale: level too small");
  size_t N = c->N;
  i64* y = (i64*)malloc(sizeof(i64) * level * N);
  moddown_rescale_front(c, y, poly, level, is_ntt);
  for (size_t i = 0; i + 1 < level; i++) moddown_rescale_limb(c, out + i * N, poly, y, level, i);
  int32_t idx[128];
  for (size_t i = 0; i + 1 < level; i++) idx[i] = (int32_t)i;
  orc_ntt(c, out, out, idx, level - 1);
  free(y);
}

/* rns_poly_impl.c:521-620.  res: level limbs as the reference leaves them (the
 * converted P part in limbs 0..level-2, the reduced last limb in limb level-1;
 * its level is then lowered by one).  raised: num_decomp(level-1) polynomials
 * of (level-1+K) limbs, coefficient form: the rescaled value in each digit's
 * own limbs, its base conversion (Modup_inplace, rns_poly_impl.c:380-434) elsewhere. */
void orc_reduce_rescale_modup(const orc_ctx* c, int64_t* res, int64_t* raised, int64_t* poly, size_t level, int is_ntt) {
  ORC_ASSERT(level >= 2, "Reduce_and_rescale_modup: level too small");
  size_t N = c->N, nl = level - 1;
  moddown_rescale_front(c, res, poly, level, is_ntt);
  i64* x = (i64*)malloc(sizeof(i64) * nl * N);
  for (size_t i = 0; i < nl; i++) moddown_rescale_limb(c, x + i * N, poly, res, level, i);
  orc_precomp(c, raised, x, nl, 0, 1);
  free(x);
}

/* rns_poly.c:1101-1125: limb 0 copied, limb i = Switch_modulus(limb 0, q_0 -> q_i) */
void orc_transform_from_level0(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level) {
  size_t N = c->N;
  memcpy(out, in, sizeof(i64) * N);
  for (size_t i = 1; i < level; i++)
    for (size_t n = 0; n < N; n++) out[i * N + n] = orc_switch_modulus(in[n], c->mod[0].val, c->mod[i].val);
}

/* rns_poly.c:483-500 */
void orc_extend(const orc_ctx* c, int64_t* out, const int64_t* in, size_t level) {
  size_t N = c->N, K = c->K;
  i64* phat_inv = (i64*)malloc(sizeof(i64) * K);
  i64* phat     = (i64*)malloc(sizeof(i64) * c->L * K);
  i64* pinv     = (i64*)malloc(sizeof(i64) * c->L);
  i64* pmod     = (i64*)malloc(sizeof(i64) * c->L);
  orc_tbl_moddown(c, phat_inv, phat, pinv, pmod);
  memset(out, 0, sizeof(i64) * (level + K) * N);
  for (size_t i = 0; i < level; i++)
    for (size_t n = 0; n < N; n++)
      out[i * N + n] = mul_mod_barrett(in[i * N + n], pmod[i], &c->mod[i]);
  free(phat_inv); free(phat); free(pinv); free(pmod);
}

/* rns_poly.c:502-529 with rns_poly_impl.c:102-162 */
void orc_dot_prod(const orc_ctx* c, int64_t* out, const int64_t* digits, const int64_t* key, size_t key_stride, size_t n_parts, size_t level, int fast) {
  size_t N = c->N, T = level + c->K, dstride = T * N;
  for (size_t t = 0; t < T; t++) {
    size_t pi = limb_prime(c, level, t);
    size_t koff = (t < level ? t : c->L + (t - level)) * N;
    const modulus_t* m = &c->mod[pi];
    for (size_t n = 0; n < N; n++) {
      if (fast) {
        u128 acc = 0;
        for (size_t d = 0; d < n_parts; d++)
          acc += (u128)(u64)digits[d * dstride + t * N + n] * (u64)key[d * key_stride + koff + n];
        out[t * N + n] = barrett128(acc, m);
      } else {
        i64 acc = 0;
        for (size_t d = 0; d < n_parts; d++)
          acc = orc_add_mod(acc, mul_mod_barrett(digits[d * dstride + t * N + n], key[d * key_stride + koff + n], m), m->val);
        out[t * N + n] = acc;
      }
    }
  }
}

/* rns_poly.c:852-1010 */
void orc_poly_add(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p) {
  size_t T = level + (with_p ? c->K : 0);
  for (size_t t = 0; t < T; t++)
    orc_hw_modadd(c, r + t * c->N, a + t * c->N, b + t * c->N, limb_prime(c, level, t), c->N);
}
void orc_poly_sub(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p) {
  size_t T = level + (with_p ? c->K : 0);
  for (size_t t = 0; t < T; t++)
    orc_hw_modsub(c, r + t * c->N, a + t * c->N, b + t * c->N, limb_prime(c, level, t), c->N);
}
void orc_poly_mul(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p) {
  size_t T = level + (with_p ? c->K : 0);
  for (size_t t = 0; t < T; t++)
    orc_hw_modmul(c, r + t * c->N, a + t * c->N, b + t * c->N, limb_prime(c, level, t), c->N);
}
/* rns_poly.c:1056-1099 */
void orc_poly_automorphism(const orc_ctx* c, int64_t* r, const int64_t* a, const int64_t* order, size_t level, int with_p) {
  size_t T = level + (with_p ? c->K : 0);
  for (size_t t = 0; t < T; t++)
    orc_hw_rotate(c, r + t * c->N, a + t * c->N, order, limb_prime(c, level, t), c->N);
}

/* ---------------------------------------------------------------------- */
/* ciphertext level, ckks/src/evaluator.c                                 */
/* ---------------------------------------------------------------------- */

/* evaluator.c:142-175 */
void orc_mul_ciph3(const orc_ctx* c, int64_t* d0, int64_t* d1, int64_t* d2, const int64_t* a0, const int64_t* a1, const int64_t* b0, const int64_t* b1, size_t level) {
  size_t n = level * c->N;
  i64* tmp = (i64*)malloc(sizeof(i64) * n);
  orc_poly_mul(c, d0, a0, b0, level, 0);
  orc_poly_mul(c, d1, a0, b1, level, 0);
  orc_poly_mul(c, tmp, a1, b0, level, 0);
  orc_poly_add(c, d1, d1, tmp, level, 0);
  orc_poly_mul(c, d2, a1, b1, level, 0);
  free(tmp);
}

/* evaluator.c:411-462: inner product with both key halves, then Mod_down */
void orc_fast_switch_key(const orc_ctx* c, int64_t* out0, int64_t* out1, const int64_t* digits, const int64_t* swk, size_t level) {
  size_t N = c->N, T = level + c->K, kpoly = (c->L + c->K) * N;
  size_t nd = orc_num_decomp(c, level);
  i64* e0 = (i64*)malloc(sizeof(i64) * T * N);
  i64* e1 = (i64*)malloc(sizeof(i64) * T * N);
  orc_dot_prod(c, e0, digits, swk, 2 * kpoly, nd, level, 0);
  orc_dot_prod(c, e1, digits, swk + kpoly, 2 * kpoly, nd, level, 0);
  orc_mod_down(c, out0, e0, level, 1);
  orc_mod_down(c, out1, e1, level, 1);
  free(e0);
  free(e1);
}

/* evaluator.c:288-306 */
void orc_relin(const orc_ctx* c, int64_t* r0, int64_t* r1, const int64_t* d0, const int64_t* d1, const int64_t* d2, const int64_t* swk, size_t level) {
  size_t N = c->N, T = level + c->K, nd = orc_num_decomp(c, level);
  i64* digits = (i64*)malloc(sizeof(i64) * nd * T * N);
  orc_precomp(c, digits, d2, level, 1, 1);
  orc_fast_switch_key(c, r0, r1, digits, swk, level);
  orc_poly_add(c, r0, r0, d0, level, 0);
  orc_poly_add(c, r1, r1, d1, level, 0);
  free(digits);
}

/* evaluator.c:342-362 */
void orc_rescale_ciph(const orc_ctx* c, int64_t* r0, int64_t* r1, const int64_t* c0, const int64_t* c1, size_t level) {
  orc_rescale(c, r0, c0, level, 1);
  orc_rescale(c, r1, c1, level, 1);
}

/* evaluator.c:503-522 with :488-501 */
void orc_fast_rotate(const orc_ctx* c, int64_t* r0, int64_t* r1, const int64_t* c0, const int64_t* digits, const int64_t* swk, const int64_t* order, size_t level) {
  size_t n = level * c->N;
  i64* t0 = (i64*)malloc(sizeof(i64) * n);
  i64* t1 = (i64*)malloc(sizeof(i64) * n);
  orc_fast_switch_key(c, t0, t1, digits, swk, level);
  orc_poly_add(c, t0, t0, c0, level, 0);
  orc_poly_automorphism(c, r0, t0, order, level, 0);
  orc_poly_automorphism(c, r1, t1, order, level, 0);
  free(t0);
  free(t1);
}

/* evaluator.c:177-190 followed by :342-362 */
void orc_mul_relin_rescale(const orc_ctx* c, int64_t* r0, int64_t* r1, const int64_t* a0, const int64_t* a1, const int64_t* b0, const int64_t* b1, const int64_t* swk, size_t level) {
  size_t n = level * c->N;
  i64* d = (i64*)malloc(sizeof(i64) * n * 5);
  orc_mul_ciph3(c, d, d + n, d + 2 * n, a0, a1, b0, b1, level);
  orc_relin(c, d + 3 * n, d + 4 * n, d, d + n, d + 2 * n, swk, level);
  orc_rescale_ciph(c, r0, r1, d + 3 * n, d + 4 * n, level);
  free(d);
}

/* ---------------------------------------------------------------------- */
/* encoder: ckks/src/encoder.c, util/src/ntt.c:598-675                     */
/* ---------------------------------------------------------------------- */

#include <complex.h>
typedef double complex dcmplx;

static dcmplx fft_rou_at(const orc_ctx* c, size_t i) { return c->fft_rou[2 * i] + c->fft_rou[2 * i + 1] * I; }

/* Embedding_inv (ntt.c:631-675): the special inverse FFT over `len` slots */
static void embedding_inv(const orc_ctx* c, dcmplx* res, const dcmplx* coeffs, size_t len) {
  size_t M = 2 * (size_t)c->N;
  dcmplx* r = (dcmplx*)malloc(sizeof(dcmplx) * len);
  memcpy(r, coeffs, sizeof(dcmplx) * len);
  size_t logn = 0;
  while (((size_t)1 << logn) < len) logn++;
  for (size_t logm = logn; logm > 0; logm--) {
    size_t idx_mod = (size_t)1 << (logm + 2), gap = M / idx_mod, num1 = (size_t)1 << logm, num2 = num1 >> 1;
    for (size_t j = 0; j < len; j += num1) {
      for (size_t i = 0; i < num2; i++) {
        size_t ie = j + i, io = j + i + num2;
        size_t rou_idx = (idx_mod - ((size_t)c->rot_group[i] % idx_mod)) * gap;
        dcmplx plus = r[ie] + r[io], minus = r[ie] - r[io];
        minus *= fft_rou_at(c, rou_idx);
        r[ie] = plus;
        r[io] = minus;
      }
    }
  }
  for (size_t i = 0; i < len; i++) res[i] = r[reverse_bits(i, (unsigned)logn)];
  free(r);
  for (size_t i = 0; i < len; i++) res[i] /= len;
}

/* Embedding (ntt.c:598-629) */
static void embedding(const orc_ctx* c, dcmplx* res, const dcmplx* coeffs, size_t len) {
  size_t M = 2 * (size_t)c->N;
  size_t logn = 0;
  while (((size_t)1 << logn) < len) logn++;
  for (size_t i = 0; i < len; i++) res[i] = coeffs[reverse_bits(i, (unsigned)logn)];
  for (size_t logm = 1; logm < logn + 1; logm++) {
    size_t idx_mod = (size_t)1 << (logm + 2), gap = M / idx_mod, num = (size_t)1 << (logm - 1);
    for (size_t j = 0; j < len; j += (size_t)1 << logm) {
      for (size_t i = 0; i < num; i++) {
        size_t ie = j + i, io = j + i + num;
        size_t rou_idx = ((size_t)c->rot_group[i] % idx_mod) * gap;
        dcmplx om = fft_rou_at(c, rou_idx) * res[io];
        dcmplx plus = res[ie] + om, minus = res[ie] - om;
        res[ie] = plus;
        res[io] = minus;
      }
    }
  }
}

const double* orc_fft_rou(const orc_ctx* c) { return c->fft_rou; }

void orc_embedding(const orc_ctx* c, double* res, const double* coeffs, size_t len, int inverse) {
  if (inverse) embedding_inv(c, (dcmplx*)res, (const dcmplx*)coeffs, len);
  else embedding(c, (dcmplx*)res, (const dcmplx*)coeffs, len);
}

static i64 max_64bit_value(void) { return (i64)(((u64)1 << 63) - ((u64)1 << 9)) - 1; } /* modular.h:279-281 */
static i64 mod_int64(i64 v, i64 m) { i64 r = v % m; return r < 0 ? r + m : r; }        /* modular.h:85-92 */

/* Encode_impl (encoder.c:234-326), 64-bit build.  values: n_values complex numbers
 * (re, im interleaved); out: level Q limbs followed by p_cnt P limbs, NTT form.
 * Returns 1, or 0 where the reference asserts (vector out of range / overflow). */
static int encode_either(const orc_ctx* c, int64_t* out, const double* values, size_t n_values, uint32_t slots,
                         size_t level, uint32_t sf_degree, size_t p_cnt, double explicit_scale);
int orc_encode(const orc_ctx* c, int64_t* out, const double* values, size_t n_values, uint32_t slots, size_t level,
               uint32_t sf_degree, size_t p_cnt) {
  return encode_either(c, out, values, n_values, slots, level, sf_degree, p_cnt, 0.0);
}
/* Encode_impl_with_scale (encoder.c:337-403): the same steps with one multiplication by `scale`, rounded by
 * llround without the half that Encode_impl adds first, no range assertion on the rounded value and no
 * further powers of the scaling factor */
int orc_encode_scaled(const orc_ctx* c, int64_t* out, const double* values, size_t n_values, uint32_t slots,
                      size_t level, double scale, size_t p_cnt) {
  ORC_ASSERT(scale > 0, "invalid scale for encode");
  return encode_either(c, out, values, n_values, slots, level, 1, p_cnt, scale);
}
static int encode_either(const orc_ctx* c, int64_t* out, const double* values, size_t n_values, uint32_t slots,
                         size_t level, uint32_t sf_degree, size_t p_cnt, double explicit_scale) {
  ORC_ASSERT(c->sf_bits, "context has no scaling factor");
  size_t N = c->N;
  double scaling_factor = (double)((u64)1 << c->sf_bits); /* param.c:68 */
  if (!slots) slots = (uint32_t)(N / 2);
  if (!level) level = c->L;
  ORC_ASSERT(level <= c->L && n_values <= slots && slots <= N / 2, "encode: bad sizes");
  uint32_t sf_bits = (uint32_t)log2(scaling_factor);
  size_t coeff_bits = c->q0_bits + (level - 1) * c->sf_bits; /* Get_coeff_bit_count */
  double scale = pow(scaling_factor, sf_degree);
  if (explicit_scale > 0) {
    ORC_ASSERT((uint32_t)log2(explicit_scale) < coeff_bits, "invalid scale for encode");
    scale = explicit_scale;
  } else {
    ORC_ASSERT(sf_degree >= 1 && (size_t)sf_bits * sf_degree < coeff_bits, "invalid scaling factor for encode");
  }
  /* Transform_msg_within_range (encoder.c:198-231) */
  dcmplx* in = (dcmplx*)calloc(slots, sizeof(dcmplx));
  dcmplx* ts = (dcmplx*)calloc(slots, sizeof(dcmplx));
  for (size_t i = 0; i < n_values; i++) in[i] = values[2 * i] + values[2 * i + 1] * I;
  embedding_inv(c, ts, in, slots);
  double max_coeff = 0.0;
  for (uint32_t i = 0; i < slots; i++) {
    double a = fabs(creal(ts[i]) * scale), b = fabs(cimag(ts[i]) * scale);
    if (a > max_coeff) max_coeff = a;
    if (b > max_coeff) max_coeff = b;
  }
  int32_t bits = (int32_t)(log2(fmax(max_coeff, __DBL_MIN__))) + 1;
  int32_t valid = (int32_t)c->q0_bits + (int32_t)(level - 1) * (int32_t)sf_bits; /* Check_msg_range (:48-59) */
  int ok = bits < valid;
  i64* message = (i64*)calloc(N, sizeof(i64));
  uint32_t gap = (uint32_t)(N / (slots * 2));
  for (uint32_t i = 0; ok && i < slots; i++) {
    double re, im;
    if (explicit_scale > 0) re = creal(ts[i]) * scale, im = cimag(ts[i]) * scale;
    else re = creal(ts[i]) * scaling_factor + 0.5, im = cimag(ts[i]) * scaling_factor + 0.5;
    if (!(re <= (double)INT64_MAX && re >= -(double)INT64_MAX && im <= (double)INT64_MAX && im >= -(double)INT64_MAX)) {
      ok = 0;
      break;
    }
    i64 r = llround(re), m = llround(im);
    message[(size_t)i * gap] = r < 0 ? max_64bit_value() + r : r;
    message[((size_t)i + slots) * gap] = m < 0 ? max_64bit_value() + m : m;
  }
  if (ok) {
    /* Transform_values_to_dcrt (crt.c:1153-1184), I64 values, with modulus */
    i64 big_bound = max_64bit_value(), big_half = big_bound >> 1;
    for (size_t t = 0; t < level + p_cnt; t++) {
      size_t pi = t < level ? t : c->L + (t - level);
      i64 q = c->mod[pi].val, diff = big_bound - q;
      for (size_t n = 0; n < N; n++) {
        i64 v = message[n];
        out[t * N + n] = v > big_half ? mod_int64(v - diff, q) : mod_int64(v, q);
      }
    }
    if (sf_degree > 1 && !(explicit_scale > 0)) { /* encoder.c:297-312: only the Q limbs */
      for (size_t t = 0; t < level; t++) {
        i64 q = c->mod[t].val, powp = (i64)scaling_factor;
        for (uint32_t d = 2; d < sf_degree; d++) powp = mul_mod_exact(powp, (i64)scaling_factor, q);
        for (size_t n = 0; n < N; n++) out[t * N + n] = mul_mod_exact(out[t * N + n], powp, q);
      }
    }
    int32_t idx[128];
    for (size_t t = 0; t < level + p_cnt; t++) idx[t] = (int32_t)(t < level ? t : c->L + (t - level));
    orc_ntt(c, out, out, idx, level + p_cnt);
  }
  free(in); free(ts); free(message);
  return ok;
}

/* Reconstruct (crt.c:1247-1275) + mpz_get_d: the centred integer with residues
 * v[0..level) as a double, truncated towards zero like mpz_get_d.  Garner's
 * mixed-radix digits, then exact evaluation in a little-endian multi-word integer. */
static double crt_to_double(const orc_ctx* c, const i64* v, size_t level) {
  i64 d[64];
  /* mixed radix: x = d0 + d1 q0 + d2 q0 q1 + ... */
  for (size_t i = 0; i < level; i++) {
    i64 q = c->mod[i].val, t = v[i] % q, prod = 1;
    /* t = (v_i - (d0 + d1 q0 + ...)) / (q0..q_{i-1}) mod q_i */
    i64 acc = 0;
    for (size_t j = 0; j < i; j++) {
      acc = orc_add_mod(acc, mul_mod_exact(d[j] % q, prod, q), q);
      prod = mul_mod_exact(prod, c->mod[j].val % q, q);
    }
    t = orc_sub_mod(t, acc, q);
    d[i] = i ? mul_mod_exact(t, inv_prime(prod, q), q) : t;
  }
  /* exact value and Q as multi-word integers */
  u64 x[66] = {0}, Q[66] = {0};
  size_t nx = 1, nQ = 1;
  Q[0] = 1;
  for (size_t i = level; i-- > 0;) { /* Horner from the top digit */
    u128 carry = 0;
    for (size_t k = 0; k < nx; k++) { u128 p = (u128)x[k] * (u64)c->mod[i].val + carry; x[k] = (u64)p; carry = p >> 64; }
    if (carry) x[nx++] = (u64)carry;
    u128 a = (u128)x[0] + (u64)d[i];
    x[0] = (u64)a;
    for (size_t k = 1; (a >> 64) && k <= nx; k++) { a = (u128)x[k] + 1; x[k] = (u64)a; if (k == nx) nx++; }
  }
  for (size_t i = 0; i < level; i++) {
    u128 carry = 0;
    for (size_t k = 0; k < nQ; k++) { u128 p = (u128)Q[k] * (u64)c->mod[i].val + carry; Q[k] = (u64)p; carry = p >> 64; }
    if (carry) Q[nQ++] = (u64)carry;
  }
  size_t n = nQ > nx ? nQ : nx;
  /* negative when x > floor(Q/2), i.e. 2x > Q (Q is odd) */
  u64 x2[67] = {0};
  for (size_t k = 0; k < n; k++) x2[k] = (x[k] << 1) | (k ? x[k - 1] >> 63 : 0);
  x2[n] = x[n - 1] >> 63;
  int neg = 0;
  if (x2[n]) neg = 1;
  else
    for (size_t k = n; k-- > 0;) {
      if (x2[k] != Q[k]) { neg = x2[k] > Q[k]; break; }
    }
  if (neg) { /* x = Q - x */
    u64 borrow = 0;
    for (size_t k = 0; k < n; k++) {
      u128 t = (u128)Q[k] - x[k] - borrow;
      x[k] = (u64)t;
      borrow = (u64)(t >> 64) & 1;
    }
  }
  /* truncate to 53 significant bits */
  size_t top = n;
  while (top > 0 && x[top - 1] == 0) top--;
  if (!top) return 0.0;
  int hb = 63 - __builtin_clzll(x[top - 1]);
  size_t bitlen = (top - 1) * 64 + (size_t)hb + 1;
  double r;
  if (bitlen <= 53) {
    r = (double)x[0];
  } else {
    size_t sh = bitlen - 53, w = sh / 64, b = sh % 64;
    u64 m = x[w] >> b;
    if (b && w + 1 < top) m |= x[w + 1] << (64 - b);
    m &= ((u64)1 << 53) - 1;
    r = ldexp((double)m, (int)sh);
  }
  return neg ? -r : r;
}

/* Decode (encoder.c:657-704).  poly: level limbs in NTT or coefficient form (a copy is
 * transformed); res: slots complex numbers (re, im interleaved). */
void orc_decode(const orc_ctx* c, double* res, const int64_t* poly, size_t level, uint32_t slots, double factor,
                int is_ntt) {
  size_t N = c->N, half = N / 2;
  if (!slots) slots = (uint32_t)half;
  uint32_t gap = (uint32_t)(half / slots);
  i64* p = (i64*)malloc(sizeof(i64) * level * N);
  memcpy(p, poly, sizeof(i64) * level * N);
  if (is_ntt) {
    int32_t idx[128];
    for (size_t t = 0; t < level; t++) idx[t] = (int32_t)t;
    orc_intt(c, p, p, idx, level);
  }
  dcmplx* msg = (dcmplx*)malloc(sizeof(dcmplx) * slots);
  i64 v[64];
  for (uint32_t i = 0; i < slots; i++) {
    for (size_t t = 0; t < level; t++) v[t] = p[t * N + (size_t)i * gap];
    double re = crt_to_double(c, v, level);
    for (size_t t = 0; t < level; t++) v[t] = p[t * N + (size_t)i * gap + half];
    double im = crt_to_double(c, v, level);
    re /= factor;
    im /= factor;
    msg[i] = re + im * I;
  }
  embedding(c, (dcmplx*)res, msg, slots);
  free(p);
  free(msg);
}
