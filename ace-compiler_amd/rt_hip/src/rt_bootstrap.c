/* rt_bootstrap.c -- CKKS bootstrapping as a composition of the device operations:
 * modulus raise, coefficients-to-slots and slots-to-coefficients as collapsed FFT
 * layers with hoisted rotations kept in the extended (QP) domain, and the modular
 * reduction as a Chebyshev series of a scaled cosine followed by double-angle steps.
 *
 * Follows the reference's algorithm and level accounting (ckks/src/bootstrap.c,
 * ckks/src/chebyshev_impl.c, ckks/src/cipher.c:491-767, ckks/src/evaluator.c:113-595,
 * context/src/ckks_context.c:239-262) so that a program gets the level it asked for;
 * the host side keeps flat arrays instead of value lists, and every polynomial
 * operation is a device call.
 */
#include <complex.h>
#include <math.h>

#include "rt_internal.h"

#ifndef M_PI
#define M_PI 3.14159265358979323846
#endif

/* ---- the approximated function ---------------------------------------------------------------
 * After r double-angle steps c <- 2c^2 - (2 pi)^(-2^(j-r)) the value is cos(2^r theta) / (2 pi), so the
 * series approximates (2 pi)^(-1/2^r) cos((2 pi K x - shift) / 2^r) on [-1, 1]; shift = pi/2 turns the
 * cosine into the sine of 2 pi K x.  The reference tabulates the Chebyshev interpolation coefficients
 * of exactly these functions (include/ckks/bootstrap.h:66-196); here they are computed. */
typedef struct {
  uint32_t k_bound, double_angle, n_coeff;
  bool     even;
  double   coeff[96];
} SIN_POLY;
static SIN_POLY Sin_poly;

static void fill_sin_poly(SIN_POLY* p, size_t hamming_weight, bool even) {
  bool low        = hamming_weight > 0 && hamming_weight <= 192;
  p->even         = even;
  p->k_bound      = low ? 32 : 512;
  p->double_angle = low ? 3 : (even ? 7 : 6);
  p->n_coeff      = (low || even) ? 55 : 89;
  uint32_t nodes  = 4 * p->n_coeff;
  double   pw = pow(2.0, p->double_angle), amp = pow(2.0 * M_PI, -1.0 / pw), shift = even ? 0.0 : M_PI / 2;
  for (uint32_t k = 0; k < p->n_coeff; ++k) {
    double acc = 0;
    for (uint32_t j = 0; j < nodes; ++j) {
      double t = M_PI * (j + 0.5) / nodes;
      acc += amp * cos((2.0 * M_PI * p->k_bound * cos(t) - shift) / pw) * cos(k * t);
    }
    p->coeff[k] = (even && (k & 1)) ? 0.0 : 2.0 * acc / nodes;
  }
}
static const SIN_POLY* sin_poly(void) {
  if (__atomic_load_n(&Sin_poly.n_coeff, __ATOMIC_ACQUIRE)) return &Sin_poly;
  Rt_shared_lock();
  if (!Sin_poly.n_coeff) {
    SIN_POLY    p;
    const char* env = getenv("RTLIB_BTS_EVEN_POLY");
    fill_sin_poly(&p, Get_context_params()->_hamming_weight, env && atoi(env) != 0);
    uint32_t n = p.n_coeff;
    p.n_coeff  = 0;
    Sin_poly   = p;
    __atomic_store_n(&Sin_poly.n_coeff, n, __ATOMIC_RELEASE); /* the count makes the rest visible */
  }
  Rt_shared_unlock();
  return &Sin_poly;
}
/* for inspection without a context: the series of a Hamming weight; returns the number of coefficients */
size_t Rt_sin_series(size_t hamming_weight, int even, double* coeff, uint32_t* k_bound, uint32_t* double_angle) {
  SIN_POLY p;
  fill_sin_poly(&p, hamming_weight, even != 0);
  memcpy(coeff, p.coeff, p.n_coeff * sizeof(double));
  *k_bound      = p.k_bound;
  *double_angle = p.double_angle;
  return p.n_coeff;
}

/* multiplicative depth of a Chebyshev series by degree (bootstrap.c:64-80), normalised input */
static uint32_t series_depth(uint32_t n_coeff) {
  static const uint32_t upto[] = {4, 5, 13, 27, 59, 119, 247, 495, 1007, 2031};
  uint32_t              deg = n_coeff - 1, d = 3;
  for (size_t i = 0; i < sizeof(upto) / sizeof(upto[0]); ++i, ++d)
    if (deg <= upto[i]) return d - 1;
  Rt_fatal(__FILE__, __LINE__, "Polynomial degree is supported from 5 to 2031 inclusive.");
}
static uint32_t approx_mod_depth(void) { return series_depth(sin_poly()->n_coeff) + sin_poly()->double_angle; }

/* ---- plan of the collapsed FFT (bootstrap.c:523-607) --------------------------------------------- */
typedef struct {
  int32_t budget, layers, rem, num_rot, b, g, num_rot_rem, b_rem, g_rem;
} FFT_PLAN;

static void select_layers(uint32_t log_slots, uint32_t budget, uint32_t* layers, uint32_t* rem) {
  uint32_t l = (uint32_t)ceil((double)log_slots / budget), rows = log_slots / l, r = log_slots % l;
  uint32_t dim = rows + (r != 0);
  if (dim < budget) {
    l -= 1;
    rows = log_slots / l;
    r    = log_slots - rows * l;
    dim  = rows + (r != 0);
    while (dim != budget) {
      rows -= 1;
      r   = log_slots - rows * l;
      dim = rows + (r != 0);
    }
  }
  *layers = l;
  *rem    = r;
}
static int32_t giant_for(int32_t num_rot, int32_t layers) {
  return 1 << (layers / 2 + (num_rot > 7 ? 2 : 1));
}
static FFT_PLAN fft_plan(uint32_t slots, uint32_t budget) {
  FFT_PLAN p;
  uint32_t layers, rem;
  select_layers((uint32_t)log2(slots), budget, &layers, &rem);
  p.budget      = (int32_t)budget;
  p.layers      = (int32_t)layers;
  p.rem         = (int32_t)rem;
  p.num_rot     = (1 << (layers + 1)) - 1;
  p.num_rot_rem = (1 << (rem + 1)) - 1;
  p.g           = giant_for(p.num_rot, p.layers);
  p.b           = (p.num_rot + 1) / p.g;
  p.g_rem = p.b_rem = 0;
  if (rem) {
    p.g_rem = giant_for(p.num_rot_rem, p.rem);
    p.b_rem = (p.num_rot_rem + 1) / p.g_rem;
  }
  return p;
}

/* index into [1, slots) of a signed rotation (bootstrap.c:197-209) */
static uint32_t reduce_rotation(int32_t index, uint32_t slots) {
  int32_t s = (int32_t)slots;
  return (uint32_t)(((index % s) + s) % s);
}

/* rotations applied inside (in) and between (out) the baby-step groups of level s (bootstrap.c:1427-1459) */
typedef struct {
  int32_t giant, baby, num_rot, in[64], out[64];
} LEVEL_ROTS;
static LEVEL_ROTS level_rots(const FFT_PLAN* p, int32_t s, bool encoding, bool is_rem, uint32_t slots) {
  LEVEL_ROTS r;
  int32_t    flag_rem = p->rem != 0, quarter = (int32_t)(G.N / 2);
  uint32_t   in_mod = encoding ? slots : (uint32_t)quarter;
  memset(&r, 0, sizeof(r));
  if (!is_rem) {
    int32_t shift = encoding ? (s - flag_rem) * p->layers + p->rem : s * p->layers;
    r.giant = p->g, r.baby = p->b, r.num_rot = p->num_rot;
    for (int32_t j = 0; j < p->g; ++j) r.in[j] = (int32_t)reduce_rotation((j - (p->num_rot + 1) / 2 + 1) * (1 << shift), in_mod);
    for (int32_t i = 0; i < p->b; ++i) r.out[i] = (int32_t)reduce_rotation(p->g * i * (1 << shift), (uint32_t)quarter);
  } else {
    int32_t mult = encoding ? 1 : 1 << (s * p->layers);
    r.giant = p->g_rem, r.baby = p->b_rem, r.num_rot = p->num_rot_rem;
    for (int32_t j = 0; j < p->g_rem; ++j) r.in[j] = (int32_t)reduce_rotation((j - (p->num_rot_rem + 1) / 2 + 1) * mult, in_mod);
    for (int32_t i = 0; i < p->b_rem; ++i) r.out[i] = (int32_t)reduce_rotation(p->g_rem * i * mult, (uint32_t)quarter);
  }
  return r;
}
/* the levels of the plan in the order they are applied; *n_steps entries of (s, is_rem) */
static void level_order(const FFT_PLAN* p, bool encoding, int32_t* s_of, bool* rem_of, int32_t* n_steps) {
  int32_t flag_rem = p->rem != 0, n = 0;
  int32_t start = encoding ? flag_rem : 0, end = encoding ? p->budget : p->budget - flag_rem;
  if (encoding)
    for (int32_t s = end - 1; s >= start; --s) s_of[n] = s, rem_of[n++] = false;
  else
    for (int32_t s = start; s < end; ++s) s_of[n] = s, rem_of[n++] = false;
  if (flag_rem) s_of[n] = encoding ? 0 : p->budget - 1, rem_of[n++] = true;
  *n_steps = n;
}

/* ---- precomputation of the plaintext diagonals (bootstrap.c:424-915) ------------------------------ */
typedef struct BTS_PRECOM {
  uint32_t           slots;
  FFT_PLAN           enc, dec;
  PLAINTEXT*         enc_plain[32]; /* per level: num_rot (num_rot_rem) plaintexts with P limbs */
  PLAINTEXT*         dec_plain[32];
  size_t             enc_count[32], dec_count[32];
  bool               keys;
  struct BTS_PRECOM* next;
} BTS_PRECOM;
static BTS_PRECOM* Precoms;

/* one butterfly layer of the special FFT as three diagonals per layer: rows s (input rotated right),
 * s + log (unrotated), s + 2 log (rotated left); (bootstrap.c:424-515) */
static DCMPLX* one_level(const DCMPLX* ksi, const uint32_t* rot_group, uint32_t slots, bool flag, bool encoding) {
  uint32_t dim = 4 * slots, logs = (uint32_t)log2(slots);
  DCMPLX*  c   = (DCMPLX*)calloc((size_t)3 * logs * slots, sizeof(DCMPLX));
  for (uint32_t m = slots; m > 1; m >>= 1) {
    uint32_t s = (uint32_t)log2(m) - 1, lenh = m >> 1, lenq = m << 2;
    DCMPLX * right = c + (size_t)s * slots, *mid = c + (size_t)(s + logs) * slots, *left = c + (size_t)(s + 2 * logs) * slots;
    for (uint32_t k = 0; k < slots; k += m)
      for (uint32_t j = 0; j < lenh; ++j) {
        uint32_t r  = rot_group[j] % lenq;
        DCMPLX   w  = ksi[(encoding ? lenq - r : r) * (dim / lenq)];
        DCMPLX   u  = 1.0;
        if (flag && m == 2) {
          u = cexp((encoding ? -1.0 : 1.0) * M_PI / 2 * I);
          w = u * w;
        }
        if (encoding) {
          mid[j + k]          = u;
          left[j + k]         = u;
          mid[j + k + lenh]   = -w;
          right[j + k + lenh] = w;
        } else {
          mid[j + k]          = u;
          left[j + k]         = w;
          mid[j + k + lenh]   = -w;
          right[j + k + lenh] = u;
        }
      }
  }
  return c;
}

/* the layers of each level multiplied together: level s -> rows[s] diagonals of `slots` entries
 * (bootstrap.c:609-781) */
static DCMPLX** collapse(const DCMPLX* ksi, const uint32_t* rot_group, uint32_t slots, const FFT_PLAN* p, bool flag,
                         bool encoding, size_t* rows) {
  uint32_t logs = (uint32_t)log2(slots);
  int32_t  flag_rem = p->rem != 0;
  DCMPLX*  c1  = one_level(ksi, rot_group, slots, flag, encoding);
  DCMPLX** out = (DCMPLX**)calloc((size_t)p->budget, sizeof(DCMPLX*));
  for (int32_t s = 0; s < p->budget; ++s) {
    bool    is_rem = flag_rem && ((encoding && s == 0) || (!encoding && s == p->budget - 1));
    int32_t layers = is_rem ? p->rem : p->layers;
    int32_t top    = encoding ? (int32_t)logs - (p->budget - 1 - s) * p->layers - 1 : s * p->layers;
    rows[s]        = (size_t)(is_rem ? p->num_rot_rem : p->num_rot);
    DCMPLX* cur    = (DCMPLX*)calloc(rows[s] * slots, sizeof(DCMPLX));
    for (int t = 0; t < 3; ++t) memcpy(cur + (size_t)t * slots, c1 + (size_t)(top + t * (int32_t)logs) * slots, slots * sizeof(DCMPLX));
    for (int32_t l = 1; l < layers; ++l) {
      DCMPLX* nxt  = (DCMPLX*)calloc(rows[s] * slots, sizeof(DCMPLX));
      int32_t have = (1 << (l + 1)) - 1, row = encoding ? top - l : top + l;
      const DCMPLX *f0 = c1 + (size_t)row * slots, *f1 = c1 + (size_t)(row + (int32_t)logs) * slots,
                   *f2 = c1 + (size_t)(row + 2 * (int32_t)logs) * slots;
      for (int32_t u = 0; u < have; ++u) {
        const DCMPLX* src = cur + (size_t)u * slots;
        for (uint32_t k = 0; k < slots; ++k) {
          if (encoding) {
            uint32_t step = 1u << (top - l);
            nxt[(size_t)(2 * u) * slots + k] += f0[k] * src[reduce_rotation((int32_t)k - (int32_t)step, slots)];
            nxt[(size_t)(2 * u + 1) * slots + k] += f1[k] * src[k];
            nxt[(size_t)(2 * u + 2) * slots + k] += f2[k] * src[reduce_rotation((int32_t)(k + step), slots)];
          } else {
            nxt[(size_t)u * slots + k] += f0[k] * src[k];
            nxt[(size_t)(u + (1 << l)) * slots + k] += f1[k] * src[k];
            nxt[(size_t)(u + (1 << (l + 1))) * slots + k] += f2[k] * src[k];
          }
        }
      }
      free(cur);
      cur = nxt;
    }
    out[s] = cur;
  }
  free(c1);
  return out;
}

/* the diagonals of every level, rotated for the baby-step/giant-step order and encoded with P limbs
 * at the level they are used on (bootstrap.c:287-422) */
static void encode_levels(BTS_PRECOM* pre, bool encoding, const DCMPLX* ksi, const uint32_t* rot_group, double scale,
                          double factor, uint32_t top_level) {
  const FFT_PLAN* p = encoding ? &pre->enc : &pre->dec;
  uint32_t        slots = pre->slots, len = slots;
  bool            sparse = slots != G.N / 2;
  size_t          rows[32];
  DCMPLX**        c = collapse(ksi, rot_group, slots, p, false, encoding, rows);
  if (sparse) { /* the second half of the vector carries the transform of i * input (bootstrap.c:805-836) */
    DCMPLX** c2 = collapse(ksi, rot_group, slots, p, true, encoding, rows);
    len         = 2 * slots;
    for (int32_t s = 0; s < p->budget; ++s) {
      DCMPLX* m = (DCMPLX*)malloc(rows[s] * len * sizeof(DCMPLX));
      for (size_t r = 0; r < rows[s]; ++r) {
        memcpy(m + r * len, c[s] + r * slots, slots * sizeof(DCMPLX));
        memcpy(m + r * len + slots, c2[s] + r * slots, slots * sizeof(DCMPLX));
      }
      free(c[s]);
      free(c2[s]);
      c[s] = m;
    }
    free(c2);
  }
  if (factor != 1.0)
    for (int32_t s = 0; s < p->budget; ++s)
      for (size_t i = 0; i < rows[s] * len; ++i) c[s][i] *= factor;

  int32_t     flag_rem = p->rem != 0, order_s[32], n_steps;
  bool        order_rem[32];
  PLAINTEXT** plains = encoding ? pre->enc_plain : pre->dec_plain;
  size_t*     counts = encoding ? pre->enc_count : pre->dec_count;
  DCMPLX*     rot    = (DCMPLX*)malloc(len * sizeof(DCMPLX));
  level_order(p, encoding, order_s, order_rem, &n_steps);
  for (int32_t step = 0; step < n_steps; ++step) {
    int32_t    s = order_s[step];
    bool       is_rem = order_rem[step];
    LEVEL_ROTS r = level_rots(p, s, encoding, is_rem, slots);
    /* the scale of the whole transform goes into one level: the remainder, else the one applied first
     * in encoding and last in decoding */
    bool     scaled = is_rem || (!flag_rem && s == (encoding ? 0 : p->budget - 1));
    uint32_t level  = top_level - (uint32_t)step; /* one rescale between consecutive levels */
    counts[s]       = rows[s];
    plains[s]       = (PLAINTEXT*)calloc(rows[s], sizeof(PLAINTEXT));
    for (int32_t i = 0; i < r.baby; ++i)
      for (int32_t j = 0; j < r.giant; ++j) {
        int32_t d = r.giant * i + j;
        if (d == r.num_rot) continue;
        const DCMPLX* v   = c[s] + (size_t)d * len;
        uint32_t      off = reduce_rotation(-r.out[i], (uint32_t)(G.N / 2));
        for (uint32_t k = 0; k < len; ++k) rot[k] = v[(k + off) % len] * (scaled ? scale : 1.0);
        PLAINTEXT* pt = &plains[s][d];
        Alloc_poly_data(&pt->_poly, G.N, level, G.K);
        pt->_poly._is_ntt   = true;
        pt->_scaling_factor = G.sc;
        pt->_sf_degree      = 1;
        pt->_slots          = len;
        ACE_OK(ace_encode(RT_CTX, pt->_poly._data, (const double*)rot, len, len, level, 1, G.K));
      }
  }
  free(rot);
  for (int32_t s = 0; s < p->budget; ++s) free(c[s]);
  free(c);
}

static BTS_PRECOM* find_precom(uint32_t slots) {
  for (BTS_PRECOM* p = __atomic_load_n(&Precoms, __ATOMIC_ACQUIRE); p; p = p->next)
    if (p->slots == slots) return p;
  return NULL;
}

static uint32_t bootstrap_depth(const BTS_PRECOM* pre) {
  return approx_mod_depth() + (uint32_t)pre->enc.budget + (uint32_t)pre->dec.budget;
}

/* Bootstrap_setup with the level budgets {3, 3} of Bootstrap_precom (bootstrap.c:1061-1197,
 * ckks_context.c:239-262) */
static BTS_PRECOM* setup_locked(uint32_t slots);
static BTS_PRECOM* setup(uint32_t slots) {
  BTS_PRECOM* pre = find_precom(slots); /* the list only grows, at its head, by whole entries */
  if (pre) return pre;
  Rt_shared_lock();
  pre = setup_locked(slots);
  Rt_shared_unlock();
  return pre;
}
static BTS_PRECOM* setup_locked(uint32_t slots) {
  BTS_PRECOM* pre = find_precom(slots);
  if (pre) return pre;
  FMT_ASSERT(slots >= 2 && (slots & (slots - 1)) == 0 && slots <= G.N / 2, "bootstrap: invalid slot count %u", slots);
  uint32_t logs = (uint32_t)log2(slots), budget = logs < 3 ? logs : 3;
  pre        = (BTS_PRECOM*)calloc(1, sizeof(BTS_PRECOM));
  pre->slots = slots;
  pre->enc   = fft_plan(slots, budget);
  pre->dec   = fft_plan(slots, budget);
  uint32_t depth = bootstrap_depth(pre);
  FMT_ASSERT(G.L > depth, "bootstrap needs %u levels, the context has %zu: set a larger multiply depth", depth, G.L - 1);

  uint32_t  slots4 = 4 * slots;
  uint32_t* rot_group = (uint32_t*)malloc(slots * sizeof(uint32_t));
  DCMPLX*   ksi = (DCMPLX*)malloc((slots4 + 1) * sizeof(DCMPLX));
  for (uint32_t i = 0, five = 1; i < slots; ++i, five = five * 5 % slots4) rot_group[i] = five;
  for (uint32_t i = 0; i < slots4; ++i) {
    double angle = 2.0 * M_PI * i / slots4;
    ksi[i]       = cos(angle) + sin(angle) * I;
  }
  ksi[slots4] = ksi[0];

  /* q0 as a power of two times `pre` (bootstrap.c:1136-1143): encoding divides by the power of two,
   * N and the bound K of the integer part, spread evenly over the levels (bootstrap.c:838-866) */
  double q0 = (double)G.q[0]._val, pw = ldexp(1.0, (int)round(log2(q0))), ratio = q0 / pw;
  double factor = 1.0 / (double)G.N / (double)sin_poly()->k_bound / pow(2.0, round(log2(q0 / G.sc)));
  factor        = pow(factor, 1.0 / pre->enc.budget);
  encode_levels(pre, true, ksi, rot_group, ratio, factor, (uint32_t)G.L);
  encode_levels(pre, false, ksi, rot_group, 1.0 / ratio, 1.0, (uint32_t)(G.L - approx_mod_depth() - (uint32_t)pre->enc.budget));
  free(ksi);
  free(rot_group);
  Rt_shared_publish(); /* the diagonals are encoded on this thread's stream and read on every thread's */
  pre->next = Precoms;
  __atomic_store_n(&Precoms, pre, __ATOMIC_RELEASE);
  return pre;
}

/* rotation keys of every step of both transforms, the sparse-packing sums, and conjugation
 * (bootstrap.c:211-285,1199-1231) */
static void need_rot_key(int32_t rot) {
  if (rot == 0 || (uint32_t)rot == G.N / 2) return;
  ROT_KEY* r = Rt_find_rot(rot);
  if (r && __atomic_load_n(&r->swk._public_keys, __ATOMIC_ACQUIRE)) return;
  Rt_shared_lock(); /* another thread may be making this key */
  r = Rt_find_rot(rot);
  if (!r || !r->swk._public_keys) Rt_generate_rotation_key(rot);
  Rt_shared_unlock();
}
static void keygen(BTS_PRECOM* pre) {
  if (__atomic_load_n(&pre->keys, __ATOMIC_ACQUIRE)) return;
  for (int enc = 1; enc >= 0; --enc) {
    const FFT_PLAN* p = enc ? &pre->enc : &pre->dec;
    int32_t         s_of[32], n;
    bool            rem_of[32];
    level_order(p, enc, s_of, rem_of, &n);
    for (int32_t t = 0; t < n; ++t) {
      LEVEL_ROTS r = level_rots(p, s_of[t], enc, rem_of[t], pre->slots);
      for (int32_t j = 0; j < r.giant; ++j) need_rot_key(r.in[j]);
      for (int32_t i = 0; i < r.baby; ++i) need_rot_key(r.out[i]);
    }
  }
  for (uint32_t j = 1; j < G.N / (2 * pre->slots); j <<= 1) need_rot_key((int32_t)(j * pre->slots));
  need_rot_key((int32_t)(2 * G.N - 1));
  __atomic_store_n(&pre->keys, true, __ATOMIC_RELEASE);
}

/* Bootstrap_precom (context/src/ckks_context.c:239-262): when the chain is deep enough to bootstrap at all, the
 * plaintext diagonals and the keys of the default slot count are made at key generation, not inside the program */
void Rt_bootstrap_prepare(void) {
  uint32_t slots = (uint32_t)(G.N / 2);
  if (slots < 2) return;
  uint32_t logs = (uint32_t)log2(slots), budget = logs < 3 ? logs : 3;
  if (G.L - 1 <= approx_mod_depth() + 2 * budget) return;
  keygen(setup(slots));
}

static void stage_clear(void);
static void mono_clear(void);
void Rt_bootstrap_finalize(void) {
  mono_clear();
  stage_clear();
  while (Precoms) {
    BTS_PRECOM* p = Precoms;
    Precoms       = p->next;
    for (int s = 0; s < 32; ++s) {
      for (size_t d = 0; d < p->enc_count[s]; ++d)
        if (p->enc_plain[s][d]._poly._data) Free_poly_data(&p->enc_plain[s][d]._poly);
      for (size_t d = 0; d < p->dec_count[s]; ++d)
        if (p->dec_plain[s][d]._poly._data) Free_poly_data(&p->dec_plain[s][d]._poly);
      free(p->enc_plain[s]);
      free(p->dec_plain[s]);
    }
    free(p);
  }
  memset(&Sin_poly, 0, sizeof(Sin_poly));
}

/* ---- evaluator pieces on whole ciphertexts (evaluator.c:113-286,401-409) --------------------------- */
static void new_ciph(CIPHER c) { memset(c, 0, sizeof(*c)); }

static void add_const(CIPHER c, double value) { /* Add_const, in place */
  int64_t w[128];
  size_t  l = Level(c);
  Rt_encode_val_words(w, value, (uint32_t)l, c->_scaling_factor);
  ACE_OK(ace_poly_add_scalars(RT_CTX, c->_c0_poly._data, c->_c0_poly._data, w, l));
}
static void scale_words(CIPHER res, CIPHER c, const int64_t* w, double sf, uint32_t deg) {
  size_t l = Level(c);
  if (res != c) {
    Init_poly(&res->_c0_poly, &c->_c0_poly);
    Init_poly(&res->_c1_poly, &c->_c1_poly);
    res->_slots = c->_slots;
  }
  res->_c0_poly._is_ntt = res->_c1_poly._is_ntt = true;
  ACE_OK(ace_poly_mul_scalars(RT_CTX, res->_c0_poly._data, c->_c0_poly._data, w, l));
  ACE_OK(ace_poly_mul_scalars(RT_CTX, res->_c1_poly._data, c->_c1_poly._data, w, l));
  res->_scaling_factor = sf;
  res->_sf_degree      = deg;
}
static void mul_const(CIPHER res, CIPHER c, double value) { /* Mul_const: the scale goes up by one degree */
  int64_t w[128];
  Rt_encode_val_words(w, value, (uint32_t)Level(c), G.sc);
  scale_words(res, c, w, c->_scaling_factor * G.sc, c->_sf_degree + 1);
}
static void mul_integer(CIPHER res, CIPHER c, uint64_t v) { /* Mul_integer: the scale stays */
  int64_t w[128];
  for (size_t t = 0; t < Level(c); ++t) w[t] = (int64_t)(v % (uint64_t)G.q[t]._val);
  scale_words(res, c, w, c->_scaling_factor, c->_sf_degree);
}
static void rescale(CIPHER c) { Rescale_ciph(c, c); }
static void set_level(CIPHER c, size_t level) {
  Set_poly_level(&c->_c0_poly, level);
  Set_poly_level(&c->_c1_poly, level);
}

/* The monomial X^power over all Q limbs in NTT form, kept on the device once built: a bootstrap multiplies by the
 * same two monomials every time, and building one means a host buffer of a whole polynomial, an upload (which waits
 * for the GPU to finish everything issued so far) and a transform. */
#define MONO_SLOTS 16
static struct {
  uint32_t power;
  int64_t* dev;
} Mono[MONO_SLOTS];
static size_t Mono_n; /* entries below it are complete, on the device too, and stay until the context ends */
static void   mono_clear(void) {
  for (size_t i = 0; i < Mono_n; ++i) Rt_dev_free(Mono[i].dev);
  Mono_n = 0;
}
static int64_t* build_monomial(uint32_t power) {
  size_t   n = G.N, l = G.L;
  int64_t* host = (int64_t*)calloc(l * n, sizeof(int64_t));
  int64_t* mono = Rt_dev_alloc(l * n);
  int32_t  idx[128];
  for (size_t t = 0; t < l; ++t) {
    host[t * n + power % n] = power < n ? 1 : G.q[t]._val - 1;
    idx[t]                  = (int32_t)t;
  }
  ACE_OK(ace_upload(RT_CTX, mono, host, l * n));
  ACE_OK(ace_ntt(RT_CTX, mono, mono, idx, l, 1, 0));
  free(host);
  return mono;
}
/* *temporary: the table is full and the caller frees the polynomial after use */
static int64_t* monomial(uint32_t power, bool* temporary) {
  power %= (uint32_t)(2 * G.N);
  *temporary = false;
  size_t seen = __atomic_load_n(&Mono_n, __ATOMIC_ACQUIRE);
  for (size_t i = 0; i < seen; ++i)
    if (Mono[i].power == power) return Mono[i].dev;
  Rt_shared_lock();
  int64_t* mono = NULL;
  for (size_t i = 0; i < Mono_n && !mono; ++i)
    if (Mono[i].power == power) mono = Mono[i].dev;
  if (!mono) {
    mono = build_monomial(power);
    if (Mono_n < MONO_SLOTS) {
      Rt_shared_publish(); /* built on this thread's stream, read on every thread's */
      Mono[Mono_n].power = power;
      Mono[Mono_n].dev   = mono;
      __atomic_store_n(&Mono_n, Mono_n + 1, __ATOMIC_RELEASE);
    } else {
      *temporary = true;
    }
  }
  Rt_shared_unlock();
  return mono;
}
CIPHER Mul_mono_ciph(CIPHER res, CIPHER c, uint32_t power) { /* Mul_by_monomial (evaluator.c:260-286) */
  size_t   l    = Level(c);
  bool     temporary;
  int64_t* mono = monomial(power, &temporary); /* limb t of a polynomial at any level is limb t of the chain */
  if (res != c) {
    Init_poly(&res->_c0_poly, &c->_c0_poly);
    Init_poly(&res->_c1_poly, &c->_c1_poly);
    res->_scaling_factor = c->_scaling_factor;
    res->_sf_degree      = c->_sf_degree;
    res->_slots          = c->_slots;
  }
  ACE_OK(ace_poly_mul(RT_CTX, res->_c0_poly._data, c->_c0_poly._data, mono, l, 0));
  ACE_OK(ace_poly_mul(RT_CTX, res->_c1_poly._data, c->_c1_poly._data, mono, l, 0));
  if (temporary) Rt_dev_free(mono);
  res->_c0_poly._is_ntt = res->_c1_poly._is_ntt = true;
  return res;
}

static void rotate_into(CIPHER res, CIPHER c, int32_t rot) { /* Eval_fast_rotate / Conjugate */
  need_rot_key(rot);
  Rotate_ciph(res, c, rot);
}

/* ---- one collapsed level with hoisted rotations in the extended domain (bootstrap.c:1233-1373) ----- */
typedef struct {
  int64_t *c0, *c1; /* level + num_p limbs each */
} EXT_CT;
static EXT_CT ext_alloc(size_t level) {
  EXT_CT e = {Rt_dev_alloc_raw((level + G.K) * G.N), Rt_dev_alloc_raw((level + G.K) * G.N)};
  return e;
}
static void ext_free(EXT_CT* e) {
  Rt_dev_free(e->c0);
  Rt_dev_free(e->c1);
}
/* both key halves against hoisted digits, then the automorphism (Fast_rotate_ext, evaluator.c:532-566) */
/* (out.c0, out.c1) = the rotation by `rot` of (sum of digits * key halves) + (c0_ext, 0), all in the extended basis;
 * accumulate bit 0 / 1: added to what out.c0 / out.c1 holds */
static void ext_rotate(EXT_CT* out, const int64_t* digits, size_t n_digits, const int64_t* c0_ext, int32_t rot,
                       size_t level, int accumulate) {
  ROT_KEY* key = Rt_find_rot(rot);
  FMT_ASSERT(key, "cannot find auto key of rotation %d", rot);
  size_t half = (G.L + G.K) * G.N;
  ACE_OK(ace_ext_rotate(RT_CTX, out->c0, out->c1, digits, key->swk._public_keys->dev, half, 2 * half, n_digits, c0_ext,
                        key->order, level, accumulate));
}
/* rescaled_already: the previous iteration ended with its Rescale_ciph (see the end of this function);
 * then_rescale: another iteration follows, which begins with a Rescale_ciph of this one's result */
static void rotate_iteration(CIPHER ct, BTS_PRECOM* pre, bool encoding, int32_t s, bool is_rem, bool first_step,
                             bool rescaled_already, bool then_rescale) {
  const FFT_PLAN* p      = encoding ? &pre->enc : &pre->dec;
  PLAINTEXT*      plains = (encoding ? pre->enc_plain : pre->dec_plain)[s];
  LEVEL_ROTS      r      = level_rots(p, s, encoding, is_rem, pre->slots);
  if (!first_step && !rescaled_already) rescale(ct);
  size_t level = Level(ct), T = level + G.K, n = G.N, nd = ace_num_decomp(RT_CTX, level);

  int64_t* digits = Rt_dev_alloc_raw(nd * T * n);
  ACE_OK(ace_precomp(RT_CTX, digits, ct->_c1_poly._data, level, 1));
  int64_t* c0_ext = Rt_dev_alloc_raw(T * n);
  ACE_OK(ace_extend(RT_CTX, c0_ext, ct->_c0_poly._data, level));
  EXT_CT  outer = ext_alloc(level);
  EXT_CT* rots = (EXT_CT*)calloc((size_t)r.giant, sizeof(EXT_CT));
  for (int32_t j = 0; j < r.giant; ++j) {
    rots[j] = ext_alloc(level);
    if (r.in[j] != 0) {
      ext_rotate(&rots[j], digits, nd, c0_ext, r.in[j], level, 0);
    } else { /* Switch_key_ext: the ciphertext itself, lifted */
      Rt_dev_copy(rots[j].c0, c0_ext, T * n);
      ACE_OK(ace_extend(RT_CTX, rots[j].c1, ct->_c1_poly._data, level));
    }
  }
  /* the inner sums of all baby-step groups first: the groups share the rotated ciphertexts, which are read once
   * for every four groups (ace_ext_plain_mac_groups).  The sums lie side by side in one buffer, so that the c1 parts
   * of consecutive groups are a sequence at a constant stride for the batched calls below. */
  int64_t*        inner_slab = Rt_dev_alloc_raw((size_t)r.baby * 2 * T * n);
  int64_t*        low        = Rt_dev_alloc_raw((size_t)r.baby * level * n);
  int64_t*        low_digits = Rt_dev_alloc_raw((size_t)r.baby * nd * T * n);
  EXT_CT*         inners = (EXT_CT*)calloc((size_t)r.baby, sizeof(EXT_CT));
  int64_t **      in_r0 = (int64_t**)calloc((size_t)r.baby, sizeof(int64_t*)), **in_r1 = (int64_t**)calloc((size_t)r.baby, sizeof(int64_t*));
  const int64_t** inp   = (const int64_t**)calloc((size_t)r.baby * (size_t)r.giant, sizeof(int64_t*));
  const int64_t * in0[64], *in1[64];
  FMT_ASSERT(r.giant <= 64, "too many rotations in one baby-step group");
  size_t plain_level = 0;
  for (int32_t j = 0; j < r.giant; ++j) {
    in0[j] = rots[j].c0;
    in1[j] = rots[j].c1;
  }
  for (int32_t i = 0; i < r.baby; ++i) {
    inners[i].c0 = inner_slab + (size_t)i * 2 * T * n;
    inners[i].c1 = inners[i].c0 + T * n;
    in_r0[i]  = inners[i].c0;
    in_r1[i]  = inners[i].c1;
    for (int32_t j = 0; j < r.giant; ++j) {
      int32_t d = r.giant * i + j;
      if (d == r.num_rot) continue; /* stays NULL: no such term */
      FMT_ASSERT(plains[d]._poly._num_primes >= level, "bootstrap plaintext below the ciphertext level");
      plain_level            = plains[d]._poly._num_primes;
      inp[i * r.giant + j] = plains[d]._poly._data;
    }
  }
  ACE_OK(ace_ext_plain_mac_groups(RT_CTX, in_r0, in_r1, (size_t)r.baby, in0, in1, (size_t)r.giant, inp, level, plain_level));
  /* The result is sum_i rotation_i(inner sum i).  Group 0 is not rotated: its two halves start the running sums
   * `first` (c0 parts that need no key switch) and `sum1`.  A rotated group's c1 part is brought down, raised again
   * and rotated with its key; its c0 part rides along as the addend; both land in (outer.c0, sum1). */
  /* One polynomial's Mod_down and Precomp leave most of the machine idle, so consecutive rotated groups go through
   * them together (ace_mod_down_batch, ace_precomp_batch: the words of single calls). */
  int64_t *first = inners[0].c0, *sum1 = inners[0].c1;
  bool     outer0_set = false;
  for (int32_t i = 1; i < r.baby;) {
    EXT_CT* in = &inners[i];
    if (r.out[i] == 0) {
      ACE_OK(ace_poly_add(RT_CTX, first, first, in->c0, level, 1));
      ACE_OK(ace_poly_add(RT_CTX, sum1, sum1, in->c1, level, 1));
      ++i;
      continue;
    }
    int32_t end = i;
    while (end < r.baby && r.out[end] != 0) ++end;
    size_t cnt = (size_t)(end - i);
    ACE_OK(ace_mod_down_batch(RT_CTX, low, level * n, in->c1, 2 * T * n, cnt, level, 1));
    ACE_OK(ace_precomp_batch(RT_CTX, low_digits, nd * T * n, low, level * n, cnt, level, 1));
    for (int32_t g = i; g < end; ++g) {
      EXT_CT into = {outer.c0, sum1};
      ext_rotate(&into, low_digits + (size_t)(g - i) * nd * T * n, nd, inners[g].c0, r.out[g], level,
                 (outer0_set ? 1 : 0) | 2);
      outer0_set = true;
    }
    i = end;
  }
  if (outer0_set) ACE_OK(ace_poly_add(RT_CTX, first, first, outer.c0, level, 1));
  free(inners);
  free(in_r0);
  free(in_r1);
  free((void*)inp);
  if (then_rescale && level > 1) {
    /* Mod_down of both sums and the Rescale_ciph that the next iteration would start with, through one forward
     * transform (the words of the calls one after the other); the results need buffers of their own */
    CIPHERTEXT down;
    new_ciph(&down);
    Rt_shape_ciph(&down, ct, ct->_scaling_factor, ct->_sf_degree); /* (sf * sc / sc, degree + 1 - 1) */
    ACE_OK(ace_mod_down_pair_rescale(RT_CTX, down._c0_poly._data, down._c1_poly._data, first, sum1, level));
    Set_poly_level(&down._c0_poly, level - 1);
    Set_poly_level(&down._c1_poly, level - 1);
    Free_ciph_poly(ct, 1);
    *ct = down;
  } else {
    ACE_OK(ace_mod_down(RT_CTX, ct->_c0_poly._data, first, level, 1));
    ACE_OK(ace_mod_down(RT_CTX, ct->_c1_poly._data, sum1, level, 1));
    ct->_scaling_factor *= G.sc;
    ct->_sf_degree += 1;
  }

  for (int32_t j = 0; j < r.giant; ++j) ext_free(&rots[j]);
  free(rots);
  Rt_dev_free(inner_slab);
  ext_free(&outer);
  Rt_dev_free(digits);
  Rt_dev_free(c0_ext);
  Rt_dev_free(low);
  Rt_dev_free(low_digits);
}

/* Coeffs_to_slots / Slots_to_coeffs (bootstrap.c:1375-1494), in place */
static void coeff_slots_transform(CIPHER ct, BTS_PRECOM* pre, bool encoding) {
  const FFT_PLAN* p = encoding ? &pre->enc : &pre->dec;
  int32_t         s_of[32], n;
  bool            rem_of[32];
  level_order(p, encoding, s_of, rem_of, &n);
  for (int32_t t = 0; t < n; ++t) rotate_iteration(ct, pre, encoding, s_of[t], rem_of[t], t == 0, t > 0, t + 1 < n);
}

/* ---- Chebyshev series by Paterson-Stockmeyer (chebyshev_impl.c) -------------------------------------
 * Coefficient arrays keep the series' convention: entry 0 is c0 of c0/2 + sum c_i T_i. */
typedef struct {
  double* v;
  size_t  n;
} SERIES;
static SERIES series_new(size_t n) {
  SERIES s = {(double*)calloc(n ? n : 1, sizeof(double)), n};
  return s;
}
static SERIES series_copy(const SERIES* a, size_t n) {
  SERIES s = series_new(n);
  memcpy(s.v, a->v, (a->n < n ? a->n : n) * sizeof(double));
  return s;
}
static uint32_t series_degree(const SERIES* s) {
  size_t d = s->n ? s->n - 1 : 0;
  while (d > 0 && s->v[d] == 0.0) --d;
  return (uint32_t)d;
}
/* f = q g + r in the Chebyshev basis, using T_a T_b = (T_{a+b} + T_{|a-b|}) / 2 (Long_div_chebyshev,
 * chebyshev_impl.c:155-263) */
static void series_divide(SERIES* q, SERIES* r, const SERIES* f, const SERIES* g) {
  uint32_t n = series_degree(f), k = series_degree(g);
  *r         = series_copy(f, n + 1);
  r->v[0] /= 2; /* true coefficients while dividing */
  if (n < k) {
    *q = series_new(1);
    r->v[0] *= 2;
    return;
  }
  *q         = series_new(n - k + 1);
  double* gt = (double*)malloc((k + 1) * sizeof(double));
  memcpy(gt, g->v, (k + 1) * sizeof(double));
  gt[0] /= 2;
  for (;;) {
    uint32_t d = n - k;
    double   c = ((d && k) ? 2.0 : 1.0) * r->v[n] / gt[k];
    q->v[d]    = c;
    for (uint32_t i = 0; i <= k; ++i) {
      if (d == 0) {
        r->v[i] -= c * gt[i];
      } else {
        uint32_t lo = i > d ? i - d : d - i;
        r->v[i + d] -= c * gt[i] / 2;
        r->v[lo] -= c * gt[i] / 2;
      }
    }
    r->v[n] = 0.0;
    while (n > 0 && r->v[n] == 0.0) --n;
    if (n < k || d == 0) break;
  }
  r->n = (size_t)n + 1;
  q->v[0] *= 2;
  r->v[0] *= 2;
  free(gt);
}

/* for inspection: f / g with n_f and n_g coefficients; q and r must hold n_f entries; returns the lengths */
void Rt_series_divide(double* q, size_t* n_q, double* r, size_t* n_r, const double* f, size_t n_f, const double* g, size_t n_g) {
  SERIES sf = {(double*)f, n_f}, sg = {(double*)g, n_g}, sq, sr;
  series_divide(&sq, &sr, &sf, &sg);
  memcpy(q, sq.v, sq.n * sizeof(double));
  memcpy(r, sr.v, sr.n * sizeof(double));
  *n_q = sq.n;
  *n_r = sr.n;
  free(sq.v);
  free(sr.v);
}

/* k and m of the evaluation: degree < k (2^m - 1), depth ceil(log2 k) + m minimal (chebyshev_impl.c:71-141) */
static void ps_degrees(uint32_t n, uint32_t* k, uint32_t* m) {
  static const uint32_t upto[16] = {2, 11, 13, 17, 55, 59, 76, 239, 247, 284, 991, 1007, 1083, 2015, 2031, 2204};
  static const uint32_t val[16]  = {1, 2, 3, 2, 3, 4, 3, 4, 5, 4, 5, 6, 5, 6, 7, 6};
  FMT_ASSERT(n >= 1 && n <= 2204, "series degree %u out of range", n);
  for (int i = 0; i < 16; ++i)
    if (n - 1 < upto[i]) {
      *m = val[i];
      *k = n / ((1u << *m) - 1) + 1;
      return;
    }
}

typedef struct {
  CIPHERTEXT *t, *t2; /* T_1..T_k and T_k, T_2k, .. T_{2^(m-1) k} of the input */
  uint32_t    k, m;
} CHEB_BASIS;

/* out = sum w_i T_i (i = 1..count) as one level (Eval_linear_wsum, chebyshev_impl.c:276-318) */
static void weighted_sum(CIPHER out, CHEB_BASIS* b, const double* w, uint32_t count) {
  const int64_t *in0[64], *in1[64];
  size_t         terms = 0, level = Level(&b->t[0]);
  FMT_ASSERT(count <= 32, "more than 32 terms in one weighted sum");
  for (uint32_t i = 0; i < count; ++i) /* the T_i share one level (see eval_chebyshev), except unused odd ones */
    if (w[i] != 0.0 && Level(&b->t[i]) < level) level = Level(&b->t[i]);
  int64_t* words = (int64_t*)malloc(32 * 128 * sizeof(int64_t));
  CIPHER   like  = NULL;
  for (uint32_t i = 0; i < count; ++i) {
    if (w[i] == 0.0) continue;
    like = &b->t[i];
    Rt_encode_val_words(words + terms * level, w[i], (uint32_t)level, G.sc);
    in0[terms]   = b->t[i]._c0_poly._data;
    in1[terms++] = b->t[i]._c1_poly._data;
  }
  FMT_ASSERT(terms, "polynomial has no non_zero coefficient");
  Init_poly(&out->_c0_poly, &like->_c0_poly);
  Init_poly(&out->_c1_poly, &like->_c1_poly);
  set_level(out, level);
  out->_c0_poly._is_ntt = out->_c1_poly._is_ntt = true;
  out->_slots          = like->_slots;
  out->_scaling_factor = like->_scaling_factor * G.sc;
  out->_sf_degree      = like->_sf_degree + 1;
  ACE_OK(ace_ciph_wsum(RT_CTX, out->_c0_poly._data, out->_c1_poly._data, in0, in1, words, terms, level));
  free(words);
  rescale(out);
}
/* a series of degree <= k whose T_k coefficient is known to be `lead` (a power of two, or 1):
 * that term is added, never multiplied, to save the level (Eval_quot_or_rem, chebyshev_impl.c:320-384) */
static void eval_low(CIPHER out, CHEB_BASIS* b, const SERIES* s, double lead) {
  SERIES   low = series_copy(s, b->k);
  uint32_t dg  = series_degree(&low);
  CIPHER   tk  = &b->t[b->k - 1];
  if (dg > 0) {
    weighted_sum(out, b, low.v + 1, dg);
    CIPHERTEXT sum;
    new_ciph(&sum);
    Copy_ciph(&sum, tk);
    for (double have = 1.0; have < lead; have *= 2) Add_ciph(&sum, &sum, &sum);
    Add_ciph(out, out, &sum);
    Free_ciph_poly(&sum, 1);
  } else {
    Copy_ciph(out, tk);
    for (double have = 1.0; have < lead; have *= 2) Add_ciph(out, out, out);
  }
  add_const(out, s->v[0] / 2);
  free(low.v);
}

/* f = (T_{k 2^(m-1)} + c) q + s, recursively (Inner_eval_chebyshev_ps, chebyshev_impl.c:386-500) */
static void eval_ps(CIPHER out, CHEB_BASIS* b, const SERIES* f, uint32_t m) {
  uint32_t k = b->k, span = k * (1u << (m - 1)) - k;
  SERIES   tkm = series_new(span + k + 1), q, r, c, s;
  tkm.v[span + k] = 1.0;
  series_divide(&q, &r, f, &tkm);
  /* r - T_span, divided by q */
  SERIES r2 = series_copy(&r, (span + 1 > r.n) ? span + 1 : r.n);
  r2.v[span] -= 1.0;
  r2.n = (size_t)series_degree(&r2) + 1;
  series_divide(&c, &s, &r2, &q);
  SERIES s2 = series_copy(&s, (s.n > span + 1) ? s.n : span + 1);
  s2.v[s2.n - 1] = 1.0;

  CIPHERTEXT cu, qu, su;
  new_ciph(&cu), new_ciph(&qu), new_ciph(&su);
  uint32_t dc     = series_degree(&c);
  bool     has_cu = dc >= 1;
  if (dc == 1) {
    if (c.v[1] != 1.0) {
      mul_const(&cu, &b->t[0], c.v[1]);
      rescale(&cu);
    } else {
      Copy_ciph(&cu, &b->t[0]);
    }
  } else if (dc > 1) {
    weighted_sum(&cu, b, c.v + 1, dc);
  }
  if (has_cu) add_const(&cu, c.v[0] / 2);

  if (series_degree(&q) > k)
    eval_ps(&qu, b, &q, m - 1);
  else
    eval_low(&qu, b, &q, q.v[q.n - 1]);
  if (series_degree(&s2) > k)
    eval_ps(&su, b, &s2, m - 1);
  else
    eval_low(&su, b, &s2, 1.0);

  CIPHER t2 = &b->t2[m - 1];
  if (has_cu) {
    set_level(&cu, Level(t2) < Level(&cu) ? Level(t2) : Level(&cu));
    Add_ciph(out, t2, &cu);
  } else {
    Copy_ciph(out, t2);
    add_const(out, c.v[0] / 2);
  }
  Rt_mul_rescale_ciph(out, out, &qu, false, NULL); /* Mul_ciph, then Rescale_ciph */
  Add_ciph(out, out, &su);

  Free_ciph_poly(&cu, 1);
  Free_ciph_poly(&qu, 1);
  Free_ciph_poly(&su, 1);
  free(tkm.v), free(q.v), free(r.v), free(c.v), free(s.v), free(r2.v), free(s2.v);
}

/* res = 2 a b - sub, one level down (the product rule of Chebyshev polynomials); sub == NULL subtracts 1 */
static void cheb_product(CIPHER res, CIPHER a, CIPHER b, CIPHER sub) {
  CIPHERTEXT prod;
  new_ciph(&prod);
  Rt_mul_rescale_ciph(&prod, a, b, true, NULL); /* Mul_ciph, Add_ciph(prod, prod), Rescale_ciph */
  if (sub)
    Sub_ciph(&prod, &prod, sub);
  else
    add_const(&prod, -1.0);
  Free_ciph_poly(res, 1);
  *res = prod;
}

/* Eval_chebyshev_ps on [-1, 1] (chebyshev_impl.c:502-678), in place */
static void eval_chebyshev(CIPHER ct, const double* coeff, uint32_t n_coeff, bool even) {
  SERIES   f = {(double*)coeff, n_coeff};
  uint32_t n = series_degree(&f), k = 0, m = 0;
  FMT_ASSERT(n >= 5, "series of degree below 5 are not supported");
  ps_degrees(n, &k, &m);
  if (even && (k & 1)) k += 1;
  CHEB_BASIS b = {(CIPHERTEXT*)calloc(k, sizeof(CIPHERTEXT)), (CIPHERTEXT*)calloc(m, sizeof(CIPHERTEXT)), k, m};
  Copy_ciph(&b.t[0], ct);
  for (uint32_t i = 2; i <= k; ++i) {
    if (even && (i & 1)) continue; /* an even series needs no odd T_i */
    uint32_t h1 = i / 2, h2 = i - h1;
    if (even && !(i & 1) && (i & (i - 1)) && (h1 & 1)) h1 += 1, h2 = i - h1; /* T_i = 2 T_{i/2+1} T_{i/2-1} - T_2 */
    CIPHER sub = (i & 1) ? &b.t[0] : (h1 == h2 ? NULL : &b.t[1]);
    cheb_product(&b.t[i - 1], &b.t[h1 - 1], &b.t[h2 - 1], sub);
  }
  for (uint32_t i = 1; i < k; ++i) { /* all at the level of T_k */
    if (even && (i & 1)) continue;
    if (Level(&b.t[i - 1]) > Level(&b.t[k - 1])) set_level(&b.t[i - 1], Level(&b.t[k - 1]));
  }
  Copy_ciph(&b.t2[0], &b.t[k - 1]);
  for (uint32_t i = 1; i < m; ++i) cheb_product(&b.t2[i], &b.t2[i - 1], &b.t2[i - 1], NULL);
  CIPHERTEXT top; /* T_{k (2^m - 1)} */
  new_ciph(&top);
  Copy_ciph(&top, &b.t2[0]);
  for (uint32_t i = 1; i < m; ++i) cheb_product(&top, &top, &b.t2[i], &b.t2[0]);

  uint32_t span = k * (1u << (m - 1)) - k;
  SERIES   f2   = series_copy(&f, 2 * span + k + 1); /* + T_{k (2^m - 1)}: monic, so every quotient is */
  f2.v[f2.n - 1] = 1.0;
  CIPHERTEXT out;
  new_ciph(&out);
  eval_ps(&out, &b, &f2, m);
  Sub_ciph(&out, &out, &top);
  Free_ciph_poly(ct, 1);
  *ct = out;

  free(f2.v);
  Free_ciph_poly(&top, 1);
  Free_ciph_poly(b.t, k);
  Free_ciph_poly(b.t2, m);
  free(b.t);
  free(b.t2);
}

/* Eval_approx_mod (bootstrap.c:1524-1559): the series, then the double-angle steps */
static void eval_approx_mod(CIPHER ct);
/* The real and the imaginary half of a fully packed ciphertext go through the same series independently: the second
 * is issued on the library's second lane, so that its kernels (one polynomial each, too small for the machine)
 * overlap with the first's.  RT_HIP_ONE_LANE=1 issues them one after the other, and so does a program that runs
 * on several host threads (a second thread has called into the runtime): their streams fill the machine already,
 * and twice as many streams as threads share the hardware's few queues (three threads: 0.66 s per ResNet-20 image
 * with the second lanes, 0.55 s without).  A second stream that was used before the other threads came still costs
 * them -- the driver then serves two of the threads' streams through one queue (0.69 s) -- so a program that will
 * run images on several threads lets every thread call in once (Rt_sync() will do) before the first bootstrap; the
 * reference's driver, whose first image is already inside its parallel loop, does so by itself. */
static void eval_approx_mod_pair(CIPHER a, CIPHER b) {
  static int one_lane = -1;
  if (one_lane < 0) one_lane = getenv("RT_HIP_ONE_LANE") && atoi(getenv("RT_HIP_ONE_LANE")) != 0;
  Rt_plaintexts_settle(); /* the second stream may be encoding weight plaintexts ahead of the program */
  if (one_lane || Rt_lane_count() > 1) {
    if (!one_lane) ACE_OK(ace_fork_release(RT_CTX)); /* a second stream from before the other threads came */
    eval_approx_mod(a);
    eval_approx_mod(b);
    return;
  }
  ACE_OK(ace_fork(RT_CTX));
  eval_approx_mod(b);
  ACE_OK(ace_fork_switch(RT_CTX));
  eval_approx_mod(a);
  ACE_OK(ace_join(RT_CTX));
}
static void eval_approx_mod(CIPHER ct) {
  const SIN_POLY* p = sin_poly();
  if (p->even) add_const(ct, -1.0 / (4.0 * p->k_bound));
  eval_chebyshev(ct, p->coeff, p->n_coeff, p->even);
  int32_t r = (int32_t)p->double_angle;
  for (int32_t j = 1; j <= r; ++j) { /* Mul_ciph, Add_ciph(ct, ct), Add_const, Rescale_ciph (bootstrap.c:1508-1515) */
    const double scalar = -1.0 / pow(2.0 * M_PI, pow(2.0, j - r));
    Rt_mul_rescale_ciph(ct, ct, ct, true, &scalar);
  }
}

/* ---- the whole procedure (bootstrap.c:1561-1830, cipher.c:565-767) ---------------------------------- */
/* level 0 of ct, in coefficient form, repeated over `raise_level` primes and transformed (the modulus raise) */
static void raise_modulus(CIPHER out, CIPHER ct, uint32_t raise_level, uint32_t slots) {
  CIPHERTEXT low;
  new_ciph(&low);
  Copy_ciph(&low, ct);
  while (low._sf_degree > 1) rescale(&low);
  if (low._c0_poly._is_ntt) Conv_ntt2poly_inplace(&low._c0_poly);
  if (low._c1_poly._is_ntt) Conv_ntt2poly_inplace(&low._c1_poly);
  Free_ciph_poly(out, 1);
  new_ciph(out);
  Alloc_poly_data(&out->_c0_poly, G.N, raise_level, 0);
  Alloc_poly_data(&out->_c1_poly, G.N, raise_level, 0);
  out->_scaling_factor = low._scaling_factor;
  out->_sf_degree      = low._sf_degree;
  out->_slots          = slots;
  Transform_values_from_level0(&out->_c0_poly, &low._c0_poly);
  Transform_values_from_level0(&out->_c1_poly, &low._c1_poly);
  Conv_poly2ntt_inplace(&out->_c0_poly);
  Conv_poly2ntt_inplace(&out->_c1_poly);
  Free_ciph_poly(&low, 1);
}

/* the scaling left after slots-to-coefficients: q0 / scale as a power of two (bootstrap.c:1790-1812) */
static void finish(CIPHER res) {
  int32_t     deg   = (int32_t)round(log2((double)G.q[0]._val / G.sc));
  const char* env   = getenv("RT_BTS_CLEAR_IMAG");
  bool        clear = env && atoi(env) != 0 && deg >= 1;
  if (clear) {
    CIPHERTEXT conj;
    new_ciph(&conj);
    rotate_into(&conj, res, (int32_t)(2 * G.N - 1));
    Add_ciph(res, res, &conj);
    Free_ciph_poly(&conj, 1);
    deg -= 1;
  }
  uint64_t ratio = (uint64_t)pow(2.0, deg);
  if (!clear || ratio > 1) mul_integer(res, res, ratio);
  while (res->_sf_degree > 1) rescale(res);
}

static CIPHER eval_bootstrap(CIPHER res, CIPHER ct, uint32_t level_after_bts, uint32_t num_slots) {
  NEED_CTX();
  FMT_ASSERT(Level(ct) > 0, "Input cipher level is exhausted");
  uint32_t    slots = num_slots ? num_slots : (ct->_slots ? ct->_slots : (uint32_t)(G.N / 2));
  BTS_PRECOM* pre   = setup(slots);
  keygen(pre);
  uint32_t depth = bootstrap_depth(pre);
  if (!level_after_bts) level_after_bts = (uint32_t)G.L - depth;
  FMT_ASSERT(level_after_bts <= G.L - depth, "The level set after bootstrapping is excessively high");
  if (Level(ct) - (ct->_sf_degree - 1) >= level_after_bts) { /* nothing to gain */
    Copy_ciph(res, ct);
    return res;
  }
  bool       full = slots == G.N / 2;
  CIPHERTEXT work, conj, sub;
  new_ciph(&work), new_ciph(&conj), new_ciph(&sub);
  raise_modulus(&work, ct, level_after_bts + depth, slots);

  if (!full) { /* sparse packing: sum the N / (2 slots) copies */
    for (uint32_t j = 1; j < G.N / (2 * slots); j <<= 1) {
      rotate_into(&conj, &work, (int32_t)(j * slots));
      Add_ciph(&work, &work, &conj);
    }
  }
  coeff_slots_transform(&work, pre, true);
  rotate_into(&conj, &work, (int32_t)(2 * G.N - 1));
  if (full) { /* real and imaginary parts are reduced separately */
    Sub_ciph(&sub, &work, &conj);
    Add_ciph(&work, &work, &conj);
    Mul_mono_ciph(&sub, &sub, (uint32_t)(3 * G.N / 2));
    while (work._sf_degree > 1) {
      rescale(&work);
      rescale(&sub);
    }
    eval_approx_mod_pair(&work, &sub);
    Mul_mono_ciph(&sub, &sub, (uint32_t)(G.N / 2));
    Add_ciph(&work, &work, &sub);
  } else {
    Add_ciph(&work, &work, &conj);
    while (work._sf_degree > 1) rescale(&work);
    eval_approx_mod(&work);
  }
  coeff_slots_transform(&work, pre, false);
  if (!full) {
    rotate_into(&conj, &work, (int32_t)slots);
    Add_ciph(&work, &work, &conj);
  }
  finish(&work);

  Free_ciph_poly(&conj, 1);
  Free_ciph_poly(&sub, 1);
  if (res->_c0_poly._data) Free_ciph_poly(res, 1);
  *res = work;
  return res;
}

CIPHER Eval_bootstrap_ciph(CIPHER res, CIPHER ct, uint32_t level_after_bts, uint32_t num_slots) {
  RTLIB_TM_START(RTM_BOOTSTRAP, rtm);
  eval_bootstrap(res, ct, level_after_bts, num_slots);
  RTLIB_TM_END(RTM_BOOTSTRAP, rtm);
  return res;
}

/* ---- the stages on their own (cipher.c:585-767) ------------------------------------------------------
 * The same pieces as above, cut where the compiler's staged operators cut them.  The imaginary half of a fully
 * packed input lives here between the first two calls. */
static __thread struct {
  bool       active, full;
  uint32_t   slots;
  CIPHERTEXT sub;
} Stage;
static void stage_clear(void) {
  if (Stage.sub._c0_poly._data) Free_ciph_poly(&Stage.sub, 1);
  memset(&Stage, 0, sizeof(Stage));
}
static uint32_t stage_slots(CIPHER ct, uint32_t num_slots) {
  return num_slots ? num_slots : (ct->_slots ? ct->_slots : (uint32_t)(G.N / 2));
}
static CIPHER stage_result(CIPHER res, CIPHER ct, CIPHERTEXT* work) { /* res takes over work's polynomials */
  if (res->_c0_poly._data && res != ct) Free_ciph_poly(res, 1);
  if (res == ct) Free_ciph_poly(ct, 1);
  *res = *work;
  return res;
}

CIPHER Eval_bootstrap_coeffs_to_slots_ciph(CIPHER res, CIPHER ct, uint32_t num_slots) {
  NEED_CTX();
  stage_clear();
  uint32_t    slots = stage_slots(ct, num_slots);
  BTS_PRECOM* pre   = setup(slots);
  keygen(pre);
  bool       full = slots == G.N / 2;
  CIPHERTEXT work, conj;
  new_ciph(&work), new_ciph(&conj);
  raise_modulus(&work, ct, (uint32_t)G.L, slots);
  if (!full) {
    for (uint32_t j = 1; j < G.N / (2 * slots); j <<= 1) {
      rotate_into(&conj, &work, (int32_t)(j * slots));
      Add_ciph(&work, &work, &conj);
    }
  }
  coeff_slots_transform(&work, pre, true);
  rotate_into(&conj, &work, (int32_t)(2 * G.N - 1));
  if (full) {
    new_ciph(&Stage.sub);
    Sub_ciph(&Stage.sub, &work, &conj);
    Add_ciph(&work, &work, &conj);
    Mul_mono_ciph(&Stage.sub, &Stage.sub, (uint32_t)(3 * G.N / 2));
    while (work._sf_degree > 1) {
      rescale(&work);
      rescale(&Stage.sub);
    }
  } else {
    Add_ciph(&work, &work, &conj);
    while (work._sf_degree > 1) rescale(&work);
  }
  Stage.active = true;
  Stage.full   = full;
  Stage.slots  = slots;
  Free_ciph_poly(&conj, 1);
  return stage_result(res, ct, &work);
}

CIPHER Eval_bootstrap_eval_mod_ciph(CIPHER res, CIPHER ct, uint32_t num_slots) {
  NEED_CTX();
  uint32_t    slots = stage_slots(ct, num_slots);
  BTS_PRECOM* pre   = setup(slots);
  keygen(pre);
  CIPHERTEXT work;
  new_ciph(&work);
  Copy_ciph(&work, ct);
  if (Stage.active && Stage.full && Stage.sub._c0_poly._data && Stage.slots == slots) {
    eval_approx_mod_pair(&work, &Stage.sub);
    Mul_mono_ciph(&Stage.sub, &Stage.sub, slots);
    Add_ciph(&work, &work, &Stage.sub);
    Free_ciph_poly(&Stage.sub, 1);
    new_ciph(&Stage.sub);
  } else {
    while (work._sf_degree > 1) rescale(&work);
    eval_approx_mod(&work);
  }
  return stage_result(res, ct, &work);
}

CIPHER Eval_bootstrap_slots_to_coeffs_ciph(CIPHER res, CIPHER ct, uint32_t num_slots) {
  NEED_CTX();
  uint32_t    slots = stage_slots(ct, num_slots);
  BTS_PRECOM* pre   = setup(slots);
  keygen(pre);
  CIPHERTEXT work, rot;
  new_ciph(&work), new_ciph(&rot);
  Copy_ciph(&work, ct);
  coeff_slots_transform(&work, pre, false);
  if (slots != G.N / 2) {
    rotate_into(&rot, &work, (int32_t)slots);
    Add_ciph(&work, &work, &rot);
    Free_ciph_poly(&rot, 1);
  }
  finish(&work);
  stage_clear();
  return stage_result(res, ct, &work);
}

CIPHER Bootstrap(CIPHER res, CIPHER ct, uint32_t level_after_bts) {
  return Eval_bootstrap_ciph(res, ct, level_after_bts, ct->_slots);
}
