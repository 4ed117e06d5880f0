/* rt_ckks.c -- the scheme-level part of the host runtime: key generation, plaintext
 * encoding entry points, encryption, decryption and decoding, program inputs and
 * outputs.  Polynomial arithmetic runs on the device through ace_hip.h; what stays
 * on the host is sampling, the few-word constants of single-value plaintexts and the
 * multi-precision reconstruction of decoded coefficients.
 */
#include <complex.h>
#include <math.h>
#include <sys/random.h>

#include "rt_internal.h"

/* ---- random numbers: xoshiro256** seeded through splitmix64 ---------------------------------
 * One generator per host thread, as in the reference's OpenMP build (util/src/prng.c:13-16).  The thread that
 * generates the keys seeds its own; any other thread's is seeded the first time it draws: from the keys' seed and
 * the thread's ordinal when that seed was given (reproducible runs), else from the operating system. */
static __thread uint64_t Rng[4];
static __thread bool     Rng_ready;
static uint64_t          Master_seed; /* the seed given to Rt_generate_keys, 0: none */
static uint64_t splitmix(uint64_t* s) {
  uint64_t z = (*s += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
static void rng_seed(uint64_t seed) {
  for (int i = 0; i < 4; ++i) Rng[i] = splitmix(&seed);
}
static inline uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
static void rng_first_use(void) {
  const char* env  = getenv("RT_HIP_SEED");
  uint64_t    seed = Master_seed ? Master_seed : env ? strtoull(env, NULL, 0) : 0;
  if (seed) {
    seed += 0xD1342543DE82EF95ull * Rt_this_lane()->ordinal;
    rng_seed(seed);
  } else {
    FMT_ASSERT(getrandom(Rng, sizeof(Rng), 0) == (ssize_t)sizeof(Rng) && (Rng[0] | Rng[1] | Rng[2] | Rng[3]),
               "no entropy source");
  }
  Rng_ready = true;
}
static uint64_t rng_next(void) {
  if (!Rng_ready) rng_first_use();
  uint64_t r = rotl(Rng[1] * 5, 7) * 9, t = Rng[1] << 17;
  Rng[2] ^= Rng[0];
  Rng[3] ^= Rng[1];
  Rng[1] ^= Rng[2];
  Rng[0] ^= Rng[3];
  Rng[2] ^= t;
  Rng[3] = rotl(Rng[3], 45);
  return r;
}
static uint64_t rng_below(uint64_t bound) { /* unbiased, by rejection */
  uint64_t lim = UINT64_MAX - UINT64_MAX % bound;
  for (;;) {
    uint64_t v = rng_next();
    if (v < lim) return v % bound;
  }
}

/* Sample_triangle (util/src/random_sample.c:80-99): -1, 1 with probability 1/4 each, else 0 */
static void sample_triangle(int64_t* v, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    uint64_t r = rng_next() & 3;
    v[i] = r == 0 ? -1 : r == 1 ? 1 : 0;
  }
}
/* Sample_ternary (random_sample.c:101-156): weight 0 draws every coefficient uniformly from
 * {-1, 0, 1}; otherwise exactly `weight` coefficients are +-1, redrawn until the +1s number
 * weight/2 to within one */
static void sample_ternary(int64_t* v, size_t n, size_t weight) {
  if (weight == 0) {
    for (size_t i = 0; i < n; ++i) v[i] = (int64_t)rng_below(3) - 1;
    return;
  }
  if (weight > n) weight = n;
  for (;;) {
    size_t ones = 0;
    memset(v, 0, n * sizeof(int64_t));
    for (size_t done = 0; done < weight;) {
      size_t i = (size_t)rng_below(n);
      if (v[i]) continue;
      v[i] = (rng_next() & 1) ? 1 : -1;
      ones += v[i] == 1;
      ++done;
    }
    if (ones + 1 >= weight / 2 && ones <= weight / 2 + 1) return;
  }
}

void Rt_sample_ternary(int64_t* v, size_t n, size_t hamming_weight) { sample_ternary(v, n, hamming_weight); }

/* ---- small helpers over the device ------------------------------------------------------------ */
static uint64_t Seed, Stream; /* of the device-side uniform sampler: one stream per polynomial */

/* signed small coefficients -> residues of `level` Q limbs (+ the P limbs), NTT form, in dev */
static void small_to_dev(int64_t* dev, const int64_t* v, size_t level, bool with_p) {
  size_t  T = level + (with_p ? G.K : 0);
  int32_t idx[128];
  for (size_t t = 0; t < T; ++t) idx[t] = (int32_t)(t < level ? t : G.L + (t - level));
  ACE_OK(ace_expand_small(RT_CTX, dev, v, level, with_p));
  ACE_OK(ace_ntt(RT_CTX, dev, dev, idx, T, 1, 0));
}
/* uniform residues, drawn on the device: a uniform polynomial is uniform in NTT form too */
static void uniform_to_dev(int64_t* dev, size_t level, bool with_p) {
  ACE_OK(ace_sample_uniform(RT_CTX, dev, level, with_p, Seed, __atomic_fetch_add(&Stream, 1, __ATOMIC_RELAXED)));
}

/* ---- keys (ckks/src/key_gen.c:127-262) ----------------------------------------------------------- */
/* a switch key taking a polynomial that multiplies s_src to a pair that decrypts under s_res (both: device,
 * L+k limbs, NTT), built in place in HBM: per digit b = -a*s_res + e + P*s_src on the digit's limbs */
static void make_switch_key(SWITCH_KEY* key, const int64_t* s_res, const int64_t* s_src) {
  size_t   n = G.N, T = G.L + G.K, ps = ace_part_size(RT_CTX);
  int64_t* dev = Rt_dev_alloc_raw(2 * G.parts * T * n);
  int64_t *e = Rt_dev_alloc_raw(T * n), *t = Rt_dev_alloc_raw(n);
  int64_t* small = (int64_t*)malloc(n * sizeof(int64_t));
  for (size_t d = 0; d < G.parts; ++d) {
    int64_t *b = dev + 2 * d * T * n, *a = b + T * n;
    uniform_to_dev(a, G.L, true);
    sample_triangle(small, n);
    small_to_dev(e, small, G.L, true);
    ACE_OK(ace_poly_mul(RT_CTX, b, a, s_res, G.L, 1));
    ACE_OK(ace_poly_sub(RT_CTX, b, e, b, G.L, 1));
    for (size_t i = d * ps; i < (d + 1) * ps && i < G.L; ++i) {
      uint64_t q = (uint64_t)G.q[i]._val, pm = 1; /* P mod q_i */
      for (size_t j = 0; j < G.K; ++j) pm = (uint64_t)((unsigned __int128)pm * ((uint64_t)G.p[j]._val % q) % q);
      ACE_OK(ace_hw_modmul_scalar(RT_CTX, t, s_src + i * n, (int64_t)pm, i, n));
      ACE_OK(ace_hw_modadd(RT_CTX, b + i * n, b + i * n, t, i, n));
    }
  }
  free(small);
  Rt_dev_free(e);
  Rt_dev_free(t);
  Rt_install_key_dev(key, dev);
}

/* sigma_k on signed coefficients: X^i -> X^(i k mod 2N), negated past N */
static void automorphism_small(int64_t* out, const int64_t* v, uint64_t k) {
  size_t n = G.N;
  for (size_t i = 0; i < n; ++i) {
    uint64_t j = (uint64_t)i * k % (2 * n);
    out[j % n] = j >= n ? -v[i] : v[i];
  }
}
static uint64_t inv_mod_pow2(uint64_t k, uint64_t m) { /* k odd, m a power of two */
  uint64_t x = k;                                        /* Newton: doubles the correct bits */
  for (int i = 0; i < 6; ++i) x *= 2 - k * x;
  return x & (m - 1);
}

void Rt_generate_rotation_key(int32_t rot_idx) {
  FMT_ASSERT(G.secret_ntt, "Rt_generate_keys() has not run");
  Rt_shared_lock(); /* one key at a time; the key is whole on the device before another thread can find it */
  size_t   n = G.N, T = G.L + G.K;
  ROT_KEY* entry = Rt_rot_entry(rot_idx);
  uint32_t k = entry->auto_idx;
  /* "fast" key: the evaluator switches the un-rotated c1 and applies the automorphism last, so the
   * key leads from s to sigma_k^-1(s) (key_gen.c:216-262) */
  int64_t* rs = (int64_t*)malloc(n * sizeof(int64_t));
  automorphism_small(rs, G.secret_small, inv_mod_pow2(k, 2 * n));
  int64_t* s_res = Rt_dev_alloc_raw(T * n);
  small_to_dev(s_res, rs, G.L, true);
  make_switch_key(&Rt_find_rot(rot_idx)->swk, s_res, G.secret_ntt);
  free(rs);
  Rt_dev_free(s_res);
  Rt_shared_unlock();
}

void Rt_generate_keys(uint64_t seed) {
  NEED_CTX();
  if (!seed) {
    const char* env = getenv("RT_HIP_SEED");
    seed = env ? strtoull(env, NULL, 0) : 0;
  }
  Master_seed = seed;
  if (seed) {
    rng_seed(seed); /* a fixed seed: reproducible runs for tests and benchmarks only */
  } else {
    /* no seed given: the whole generator state comes from the operating system's entropy pool (the reference seeds
     * its generator from /dev/urandom, util/src/prng.c:56-109), so the secret cannot be found by a seed search */
    if (getrandom(Rng, sizeof(Rng), 0) != (ssize_t)sizeof(Rng)) {
      FILE* f = fopen("/dev/urandom", "rb");
      FMT_ASSERT(f && fread(Rng, sizeof(Rng), 1, f) == 1, "no entropy source for key generation");
      fclose(f);
    }
    FMT_ASSERT(Rng[0] | Rng[1] | Rng[2] | Rng[3], "entropy source returned zeros");
    seed = rng_next(); /* the device-side stream of public uniform polynomials */
  }
  Seed      = seed;
  Stream    = 0;
  Rng_ready = true;
  Rt_ckks_finalize(); /* a second call replaces the keys */
  CKKS_PARAMS* prm = Get_context_params();
  size_t       n = G.N, T = G.L + G.K, hw = prm->_hamming_weight;
  G.secret_small = (int64_t*)malloc(n * sizeof(int64_t));
  sample_ternary(G.secret_small, n, hw);
  G.secret_ntt = Rt_dev_alloc_raw(T * n);
  small_to_dev(G.secret_ntt, G.secret_small, G.L, true);
  /* public key: pk1 = a, pk0 = -a s + e  (L limbs) */
  G.pk0 = Rt_dev_alloc_raw(G.L * n);
  G.pk1 = Rt_dev_alloc_raw(G.L * n);
  int64_t* small = (int64_t*)malloc(n * sizeof(int64_t));
  int64_t* e     = Rt_dev_alloc_raw(G.L * n);
  uniform_to_dev(G.pk1, G.L, false);
  sample_triangle(small, n);
  small_to_dev(e, small, G.L, false);
  ACE_OK(ace_poly_mul(RT_CTX, G.pk0, G.pk1, G.secret_ntt, G.L, 0));
  ACE_OK(ace_poly_sub(RT_CTX, G.pk0, e, G.pk0, G.L, 0));
  Rt_dev_free(e);
  free(small);
  /* relinearisation key: from s^2 to s */
  int64_t* s2 = Rt_dev_alloc_raw(T * n);
  ACE_OK(ace_poly_mul(RT_CTX, s2, G.secret_ntt, G.secret_ntt, G.L, 1));
  make_switch_key(&G.relin, G.secret_ntt, s2);
  Rt_dev_free(s2);
  for (size_t i = 0; i < prm->_num_rot_idx; ++i)
    if (!Rt_find_rot(prm->_rot_idxs[i])) Rt_generate_rotation_key(prm->_rot_idxs[i]); /* index 0 included: generated code asks for it */
  Rt_bootstrap_prepare();
}

void Rt_get_secret(int64_t* host_small) {
  FMT_ASSERT(G.secret_small, "Rt_generate_keys() has not run");
  memcpy(host_small, G.secret_small, G.N * sizeof(int64_t));
}
void Rt_get_public_key(int64_t* host_pk0, int64_t* host_pk1) {
  FMT_ASSERT(G.pk0, "Rt_generate_keys() has not run");
  ACE_OK(ace_download(RT_CTX, host_pk0, G.pk0, G.L * G.N));
  ACE_OK(ace_download(RT_CTX, host_pk1, G.pk1, G.L * G.N));
}

void Rt_ckks_finalize(void) {
  free(G.secret_small);
  if (G.secret_ntt) Rt_dev_free(G.secret_ntt);
  if (G.pk0) Rt_dev_free(G.pk0);
  if (G.pk1) Rt_dev_free(G.pk1);
  G.secret_small = NULL;
  G.secret_ntt = G.pk0 = G.pk1 = NULL;
}

/* ---- plaintexts ------------------------------------------------------------------------------------- */
static void init_plain(PLAIN plain, size_t level, double scale, uint32_t sf_degree, uint32_t slots) {
  POLY p = &plain->_poly;
  if (p->_data && (p->_num_primes != level || p->_num_primes_p != 0)) Free_poly_data(p);
  if (!p->_data) Alloc_poly_data(p, G.N, level, 0);
  plain->_scaling_factor = scale;
  plain->_sf_degree      = sf_degree;
  plain->_slots          = slots;
  p->_is_ntt             = true;
}

static void check_sf(uint32_t sf_degree, size_t level) {
  CKKS_PARAMS* prm = Get_context_params();
  FMT_ASSERT(sf_degree >= 1 && prm->_scaling_mod_size * sf_degree <
                                   prm->_first_mod_size + (level - 1) * prm->_scaling_mod_size,
             "invalid scaling factor for encode");
}

/* Encode_val (ckks/src/encoder.c:428-523): the residues of trunc(value * scale).  A product beyond
 * 61 bits is encoded divided by a power of two, which is multiplied back in modulo each prime. */
void Rt_encode_val_words(int64_t* res, double value, uint32_t level, double scale) {
  CKKS_PARAMS* prm = Get_context_params();
  FMT_ASSERT(level > 0 && level <= G.L, "level should not be larger than q_cnt");
  size_t bits = prm->_first_mod_size + (level - 1) * prm->_scaling_mod_size;
  FMT_ASSERT(scale > 0 && (uint32_t)log2(scale) < bits, "invalid scale for encode");
  if (value == 0.0) {
    memset(res, 0, level * sizeof(int64_t));
    return;
  }
  int32_t log_scale  = (int32_t)(log2(fabs(value * scale)));
  int32_t log_valid  = log_scale <= 61 ? log_scale : 61;
  int32_t log_approx = log_scale - log_valid;
  double  scaled     = value / pow(2, log_approx) * scale;
  FMT_ASSERT(scaled <= 9223372036854775807.0 && scaled >= -9223372036854775807.0,
             "encode %f with scale %f overflow, please choose a smaller scale", value, scale);
  FMT_ASSERT(log_scale + 1 < (int32_t)bits,
             "encode value out of range, please increase encoding level or increase first_mod_size & "
             "scale_mod_size or decrease scale of msg");
  int64_t v = (int64_t)scaled;
  for (uint32_t t = 0; t < level; ++t) {
    uint64_t q = (uint64_t)G.q[t]._val;
    int64_t  r = v % (int64_t)q;
    if (r < 0) r += (int64_t)q;
    uint64_t back = 1; /* 2^log_approx mod q, in steps of at most 60 bits */
    for (int32_t left = log_approx; left > 0;) {
      int32_t step = left <= 60 ? left : 60;
      back         = (uint64_t)((unsigned __int128)back * (((uint64_t)1 << step) % q) % q);
      left -= step;
    }
    res[t] = (int64_t)((unsigned __int128)(uint64_t)r * back % q);
  }
}

/* Encode_val_at_level (encoder.c:544-575): the same residue in every coefficient */
static void encode_value(PLAIN plain, double value, uint32_t sc_degree, uint32_t level) {
  if (level == 0) level = (uint32_t)G.L;
  FMT_ASSERT(level <= G.L, "level should not be larger than mul_depth + 1");
  check_sf(sc_degree, level);
  double scale = pow(G.sc, sc_degree);
  init_plain(plain, level, scale, sc_degree, G.N / 2);
  int64_t words[128];
  Rt_encode_val_words(words, value, level, scale);
  for (uint32_t t = 0; t < level; ++t) {
    int64_t* limb = plain->_poly._data + (size_t)t * G.N;
    ACE_OK(ace_zero(RT_CTX, limb, G.N));
    ACE_OK(ace_hw_modadd_scalar(RT_CTX, limb, limb, words[t], t, G.N));
  }
}

static void encode_vector(PLAIN plain, const double* re_im, size_t len, uint32_t sc_degree, uint32_t level) {
  if (level == 0) level = (uint32_t)G.L;
  FMT_ASSERT(level <= G.L, "level should not be larger than mul_depth + 1");
  init_plain(plain, level, pow(G.sc, sc_degree), sc_degree, G.N / 2);
  ACE_OK(ace_encode(RT_CTX, plain->_poly._data, re_im, len, 0, level, sc_degree, 0));
}
/* a plaintext of `level` limbs at scale degree sc_degree whose polynomial the caller fills in (NTT form) */
int64_t* Rt_plain_prepare(PLAIN plain, uint32_t sc_degree, uint32_t level) {
  if (level == 0) level = (uint32_t)G.L;
  FMT_ASSERT(level <= G.L, "level should not be larger than mul_depth + 1");
  init_plain(plain, level, pow(G.sc, sc_degree), sc_degree, G.N / 2);
  return plain->_poly._data;
}
/* real-valued messages go to the device as they are (doubles or floats) and are widened there */
void Rt_encode_real(PLAIN plain, const void* values, int is_f32, size_t len, uint32_t sc_degree, uint32_t level) {
  if (level == 0) level = (uint32_t)G.L;
  FMT_ASSERT(level <= G.L, "level should not be larger than mul_depth + 1");
  init_plain(plain, level, pow(G.sc, sc_degree), sc_degree, G.N / 2);
  ACE_OK(ace_encode_real(RT_CTX, plain->_poly._data, values, is_f32, len, 0, level, sc_degree, 0));
}

/* n_vec real-valued vectors into the polynomials dev_base + v * stride (level limbs each, NTT form) */
void Rt_encode_real_batch(int64_t* dev_base, size_t stride, const void* const* values, int is_f32, size_t len,
                          size_t n_vec, uint32_t sc_degree, uint32_t level) {
  if (level == 0) level = (uint32_t)G.L;
  FMT_ASSERT(level <= G.L, "level should not be larger than mul_depth + 1");
  ACE_OK(ace_encode_real_batch(RT_CTX, dev_base, stride, values, is_f32, len, n_vec, 0, level, sc_degree, 0));
}

void Encode_double(PLAIN plain, double* input, size_t len, uint32_t sc_degree, uint32_t level) {
  if (len == 1) {
    encode_value(plain, *input, sc_degree, level);
    return;
  }
  Rt_encode_real(plain, input, 0, len, sc_degree, level);
}
void Encode_float(PLAIN plain, float* input, size_t len, uint32_t sc_degree, uint32_t level) {
  if (len == 1) {
    encode_value(plain, (double)*input, sc_degree, level);
    return;
  }
  Rt_encode_real(plain, input, 1, len, sc_degree, level);
}
void Encode_dcmplx(PLAIN plain, DCMPLX* input, size_t len, uint32_t sc_degree, uint32_t level) {
  encode_vector(plain, (const double*)input, len, sc_degree, level);
}
void Encode_double_mask(PLAIN plain, double cst, size_t len, uint32_t sc_degree, uint32_t level) {
  double* v = (double*)calloc(2 * len, sizeof(double));
  for (size_t i = 0; i < len; ++i) v[2 * i] = cst;
  encode_vector(plain, v, len, sc_degree, level);
  free(v);
}
void Encode_float_mask(PLAIN plain, float cst, size_t len, uint32_t sc_degree, uint32_t level) {
  Encode_double_mask(plain, (double)cst, len, sc_degree, level);
}
void Encode_dcmplx_ext(PLAIN plain, DCMPLX* input, size_t len, uint32_t level, uint32_t p_cnt) {
  if (level == 0) level = (uint32_t)G.L;
  FMT_ASSERT(level <= G.L, "level should not be larger than mul_depth + 1");
  FMT_ASSERT(p_cnt == 0 || p_cnt == G.K, "extended plaintexts carry all P limbs");
  POLY p = &plain->_poly;
  if (p->_data && (p->_num_primes != level || p->_num_primes_p != p_cnt)) Free_poly_data(p);
  if (!p->_data) Alloc_poly_data(p, G.N, level, p_cnt);
  plain->_scaling_factor = G.sc;
  plain->_sf_degree      = 1;
  plain->_slots          = G.N / 2;
  p->_is_ntt             = true;
  ACE_OK(ace_encode(RT_CTX, p->_data, (const double*)input, len, 0, level, 1, p_cnt));
}
/* Encode_float_with_scale (ckks/src/plain.c:104-123): the scale is given, the degree recorded is the least
 * power of the scaling factor that reaches it (Get_approx_sf_degree, encoder.c:328-335) */
void Encode_float_with_scale(PLAIN plain, float* input, size_t len, double scale, uint32_t level) {
  NEED_CTX();
  if (level == 0) level = (uint32_t)G.L;
  FMT_ASSERT(level <= G.L, "level should not be larger than mul_depth + 1");
  FMT_ASSERT(scale > 0 && G.sc != 1, "invalid scale for encode");
  uint32_t deg = (uint32_t)floor(log2(scale) / log2(G.sc));
  if (scale > pow(G.sc, deg)) ++deg;
  init_plain(plain, level, scale, deg, G.N / 2);
  if (len == 1) { /* Encode_val_at_level_with_scale (encoder.c:580-605) */
    int64_t words[128];
    Rt_encode_val_words(words, (double)*input, level, scale);
    for (uint32_t t = 0; t < level; ++t) {
      int64_t* limb = plain->_poly._data + (size_t)t * G.N;
      ACE_OK(ace_zero(RT_CTX, limb, G.N));
      ACE_OK(ace_hw_modadd_scalar(RT_CTX, limb, limb, words[t], t, G.N));
    }
    return;
  }
  double* v = (double*)calloc(2 * len, sizeof(double));
  for (size_t i = 0; i < len; ++i) v[2 * i] = (double)input[i];
  ACE_OK(ace_encode_scaled(RT_CTX, plain->_poly._data, v, len, 0, level, scale, 0));
  free(v);
}
/* Encode_single_double (ckks/src/plain.c:139-147): `level` host words */
void Encode_single_double(int64_t* res, double input, uint32_t sc_degree, uint32_t level) {
  NEED_CTX();
  Rt_encode_val_words(res, input, level, pow(G.sc, sc_degree));
}
void Encode_single_float(int64_t* res, float input, uint32_t sc_degree, uint32_t level) {
  Encode_single_double(res, (double)input, sc_degree, level);
}
void Free_plain_poly(PLAIN plain) { Free_poly_data(&plain->_poly); }

/* result shaped like c at the lower of the two levels (ckks/src/cipher.c:58-84) */
static void shape_like(CIPHER res, CIPHER c, PLAIN plain, double sf, uint32_t deg) {
  size_t level = Level(c), pl = plain->_poly._num_primes;
  if (res != c) {
    Init_poly(&res->_c0_poly, &c->_c0_poly);
    Init_poly(&res->_c1_poly, &c->_c1_poly);
  }
  res->_scaling_factor  = sf;
  res->_sf_degree       = deg;
  res->_slots           = c->_slots;
  res->_c0_poly._is_ntt = res->_c1_poly._is_ntt = true;
  if (level > pl) level = pl;
  Set_poly_level(&res->_c0_poly, level);
  Set_poly_level(&res->_c1_poly, level);
}
void Init_ciph_same_scale_plain(CIPHER res, CIPHER c, PLAIN plain) {
  shape_like(res, c, plain, c->_scaling_factor, c->_sf_degree);
}
void Init_ciph_up_scale_plain(CIPHER res, CIPHER c, PLAIN plain) {
  shape_like(res, c, plain, c->_scaling_factor * plain->_scaling_factor, c->_sf_degree + plain->_sf_degree);
}

CIPHER Add_plain(CIPHER res, CIPHER c, PLAIN plain) {
  FMT_ASSERT(c->_scaling_factor == plain->_scaling_factor, "Scaling factors are not equal.");
  Init_ciph_same_scale_plain(res, c, plain);
  size_t level = Level(res), n = G.N;
  ACE_OK(ace_poly_add(RT_CTX, res->_c0_poly._data, c->_c0_poly._data, plain->_poly._data, level, 0));
  Rt_dev_copy(res->_c1_poly._data, c->_c1_poly._data, level * n);
  return res;
}
CIPHER Mul_plain(CIPHER res, CIPHER c, PLAIN plain) {
  Init_ciph_up_scale_plain(res, c, plain);
  size_t level = Level(res);
  ACE_OK(ace_poly_mul(RT_CTX, res->_c0_poly._data, c->_c0_poly._data, plain->_poly._data, level, 0));
  ACE_OK(ace_poly_mul(RT_CTX, res->_c1_poly._data, c->_c1_poly._data, plain->_poly._data, level, 0));
  return res;
}

/* ---- encryption / decryption (ckks/src/encryptor.c:19-75, decryptor.c) ------------------------------- */
CIPHER Encrypt(CIPHER res, PLAIN plain) {
  NEED_CTX();
  if (!G.pk0) Rt_generate_keys(0);
  POLY pt = &plain->_poly;
  FMT_ASSERT(pt->_num_primes_p == 0, "Encrypt_msg: plain should not be extended");
  size_t level = pt->_num_primes, n = G.N;
  Init_poly(&res->_c0_poly, pt);
  Init_poly(&res->_c1_poly, pt);
  res->_scaling_factor = plain->_scaling_factor;
  res->_sf_degree      = plain->_sf_degree;
  res->_slots          = plain->_slots;
  int64_t* small = (int64_t*)malloc(n * sizeof(int64_t));
  int64_t *u = Rt_dev_alloc(level * n), *e = Rt_dev_alloc(level * n);
  sample_triangle(small, n);
  small_to_dev(u, small, level, false);
  /* c0 = pk0 u + e1 + m ; c1 = pk1 u + e2 */
  sample_triangle(small, n);
  small_to_dev(e, small, level, false);
  ACE_OK(ace_poly_mul(RT_CTX, res->_c0_poly._data, G.pk0, u, level, 0));
  ACE_OK(ace_poly_add(RT_CTX, res->_c0_poly._data, res->_c0_poly._data, e, level, 0));
  ACE_OK(ace_poly_add(RT_CTX, res->_c0_poly._data, res->_c0_poly._data, pt->_data, level, 0));
  sample_triangle(small, n);
  small_to_dev(e, small, level, false);
  ACE_OK(ace_poly_mul(RT_CTX, res->_c1_poly._data, G.pk1, u, level, 0));
  ACE_OK(ace_poly_add(RT_CTX, res->_c1_poly._data, res->_c1_poly._data, e, level, 0));
  res->_c0_poly._is_ntt = res->_c1_poly._is_ntt = true;
  free(small);
  Rt_dev_free(u);
  Rt_dev_free(e);
  return res;
}

void Rt_decrypt(PLAIN res, CIPHER c) {
  FMT_ASSERT(G.secret_ntt, "Rt_generate_keys() has not run");
  size_t level = Level(c);
  init_plain(res, level, c->_scaling_factor, c->_sf_degree, c->_slots);
  ACE_OK(ace_poly_mul(RT_CTX, res->_poly._data, c->_c1_poly._data, G.secret_ntt, level, 0));
  ACE_OK(ace_poly_add(RT_CTX, res->_poly._data, res->_poly._data, c->_c0_poly._data, level, 0));
}

/* ---- decoding (ckks/src/encoder.c:657-704): Reconstruct, the conversion to double and the embedding run on the
 * device (ace_decode); only the slots' complex numbers come back ------------------------------------------ */
void Rt_decode(DCMPLX* res, PLAIN plain) {
  POLY     p     = &plain->_poly;
  uint32_t slots = plain->_slots ? plain->_slots : (uint32_t)(G.N / 2);
  FMT_ASSERT(p->_num_primes_p == 0, "decoding an extended plaintext is not supported");
  ACE_OK(ace_decode(RT_CTX, (double*)res, p->_data, p->_num_primes, p->_is_ntt, slots, plain->_scaling_factor));
}

DCMPLX* Get_dcmplx_msg_from_plain(PLAIN plain) {
  uint32_t slots = plain->_slots ? plain->_slots : G.N / 2;
  DCMPLX*  vec   = (DCMPLX*)malloc(slots * sizeof(DCMPLX));
  Rt_decode(vec, plain);
  return vec;
}
double* Get_msg_from_plain(PLAIN plain) {
  uint32_t slots = plain->_slots ? plain->_slots : G.N / 2;
  DCMPLX*  vec   = Get_dcmplx_msg_from_plain(plain);
  double*  data  = (double*)malloc(slots * sizeof(double));
  for (uint32_t i = 0; i < slots; ++i) data[i] = creal(vec[i]);
  free(vec);
  return data;
}

/* ---- runtime validation aids (ckks/src/cipher.c:188-240, common/src/rt_validate.c:16-55) ------------- */
DCMPLX* Get_msg_with_imag(CIPHER c) {
  FMT_ASSERT(c->_c0_poly._num_primes_p == 0, "Get_msg: extended ciphertexts are not supported");
  PLAINTEXT pt;
  memset(&pt, 0, sizeof(pt));
  Rt_decrypt(&pt, c);
  DCMPLX* v = Get_dcmplx_msg_from_plain(&pt);
  Free_plain_poly(&pt);
  return v;
}
double* Get_msg(CIPHER c) {
  uint32_t slots = c->_slots ? c->_slots : G.N / 2;
  DCMPLX*  v     = Get_msg_with_imag(c);
  double*  r     = (double*)malloc(slots * sizeof(double));
  for (uint32_t i = 0; i < slots; ++i) r[i] = creal(v[i]);
  free(v);
  return r;
}
/* the printers of ckks/src/cipher.c:228-338, in the reference's formats */
static void print_msg_range(FILE* fp, const DCMPLX* msg, uint32_t n) {
  double   lo_re = creal(msg[0]), hi_re = lo_re, lo_im = cimag(msg[0]), hi_im = lo_im;
  uint32_t lo_re_at = 0, hi_re_at = 0, lo_im_at = 0, hi_im_at = 0;
  for (uint32_t i = 1; i < n; ++i) {
    double re = creal(msg[i]), im = cimag(msg[i]);
    if (re > hi_re) hi_re = re, hi_re_at = i;
    else if (re < lo_re) lo_re = re, lo_re_at = i;
    if (im > hi_im) hi_im = im, hi_im_at = i;
    else if (im < lo_im) lo_im = im, lo_im_at = i;
  }
  fprintf(fp, "msg_range[%d]: real(%.17f[%d] ~ %.17f[%d]), imag(%.17f[%d] ~ %.17f[%d])\n", n, lo_re, lo_re_at, hi_re,
          hi_re_at, lo_im, lo_im_at, hi_im, hi_im_at);
}
static uint32_t slots_of(CIPHER c) { return c->_slots ? c->_slots : G.N / 2; }
void Print_cipher_info(FILE* fp, const char* name, CIPHER c) {
  fprintf(fp, "\n[%s] ciph_info: %d %d %ld %ld\n", name, c->_sf_degree, c->_slots, (long)c->_c0_poly._num_primes,
          (long)c->_c0_poly._num_primes_p);
}
static void print_msg(FILE* fp, const char* name, CIPHER c, uint32_t len, uint32_t b_len, bool imag) {
  DCMPLX*  m = Get_msg_with_imag(c);
  uint32_t n = slots_of(c);
  Print_cipher_info(fp, name, c);
  fprintf(fp, b_len ? "[%s] msg: [ \n" : "[%s] msg: [ ", name);
  for (uint32_t i = 0; i < len && i < n; ++i) {
    if (b_len && i % b_len == 0) fprintf(fp, "\n");
    if (imag) fprintf(fp, "(%.17f, %.17fI) ", creal(m[i]), cimag(m[i]));
    else fprintf(fp, "%.17f ", creal(m[i]));
  }
  fprintf(fp, "] ");
  print_msg_range(fp, m, n);
  free(m);
}
void Print_cipher_msg(FILE* fp, const char* name, CIPHER c, uint32_t len) { print_msg(fp, name, c, len, 0, false); }
void Print_cipher_msg_by_block_len(FILE* fp, const char* name, CIPHER c, uint32_t len, uint32_t b_len) {
  FMT_ASSERT(b_len, "block length must not be zero");
  print_msg(fp, name, c, len, b_len, false);
}
void Print_cipher_msg_with_imag(FILE* fp, const char* name, CIPHER c, uint32_t len) { print_msg(fp, name, c, len, 0, true); }
void Print_cipher_range(FILE* fp, const char* name, CIPHER c) {
  DCMPLX* m = Get_msg_with_imag(c);
  fprintf(fp, "[%s] ", name);
  print_msg_range(fp, m, slots_of(c));
  free(m);
}
void Print_cipher_poly(FILE* fp, const char* name, CIPHER c) {
  Print_cipher_info(fp, name, c);
  fprintf(fp, "@c0:\n");
  Print_poly_lite(fp, &c->_c0_poly);
  fprintf(fp, "@c1:\n");
  Print_poly_lite(fp, &c->_c1_poly);
}
void Dump_cipher_msg(const char* name, CIPHER c, uint32_t len) { Print_cipher_msg(stderr, name, c, len); }

/* Within_value_range (cipher.c:172-186, encoder.c:48-101): would `msg`, encoded at the ciphertext's scale and
 * level, stay below half the level's modulus?  The inverse embedding runs on the device. */
bool Within_value_range(CIPHER c, double* msg, uint32_t len) {
  uint32_t n = slots_of(c);
  FMT_ASSERT(len <= n, "length of msg should less than slots");
  CKKS_PARAMS* prm = Get_context_params();
  double*      in  = (double*)calloc(2 * (size_t)n, sizeof(double));
  double*      out = (double*)calloc(2 * (size_t)n, sizeof(double));
  for (uint32_t i = 0; i < len; ++i) in[2 * i] = msg[i];
  ACE_OK(ace_embedding_inv(RT_CTX, out, in, n));
  double biggest = 0; /* Transform_msg_within_range, encoder.c:217-231 */
  for (size_t i = 0; i < 2 * (size_t)n; ++i) {
    double up = fabs(out[i] * c->_scaling_factor);
    if (up > biggest) biggest = up;
  }
  free(in);
  free(out);
  int32_t bits  = (int32_t)(log2(fmax(biggest, __DBL_MIN__))) + 1;
  int32_t valid = (int32_t)prm->_first_mod_size + (int32_t)(Level(c) - 1) * (int32_t)prm->_scaling_mod_size;
  return bits < valid;
}

/* Real_relu (cipher.c:340-366): the exact ReLU through the secret key, for validating the approximated one */
CIPHER Real_relu(CIPHER c) {
  uint32_t n = slots_of(c);
  DCMPLX*  m = Get_msg_with_imag(c);
  for (uint32_t i = 0; i < n; ++i)
    if (creal(m[i]) <= 0) m[i] *= 0.0;
  PLAINTEXT pt;
  memset(&pt, 0, sizeof(pt));
  init_plain(&pt, Level(c), pow(G.sc, c->_sf_degree), c->_sf_degree, n);
  ACE_OK(ace_encode(RT_CTX, pt._poly._data, (const double*)m, n, n, Level(c), c->_sf_degree, 0));
  CIPHER res = (CIPHER)calloc(1, sizeof(CIPHERTEXT));
  Encrypt(res, &pt);
  Free_plain_poly(&pt);
  free(m);
  return res;
}
/* ---- tensors, program inputs and outputs (common/tensor.h, ckks/src/rtlib.c:66-229) ---------------- */
TENSOR* Alloc_tensor(size_t n, size_t c, size_t h, size_t w, const double* val) {
  size_t  len = n * c * h * w;
  TENSOR* t   = (TENSOR*)malloc(sizeof(TENSOR) + len * sizeof(double));
  t->_shape   = (SHAPE){n, c, h, w};
  if (val) memcpy(t->_vals, val, len * sizeof(double));
  else memset(t->_vals, 0, len * sizeof(double));
  return t;
}
void Free_tensor(TENSOR* t) { free(t); }
void Print_tensor(FILE* fp, TENSOR* t) {
  size_t len = TENSOR_SIZE(t);
  fprintf(fp, "[%zu %zu %zu %zu] {", TENSOR_N(t), TENSOR_C(t), TENSOR_H(t), TENSOR_W(t));
  for (size_t i = 0; i < len && i < 16; ++i) fprintf(fp, " %g", t->_vals[i]);
  fprintf(fp, len > 16 ? " ... }\n" : " }\n");
}

static DATA_SCHEME* find_scheme(const char* name, bool input) {
  int cnt = input ? (Get_input_count ? Get_input_count() : 0) : (Get_output_count ? Get_output_count() : 0);
  for (int i = 0; i < cnt; ++i) {
    DATA_SCHEME* s = input ? Get_encode_scheme(i) : Get_decode_scheme(i);
    FMT_ASSERT(s, "invalid encode scheme");
    if (strcmp(s->_name, name) == 0) return s;
  }
  Rt_fatal(__FILE__, __LINE__, "not find the %s \"%s\"", input ? "input" : "output", name);
}

static void prepare_input(TENSOR* input, const char* name, bool dup) {
  NEED_CTX();
  DATA_SCHEME* sch = find_scheme(name, true);
  FMT_ASSERT(sch->_count > 0, "no desc found in scheme");
  size_t total = TENSOR_SIZE(input), hw = TENSOR_H(input) * TENSOR_W(input);
  size_t level = G.input_level ? G.input_level : G.L;
  for (int i = 0; i < sch->_count; ++i) {
    const MAP_DESC* d = &sch->_desc[i];
    size_t          len;
    double*         v;
    if (d->_count == 0) { /* the whole tensor in one ciphertext */
      len = dup ? G.N / 2 : total;
      FMT_ASSERT(total <= len, "tensor larger than the slot count");
      v = (double*)calloc(2 * len, sizeof(double));
      for (size_t k = 0; k < total; ++k) v[2 * k] = input->_vals[k];
      if (dup) { /* Pre_encode_scheme_dup (rtlib.c:19-33): repeated with the period of the next power of two */
        size_t period = 1;
        while (period < total) period <<= 1;
        for (size_t k = period; k < len; ++k) v[2 * k] = v[2 * (k % period)];
      }
    } else { /* a chunk with optional padding from its neighbours (Pre_encode_scheme) */
      FMT_ASSERT(d->_kind == NORMAL && d->_stride == 1, "TODO: other kind / stride");
      FMT_ASSERT((size_t)d->_count < total && (size_t)(d->_start + d->_count) <= total, "chunk out of image bound");
      size_t loc = (size_t)d->_start, pad = (size_t)d->_pad;
      bool   begin = loc % hw == 0, end = (loc + (size_t)d->_count) % hw == 0;
      len = (size_t)d->_count + 2 * pad;
      v   = (double*)calloc(2 * len, sizeof(double));
      for (size_t k = 0; k < pad; ++k) v[2 * k] = begin ? 0 : input->_vals[loc - (pad - k)];
      for (size_t k = 0; k < (size_t)d->_count; ++k) v[2 * (k + pad)] = input->_vals[loc + k];
      for (size_t k = 0; k < pad; ++k) v[2 * (k + pad + (size_t)d->_count)] = end ? 0 : input->_vals[loc + (size_t)d->_count + k];
    }
    PLAINTEXT pt;
    memset(&pt, 0, sizeof(pt));
    encode_vector(&pt, v, len, 1, (uint32_t)level);
    IO_SLOT*    s  = Rt_add_slot(&LANE.in, &LANE.n_in, name, (size_t)i);
    CIPHERTEXT* ct = (CIPHERTEXT*)calloc(1, sizeof(CIPHERTEXT));
    Encrypt(ct, &pt);
    s->ct = ct;
    Free_plain_poly(&pt);
    free(v);
  }
}

void Prepare_input(TENSOR* input, const char* name) { prepare_input(input, name, false); }
void Prepare_input_dup(TENSOR* input, const char* name) { prepare_input(input, name, true); }

double* Handle_output(const char* name) {
  NEED_CTX();
  DATA_SCHEME* sch = find_scheme(name, false);
  FMT_ASSERT(sch->_count > 0, "no desc found in scheme");
  size_t len = sch->_shape._n * sch->_shape._c * sch->_shape._h * sch->_shape._w;
  if (len == 0) len = G.N / 2;
  double* ret = (double*)calloc(len, sizeof(double));
  for (int i = 0; i < sch->_count; ++i) {
    IO_SLOT* s = Rt_find_slot(LANE.out, LANE.n_out, name, (size_t)i);
    FMT_ASSERT(s && s->ct, "not find data");
    PLAINTEXT pt;
    memset(&pt, 0, sizeof(pt));
    Rt_decrypt(&pt, s->ct);
    uint32_t slots = pt._slots ? pt._slots : G.N / 2;
    DCMPLX*  vec   = (DCMPLX*)malloc(slots * sizeof(DCMPLX));
    Rt_decode(vec, &pt);
    const MAP_DESC* d = &sch->_desc[i];
    if (d->_count == 0) {
      for (size_t k = 0; k < len && k < slots; ++k) ret[k] = creal(vec[k]);
    } else {
      FMT_ASSERT(d->_kind == NORMAL && (size_t)d->_count <= len && (size_t)(d->_start + d->_count * d->_stride) <= len,
                 "chunk out of image bound");
      for (size_t k = 0, loc = (size_t)d->_start; k < (size_t)d->_count; ++k, loc += (size_t)d->_stride)
        ret[loc] = creal(vec[k]);
    }
    free(vec);
    Free_plain_poly(&pt);
  }
  return ret;
}
