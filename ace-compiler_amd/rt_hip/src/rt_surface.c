/* rt_surface.c -- the rest of the program-facing surface of the ANT runtime: entry points that the
 * compiler's emitters can produce but the committed programs rarely use.  Each is a thin composition of
 * the entry points in rt_hip.c / rt_ckks.c, with the reference's name, argument order and return
 * convention (cited per function; paths relative to fhe-cmplr/rtlib/ant).
 */
#include <complex.h>
#include <math.h>
#include <sys/random.h>

#include "rt_internal.h"

/* ---- VALUE_LIST (include/util/type.h:399-418, util/src/type.c:14-20) ---------------------------------- */
static size_t value_size(VALUE_TYPE t) {
  switch (t) {
    case DBL_TYPE: return sizeof(double);
    case DCMPLX_TYPE: return sizeof(DCMPLX);
    case UI32_TYPE:
    case I32_TYPE: return sizeof(int32_t);
    case I64_TYPE:
    case UI64_TYPE: return sizeof(int64_t);
    case I128_TYPE: return sizeof(__int128);
    case PTR_TYPE:
    case VL_PTR_TYPE: return sizeof(void*);
    default: Rt_fatal(__FILE__, __LINE__, "value lists of type 0x%x are not supported", (unsigned)t);
  }
}
VALUE_LIST* Alloc_value_list(VALUE_TYPE type, size_t len) {
  VALUE_LIST* l = (VALUE_LIST*)malloc(sizeof(VALUE_LIST));
  l->_type      = type;
  l->_length    = len;
  l->_vals._a   = len ? (char*)calloc(len, value_size(type)) : NULL;
  return l;
}
void Free_value_list(VALUE_LIST* l) {
  if (!l) return;
  if (l->_type == VL_PTR_TYPE)
    for (size_t i = 0; i < l->_length; ++i) Free_value_list(l->_vals._v[i]);
  free(l->_vals._a);
  free(l);
}

/* ---- polynomials -------------------------------------------------------------------------------------- */
POLY Init_poly_by_opnd(POLY res, POLY opnd1, POLY opnd2, bool is_ext) {
  POLY picked;
  if (opnd1 == NULL || Poly_level(opnd1) == 0) picked = opnd2;
  else if (opnd2 == NULL || Poly_level(opnd2) == 0) picked = opnd1;
  else picked = Poly_level(opnd1) <= Poly_level(opnd2) ? opnd1 : opnd2;
  if (picked == NULL) return res; /* both operands are zero ciphertexts */
  if (res->_data != NULL && Poly_level(res) >= Poly_level(picked)) {
    FMT_ASSERT(Get_rdgree(res) == Get_rdgree(picked), "unmatched size");
    Set_poly_level(res, Poly_level(picked));
    if (is_ext) FMT_ASSERT(Num_p(res) == Get_p_cnt(), "invalid p number");
  } else {
    if (res->_data != NULL) Free_poly_data(res);
    Alloc_poly_data(res, Get_rdgree(picked), Poly_level(picked), is_ext ? Get_p_cnt() : 0);
  }
  Set_is_ntt(res, true);
  return res;
}

void Set_coeff_at(POLY p, int64_t val, uint32_t idx) {
  FMT_ASSERT(p, "null poly");
  FMT_ASSERT(idx < Get_poly_alloc_len(p), "idx outof bound");
  ACE_OK(ace_upload(RT_CTX, p->_data + idx, &val, 1));
}

static int64_t* download_whole(POLY p) {
  size_t   n = Get_poly_len(p);
  int64_t* h = (int64_t*)malloc((n ? n : 1) * sizeof(int64_t));
  Rt_download_poly(h, p);
  return h;
}
void Print_poly_rawdata(FILE* fp, POLY p) { /* rns_poly.c:1262-1280 */
  int64_t* h = download_whole(p);
  fprintf(fp, "raw data: \n");
  for (size_t t = 0; t < Get_num_pq(p); ++t) {
    fprintf(fp, "%s%zu: ", t < Poly_level(p) ? "q" : "p", t < Poly_level(p) ? t : t - Poly_level(p));
    for (uint32_t i = 0; i < p->_ring_degree; ++i) fprintf(fp, "%ld ", (long)h[t * p->_ring_degree + i]);
    fprintf(fp, "\n");
  }
  free(h);
}
void Print_poly(FILE* fp, POLY p) { Print_poly_rawdata(fp, p); }
void Print_poly_lite(FILE* fp, POLY p) { /* the first coefficients of the first limbs */
  int64_t* h = download_whole(p);
  size_t   limbs = Get_num_pq(p) < 2 ? Get_num_pq(p) : 2, coefs = p->_ring_degree < 8 ? p->_ring_degree : 8;
  fprintf(fp, "level %zu, p %zu, %s:", Poly_level(p), Num_p(p), Is_ntt(p) ? "ntt" : "coeff");
  for (size_t t = 0; t < limbs; ++t) {
    fprintf(fp, " [");
    for (size_t i = 0; i < coefs; ++i) fprintf(fp, " %ld", (long)h[t * p->_ring_degree + i]);
    fprintf(fp, " ...]");
  }
  fprintf(fp, "\n");
  free(h);
}

/* Sample_uniform_poly / Sample_ternary_poly (rns_poly.c:1127-1185): the reference's generator cannot be
 * reproduced; values come from the device hash and the host generator that Rt_generate_keys uses */
static uint64_t Sample_stream = 0x5A17ull << 32;
void Sample_uniform_poly(POLY p) {
  NEED_CTX();
  FMT_ASSERT(Num_p(p) == 0 || Num_p(p) == G.K, "Sample_uniform_poly: a polynomial carries all P limbs or none");
  FMT_ASSERT(Num_p(p) == 0 || Num_alloc(p) == Poly_level(p) + G.K, "Sample_uniform_poly: allocate the polynomial at its level");
  const char* env  = getenv("RT_HIP_SEED");
  uint64_t    seed = env ? strtoull(env, NULL, 0) : 0;
  if (!seed) /* from the operating system, like the keys: a caller may use the polynomial as a mask */
    FMT_ASSERT(getrandom(&seed, sizeof(seed), 0) == (ssize_t)sizeof(seed), "Sample_uniform_poly: getrandom failed");
  ACE_OK(ace_sample_uniform(RT_CTX, p->_data, Poly_level(p), Num_p(p) != 0, seed, __atomic_add_fetch(&Sample_stream, 1, __ATOMIC_RELAXED)));
}
void Sample_ternary_poly(POLY p, size_t hamming_weight) {
  NEED_CTX();
  FMT_ASSERT(Num_p(p) == 0 || (Num_p(p) == G.K && Num_alloc(p) == Poly_level(p) + G.K),
             "Sample_ternary_poly: allocate an extended polynomial at its level");
  size_t   n = p->_ring_degree;
  int64_t* v = (int64_t*)calloc(n, sizeof(int64_t));
  Rt_sample_ternary(v, n, hamming_weight);
  ACE_OK(ace_expand_small(RT_CTX, p->_data, v, Poly_level(p), Num_p(p) != 0));
  free(v);
}

VALUE_LIST* Alloc_precomp(POLY input) {
  size_t      nd   = Num_decomp(input);
  VALUE_LIST* list = Alloc_value_list(PTR_TYPE, nd);
  POLY_ARR    arr  = Rt_alloc_precomp(input, NULL);
  for (size_t d = 0; d < nd; ++d) Set_ptr_value(list, d, (PTR)&arr[d]);
  return list;
}
void Free_precomp(VALUE_LIST* precompute) {
  if (!precompute) return;
  if (LIST_LEN(precompute)) Free_polys((POLY_ARR)PTR_VALUE_AT(precompute, 0)); /* the digits are one array over one slab */
  Free_value_list(precompute);
}

void Chk_level(POLY res, POLY p0, POLY p1) {
  if (Poly_level(res) != Poly_level(p0) || Num_p(res) != Num_p(p0)) printf("level not match\n");
  if (p1 && (Poly_level(res) != Poly_level(p1) || Num_p(res) != Num_p(p1))) printf("level not match\n");
}

void Conv_poly2ntt(POLY res, POLY poly) {
  FMT_ASSERT(!Is_ntt(poly), "already ntt form");
  FMT_ASSERT(Is_size_match(res, poly) && Num_p(res) >= Num_p(poly), "size not match");
  if (res != poly) {
    size_t n = poly->_ring_degree;
    Rt_dev_copy(res->_data, poly->_data, Poly_level(poly) * n);
    if (Num_p(poly)) Rt_dev_copy(res->_data + Rt_p_offset(res), poly->_data + Rt_p_offset(poly), Num_p(poly) * n);
    res->_is_ntt = false;
  }
  Conv_poly2ntt_inplace(res);
}

POLY Mul_poly_fast(POLY res, POLY poly1, POLY poly2, POLY poly2_prec) {
  FMT_ASSERT(poly2_prec && poly2_prec->_data, "invalid precomputed of poly2");
  FMT_ASSERT(Is_size_match(res, poly2_prec), "level not matched");
  return Mul_poly(res, poly1, poly2);
}

/* scalars over the limbs of a polynomial: Q limb t uses scalars[t], P limb t scalars[level + t] */
typedef int64_t* (*hw_scalar_fn)(int64_t*, int64_t*, int64_t, MODULUS*, uint32_t);
static POLY per_limb_scalars(hw_scalar_fn fn, POLY res, POLY poly, const int64_t* q_scalars, const int64_t* p_scalars,
                             int64_t one_for_all, size_t first, size_t last) {
  FMT_ASSERT(Is_size_match(res, poly), "size not match");
  size_t level = Poly_level(res), n = res->_ring_degree;
  FMT_ASSERT(level <= G.L, "primes not match");
  for (size_t t = first; t < level && t < last; ++t) {
    int64_t q = G.q[t]._val, s = q_scalars ? q_scalars[t] : one_for_all % q;
    if (s < 0) s += q;
    fn(Coeffs(res, t, (uint32_t)n), Coeffs(poly, t, (uint32_t)n), s, &G.q[t], (uint32_t)n);
  }
  if (Num_p(res) && last >= level) {
    FMT_ASSERT(Num_p(res) == Num_p(poly), "unmatched p primes cnt");
    for (size_t t = 0; t < Num_p(res); ++t) {
      int64_t q = G.p[t]._val, s = p_scalars ? p_scalars[t] : one_for_all % q;
      if (s < 0) s += q;
      fn(Get_p_coeffs(res) + t * n, Get_p_coeffs(poly) + t * n, s, &G.p[t], (uint32_t)n);
    }
  }
  Set_is_ntt(res, Is_ntt(poly));
  return res;
}
static const int64_t* list_words(VALUE_LIST* scalars, POLY res, bool with_p) {
  FMT_ASSERT(scalars && LIST_TYPE(scalars) == I64_TYPE, "invalid value type");
  FMT_ASSERT(LIST_LEN(scalars) >= Poly_level(res) + (with_p ? Num_p(res) : 0), "length of scalars not match");
  return Get_i64_values(scalars);
}
POLY Scalars_integer_add_poly(POLY res, POLY poly, VALUE_LIST* scalars) {
  const int64_t* w = list_words(scalars, res, true);
  return per_limb_scalars(Hw_modadd_scalar, res, poly, w, w + Poly_level(res), 0, 0, (size_t)-1);
}
POLY Scalars_integer_multiply_poly(POLY res, POLY poly, VALUE_LIST* scalars) {
  const int64_t* w = list_words(scalars, res, true);
  return per_limb_scalars(Hw_modmul_scalar, res, poly, w, w + Poly_level(res), 0, 0, (size_t)-1);
}
POLY Scalar_integer_multiply_poly(POLY res, POLY poly, int64_t scalar) {
  return per_limb_scalars(Hw_modmul_scalar, res, poly, NULL, NULL, scalar, 0, (size_t)-1);
}
POLY Scalars_integer_multiply_poly_qpart(POLY res, POLY poly, VALUE_LIST* scalars, size_t part_idx) {
  const int64_t* w  = list_words(scalars, res, false);
  size_t         ps = ace_part_size(RT_CTX), first = ps * part_idx, last = first + ps;
  if (last > Poly_level(res)) last = Poly_level(res);
  return per_limb_scalars(Hw_modmul_scalar, res, poly, w, NULL, 0, first, last); /* the other limbs stay as they are */
}

POLY Automorphism_transform(POLY res, POLY poly, VALUE_LIST* precomp) {
  uint32_t n = Get_rdgree(poly);
  FMT_ASSERT(Is_size_match(res, poly), "op not matched");
  FMT_ASSERT(precomp && LIST_LEN(precomp) == n, "invalid index table length");
  FMT_ASSERT(res->_data != poly->_data, "Automorphism_transform: res must not be the operand");
  int64_t* order = Rt_dev_alloc_raw(n);
  ACE_OK(ace_upload(RT_CTX, order, Get_i64_values(precomp), n));
  for (size_t t = 0; t < Poly_level(res); ++t) Hw_rotate(Coeffs(res, t, n), Coeffs(poly, t, n), order, &G.q[t], n);
  for (size_t t = 0; t < Num_p(res); ++t)
    Hw_rotate(Get_p_coeffs(res) + t * (size_t)n, Get_p_coeffs(poly) + t * (size_t)n, order, &G.p[t], n);
  Rt_dev_free(order);
  Set_is_ntt(res, Is_ntt(poly));
  return res;
}

/* ---- limb views and one-limb arithmetic (rns_poly.c:1289-1317, lpoly/src/poly.c) ------------------------ */
static L_POLY limb_view(POLY p, size_t idx) {
  L_POLY l;
  Init_lpoly_data(&l, Get_rdgree(p), Coeffs(p, idx, Get_rdgree(p)));
  Set_lpoly_ntt(&l, Is_ntt(p));
  return l;
}
L_POLY Lpoly_from_poly(POLY poly, size_t idx) {
  FMT_ASSERT(idx < Get_num_pq(poly), "idx overflow");
  return limb_view(poly, idx);
}
L_POLY Lpoly_from_poly_arr(size_t size, POLY_ARR poly_arr, size_t idx) {
  size_t num_pq = Get_q_cnt() + Get_p_cnt();
  FMT_ASSERT(idx < size * num_pq, "idx overflow");
  return limb_view(&poly_arr[idx / num_pq], idx % num_pq);
}
void Set_poly_data(POLY poly, L_POLY lpoly, size_t idx) {
  FMT_ASSERT(idx < Get_num_pq(poly), "Set_poly_data_from_lpoly: idx overflow");
  Set_coeffs(poly, (uint32_t)idx, Get_rdgree(poly), Get_lpoly_coeffs(&lpoly));
}
void Zero_lpoly(LPOLY p) { ACE_OK(ace_zero(RT_CTX, p->_data, p->_ring_degree)); }
void Copy_lpoly(LPOLY res, L_POLY poly) {
  Rt_dev_copy(res->_data, poly._data, res->_ring_degree);
  res->_is_ntt = poly._is_ntt;
}
void Print_lpoly(FILE* fp, LPOLY p) {
  FMT_ASSERT(p, "null lpoly");
  int64_t* h = (int64_t*)malloc(p->_ring_degree * sizeof(int64_t));
  ACE_OK(ace_download(RT_CTX, h, p->_data, p->_ring_degree));
  fprintf(fp, "is_ntt: %s, raw data: \n", p->_is_ntt ? "Y" : "N");
  for (uint32_t j = 0; j < p->_ring_degree; ++j) fprintf(fp, "%ld ", (long)h[j]);
  fprintf(fp, "\n");
  free(h);
}
#define LPOLY2(NAME, HW)                                                       \
  LPOLY NAME(LPOLY res, L_POLY poly1, L_POLY poly2, MODULUS* mod) {            \
    FMT_ASSERT(poly1._is_ntt == poly2._is_ntt, "ntt not match");               \
    HW(res->_data, poly1._data, poly2._data, mod, res->_ring_degree);          \
    res->_is_ntt = poly1._is_ntt;                                              \
    return res;                                                                \
  }
#define LPOLY1(NAME, HW)                                                       \
  LPOLY NAME(LPOLY res, L_POLY poly, int64_t scalar, MODULUS* mod) {           \
    HW(res->_data, poly._data, scalar, mod, res->_ring_degree);                \
    res->_is_ntt = poly._is_ntt;                                               \
    return res;                                                                \
  }
LPOLY2(Add_lpoly, Hw_modadd)
LPOLY2(Sub_lpoly, Hw_modsub)
LPOLY2(Mul_lpoly, Hw_modmul)
LPOLY2(Mac_lpoly, Hw_modmuladd)
LPOLY1(Add_scalar, Hw_modadd_scalar)
LPOLY1(Sub_scalar, Hw_modsub_scalar)
LPOLY1(Mul_scalar, Hw_modmul_scalar)
LPOLY1(Mac_scalar, Hw_modmuladd_scalar)
void Ntt(LPOLY res, L_POLY poly, size_t idx) {
  FMT_ASSERT(!poly._is_ntt, "already ntt form");
  Hw_ntt(res->_data, poly._data, idx, res->_ring_degree);
  res->_is_ntt = true;
}
void Intt(LPOLY res, L_POLY poly, size_t idx) {
  FMT_ASSERT(poly._is_ntt, "already coeffcient form");
  Hw_intt(res->_data, poly._data, idx, res->_ring_degree);
  res->_is_ntt = false;
}

/* ---- ciphertexts (ckks/src/cipher.c) -------------------------------------------------------------------- */
static POLY ciph_limb(POLY c0, POLY c1, POLY c2, size_t idx, size_t* limb) {
  size_t num_pq = Get_num_pq(c0);
  FMT_ASSERT(idx < (c2 ? 3 : 2) * num_pq, "invalid idx");
  *limb = idx % num_pq;
  return idx < num_pq ? c0 : idx < 2 * num_pq ? c1 : c2;
}
L_POLY Lpoly_from_ciph(CIPHER c, size_t idx) {
  size_t limb;
  POLY   p = ciph_limb(&c->_c0_poly, &c->_c1_poly, NULL, idx, &limb);
  return limb_view(p, limb);
}
L_POLY Lpoly_from_ciph3(CIPHER3 c, size_t idx) {
  size_t limb;
  POLY   p = ciph_limb(&c->_c0_poly, &c->_c1_poly, &c->_c2_poly, idx, &limb);
  return limb_view(p, limb);
}
void Set_ciph_data(CIPHER c, L_POLY poly, size_t idx) {
  size_t limb;
  POLY   p = ciph_limb(&c->_c0_poly, &c->_c1_poly, NULL, idx, &limb);
  FMT_ASSERT(p->_data, "invalid coeffs");
  Set_coeffs(p, (uint32_t)limb, Degree(), poly._data);
  Set_is_ntt(p, poly._is_ntt);
}
void Set_ciph3_data(CIPHER3 c, L_POLY poly, size_t idx) {
  size_t limb;
  POLY   p = ciph_limb(&c->_c0_poly, &c->_c1_poly, &c->_c2_poly, idx, &limb);
  FMT_ASSERT(p->_data, "invalid coeffs");
  Set_coeffs(p, (uint32_t)limb, Degree(), poly._data);
  Set_is_ntt(p, poly._is_ntt);
}

/* cipher.c:856-890: the per-limb code generator writes the limbs of a result of `level` primes back to back
 * through c0 and on into c1, whatever level the ciphertext was allocated at; the first 2 * level limbs of
 * that sequence become c0 and c1 at `level`, and the rest of the way down is modulus switching */
void Reset_ciph(CIPHER c, size_t level) {
  POLY c0 = &c->_c0_poly, c1 = &c->_c1_poly;
  FMT_ASSERT(Num_p(c0) == 0, "unsupport ciph with expanded");
  size_t q_cnt = Poly_level(c0), n = c0->_ring_degree;
  FMT_ASSERT(level <= q_cnt, "level overflow");
  if (level == q_cnt) return;
  size_t   cur = Get_num_pq(c0);
  int64_t *d0 = Rt_dev_alloc_raw(level * n), *d1 = Rt_dev_alloc_raw(level * n);
  bool     is_ntt = Is_ntt(c0);
  Rt_dev_copy(d0, c0->_data, level * n);
  if (2 * level <= cur) {
    Rt_dev_copy(d1, c0->_data + level * n, level * n);
  } else {
    Rt_dev_copy(d1, c0->_data + level * n, (cur - level) * n);
    Rt_dev_copy(d1 + (cur - level) * n, c1->_data, (2 * level - cur) * n);
  }
  Free_poly_data(c0);
  Free_poly_data(c1);
  Init_poly_data(c0, (uint32_t)n, level, 0, d0);
  Init_poly_data(c1, (uint32_t)n, level, 0, d1);
  Set_is_ntt(c0, is_ntt);
  Set_is_ntt(c1, is_ntt);
  for (size_t i = Poly_level(c0); i > level; --i) Modswitch_ciph(c);
}

void Free_cipher(CIPHER c) {
  if (!c) return;
  Free_ciph_poly(c, 1);
  free(c);
}
void Init_ciph3_same_scale(CIPHER3 res, CIPHER3 a, CIPHER3 b) { Init_ciph3_same_scale_ciph3(res, a, b); }
void Init_ciph3_down_scale(CIPHER3 res, CIPHER3 c) {
  FMT_ASSERT(c->_sf_degree >= 2, "Scale degree of result dec to zero");
  Init_poly(&res->_c0_poly, &c->_c0_poly);
  Init_poly(&res->_c1_poly, &c->_c1_poly);
  Init_poly(&res->_c2_poly, &c->_c2_poly);
  res->_scaling_factor = c->_scaling_factor / Get_default_sc();
  res->_sf_degree      = c->_sf_degree - 1;
  res->_slots          = c->_slots;
}
void Init_ciph_up_scale_scalars(CIPHER res, CIPHER c, size_t len) { /* cipher.c:85-92 */
  size_t level = Level(c);
  Rt_shape_ciph(res, c, c->_scaling_factor * Get_default_sc(), c->_sf_degree + 1);
  if (level > len) {
    Set_poly_level(&res->_c0_poly, len);
    Set_poly_level(&res->_c1_poly, len);
  }
}

void Modswitch_ciph(CIPHER c) {
  size_t level = Level(c);
  FMT_ASSERT(level > 1 && (uint32_t)log2(c->_scaling_factor) <= (level - 1) * (uint32_t)log2(G.sc),
             "Modswitch: invalid scaling factor of ciph");
  Modswitch(&c->_c0_poly, &c->_c0_poly);
  Modswitch(&c->_c1_poly, &c->_c1_poly);
}

/* Mul_scalars (evaluator.c:218-235) with the residues of Encode_val(1.0, scale = 2^mod_size) */
CIPHER Upscale_ciph(CIPHER res, CIPHER c, uint32_t mod_size) {
  CKKS_PARAMS* prm   = Get_context_params();
  size_t       level = Level(c);
  double       up = pow(2.0, mod_size), sf = c->_scaling_factor * up;
  FMT_ASSERT((uint32_t)log2(sf) < prm->_first_mod_size + (level - 1) * prm->_scaling_mod_size, "Upscale: mod_size is two high");
  int64_t words[128];
  Rt_encode_val_words(words, 1.0, (uint32_t)level, up);
  VALUE_LIST box = {I64_TYPE, level, {._i = words}};
  Rt_shape_ciph(res, c, sf, c->_sf_degree + 1);
  Scalars_integer_multiply_poly(&res->_c0_poly, &c->_c0_poly, &box);
  Scalars_integer_multiply_poly(&res->_c1_poly, &c->_c1_poly, &box);
  return res;
}
CIPHER Downscale_ciph(CIPHER res, CIPHER c, uint32_t waterline) {
  FMT_ASSERT(Level(c) > 1, "Downscale: multiply level is not big enought for more operation, try to use larger depth");
  uint32_t sf_bits = (uint32_t)log2(G.sc), have = (uint32_t)log2(c->_scaling_factor);
  FMT_ASSERT(waterline <= sf_bits, "Downscale: waterline should not larger than scaling factor");
  FMT_ASSERT(have > sf_bits && have < waterline + sf_bits,
             "Downscale: waterline is set too low or the scale of input ciph is too high");
  Upscale_ciph(c, c, waterline + sf_bits - have); /* the operand itself is scaled up, as in the reference */
  c->_sf_degree += 1;
  return Rescale_ciph(res, c);
}
CIPHER Raise_mod(CIPHER res, CIPHER c, uint32_t mod_size) {
  uint32_t   raise = mod_size ? mod_size : (uint32_t)Get_q_cnt();
  FMT_ASSERT(raise <= Get_q_cnt(), "Raise_mod: more primes than the context has");
  CIPHERTEXT low;
  memset(&low, 0, sizeof(low));
  Copy_ciph(&low, c);
  while (low._sf_degree > 1) Rescale_ciph(&low, &low);
  if (Is_ntt(&low._c0_poly)) Conv_ntt2poly_inplace(&low._c0_poly);
  if (Is_ntt(&low._c1_poly)) Conv_ntt2poly_inplace(&low._c1_poly);
  uint32_t slots = c->_slots;
  if (res->_c0_poly._data) Free_ciph_poly(res, 1);
  memset(res, 0, sizeof(*res));
  Alloc_poly_data(&res->_c0_poly, G.N, raise, 0);
  Alloc_poly_data(&res->_c1_poly, G.N, raise, 0);
  res->_scaling_factor = low._scaling_factor;
  res->_sf_degree      = low._sf_degree;
  res->_slots          = slots;
  Transform_values_from_level0(&res->_c0_poly, &low._c0_poly);
  Transform_values_from_level0(&res->_c1_poly, &low._c1_poly);
  Free_ciph_poly(&low, 1);
  Conv_poly2ntt_inplace(&res->_c0_poly);
  Conv_poly2ntt_inplace(&res->_c1_poly);
  return res;
}

/* ---- plaintexts (ckks/src/plain.c) ---------------------------------------------------------------------- */
void Copy_plain(PLAIN res, PLAIN plain) {
  POLY src = &plain->_poly, dst = &res->_poly;
  if (dst->_data && (dst->_ring_degree != src->_ring_degree || dst->_num_primes != src->_num_primes ||
                     dst->_num_primes_p != src->_num_primes_p || dst->_num_alloc_primes != Get_num_pq(src)))
    Free_poly_data(dst);
  if (!dst->_data) Alloc_poly_data(dst, src->_ring_degree, src->_num_primes, src->_num_primes_p);
  res->_slots          = plain->_slots;
  res->_scaling_factor = plain->_scaling_factor;
  res->_sf_degree      = plain->_sf_degree;
  Copy_poly(dst, src);
}
L_POLY Lpoly_from_plain(PLAIN plain, size_t idx) {
  FMT_ASSERT(idx < Get_num_pq(&plain->_poly), "invalid idx");
  return limb_view(&plain->_poly, idx);
}
struct PLAINTEXT_BUFFER* Encode_dcmplx_ext_buffer(const void* input, size_t len, uint32_t level, uint32_t p_cnt) {
  NEED_CTX();
  FMT_ASSERT(p_cnt == 0 || p_cnt <= Get_p_cnt(), "Encode_dcmplx_ext_buffer p_cnt exceeds active encode-context p count");
  PLAINTEXT pt;
  memset(&pt, 0, sizeof(pt));
  Encode_dcmplx_ext(&pt, (DCMPLX*)input, len, level, p_cnt);
  size_t words  = Get_poly_len(&pt._poly);
  size_t pt_len = sizeof(PLAINTEXT) + words * sizeof(int64_t);
  struct PLAINTEXT_BUFFER* buf = (struct PLAINTEXT_BUFFER*)calloc(1, sizeof(struct PLAINTEXT_BUFFER) + pt_len);
  FMT_ASSERT(buf, "Failed to malloc sizeofPLAINTEXT_BUFFER");
  memcpy(buf->_magic, "ANTPLAIN", 8);
  buf->_version = RT_DATA_VERSION;
  buf->_size    = (uint32_t)pt_len;
  PLAINTEXT image = pt;
  image._poly._data = NULL; /* the reader points it at the words that follow */
  memcpy(buf->_data, &image, sizeof(PLAINTEXT));
  Rt_download_poly((int64_t*)(buf->_data + sizeof(PLAINTEXT)), &pt._poly);
  Free_plain_poly(&pt);
  return buf;
}

/* ---- tensors (common/src/tensor.c) ------------------------------------------------------------------------ */
bool Is_tensor_match(TENSOR* t1, TENSOR* t2) {
  return TENSOR_N(t1) == TENSOR_N(t2) && TENSOR_C(t1) == TENSOR_C(t2) && TENSOR_H(t1) == TENSOR_H(t2) &&
         TENSOR_W(t1) == TENSOR_W(t2);
}
TENSOR* Add_tensor(TENSOR* t1, TENSOR* t2) {
  FMT_ASSERT(Is_tensor_match(t1, t2), "tensor shape not match");
  TENSOR* r = Alloc_tensor(TENSOR_N(t1), TENSOR_C(t1), TENSOR_H(t1), TENSOR_W(t1), NULL);
  size_t  n = TENSOR_SIZE(t1);
  for (size_t i = 0; i < n; ++i) r->_vals[i] = t1->_vals[i] + t2->_vals[i];
  return r;
}
