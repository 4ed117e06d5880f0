/* A plain-float stand-in for the runtime, for tests only: what a compiled program computes when every ciphertext
 * is its message.  A "polynomial" is one limb of Degree() = N/2 doubles, the slots of the message; a ciphertext is
 * (message, 0); rotation keys and the relinearisation key are absent (Num_decomp = 0), so the key switches the
 * compiler writes out limb by limb add nothing, and what remains of a rotation is Hw_rotate with the table of
 * Auto_order, of a product the slot-wise product, of Rescale and Bootstrap a copy.  A generated program
 * (rtlib/ant/dataset/*.inc) is included unchanged over this header in place of rt_ant/rt_ant.h and run on the
 * host; its output is what the same program must decrypt to on the GPU, up to the scheme's noise and the
 * bootstraps' error.  Semantics restated from the reference's program-facing API: include/poly/rns_poly.h:140-468,
 * include/hal/hal.h:24-111 (Hw_* element-wise on one limb), ckks/include/cipher.h, ckks/src/plain.c:29-63 (an encoded
 * vector fills the first `len` slots, the others are zero; a single value fills every slot), porting/pt_mgr.c:188-243
 * (Pt_from_msg: `len` values of entry `index`); an input tensor under the NORMAL data scheme is its values in order
 * (the harness fills it in).  Weight entries are the reproducible pseudo-random values the runtime substitutes for a
 * missing weight file (RT_HIP_SYNTHETIC_WEIGHTS=<amplitude>), restated below. */
#ifndef SHADOW_RT_ANT_H
#define SHADOW_RT_ANT_H
#include <math.h>
#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

typedef enum { LIB_ANT = 0 } LIB_PROV;
typedef enum { DE_MSG_F32 = 0, DE_MSG_F64 = 1, DE_PLAINTEXT = 2 } DATA_ENTRY_TYPE;
typedef enum { NORMAL = 0 } MAP_KIND;
typedef struct { MAP_KIND _kind; int _a, _b, _c, _d; } MAP_DESC;
typedef struct { const char* _name; size_t _shape[4]; int _count; MAP_DESC* _desc; } DATA_SCHEME;
typedef struct {
  LIB_PROV _provider;
  uint32_t _poly_degree;
  size_t   _sec_level, _mul_depth, _input_level, _first_mod_size, _scaling_mod_size, _num_q_parts, _hamming_weight;
  size_t   _num_rot_idx;
  int32_t  _rot_idxs[];
} CKKS_PARAMS;
typedef struct { const char* _file_name; const char* _file_uuid; DATA_ENTRY_TYPE _entry_type; } RT_DATA_INFO;
typedef struct { int64_t _val; } MODULUS;
typedef struct { int _unused; } SWITCH_KEY;

typedef struct {
  uint32_t _ring_degree;
  size_t   _num_primes;
  int64_t* _data; /* Degree() doubles, kept behind the pointer type the generated code expects */
} POLYNOMIAL;
typedef POLYNOMIAL* POLY;
typedef struct { POLYNOMIAL _poly; uint32_t _level, _sc_degree; } PLAINTEXT;
typedef PLAINTEXT* PLAIN;
typedef struct { POLYNOMIAL _c0_poly, _c1_poly; uint32_t _level, _sc_degree; } CIPHERTEXT;
typedef CIPHERTEXT* CIPHER;
typedef struct { POLYNOMIAL _c0_poly, _c1_poly, _c2_poly; uint32_t _level, _sc_degree; } CIPHERTEXT3;
typedef CIPHERTEXT3* CIPHER3;

CKKS_PARAMS*  Get_context_params(void);
RT_DATA_INFO* Get_rt_data_info(void);
bool          Main_graph(void);

extern uint32_t Shadow_slots;     /* N / 2 */
extern uint32_t Shadow_top_level; /* mul_depth + 1 */
extern double   Shadow_amplitude;
extern MODULUS  Shadow_moduli[128];
static inline uint32_t Degree(void) { return Shadow_slots; }
static inline double*  Sh(int64_t* p) { return (double*)(void*)p; }

/* ---- polynomials ---- */
static inline void Alloc_poly_data(POLY p, uint32_t degree, size_t level, size_t extra) {
  (void)level, (void)extra;
  p->_ring_degree = degree;
  p->_num_primes  = 1;
  p->_data        = (int64_t*)calloc(degree, sizeof(double));
}
static inline POLY Alloc_poly(uint32_t degree, size_t level, size_t extra) {
  POLY p = (POLY)calloc(1, sizeof(POLYNOMIAL));
  Alloc_poly_data(p, degree, level, extra);
  return p;
}
static inline void Free_poly_data(POLY p) {
  free(p->_data);
  p->_data       = NULL;
  p->_num_primes = 0;
}
static inline void Free_poly(POLY p) {
  Free_poly_data(p);
  free(p);
}
static inline size_t   Poly_level(POLY p) { return p->_data ? 1 : 0; }
static inline size_t   Num_p(POLY p) { (void)p; return 0; }
static inline size_t   Num_alloc(POLY p) { (void)p; return 1; }
static inline size_t   Num_decomp(POLY p) { (void)p; return 0; } /* no digits: key switches add nothing */
static inline int64_t* Coeffs(POLY p, size_t limb, uint32_t degree) { return p->_data + limb * (size_t)degree; }
static inline void     Set_coeffs(POLY dst, uint32_t limb, uint32_t degree, int64_t* src) {
  if (dst->_data + (size_t)limb * degree != src) memcpy(dst->_data + (size_t)limb * degree, src, degree * sizeof(double));
}
static inline MODULUS*    Q_modulus(void) { return Shadow_moduli; }
static inline MODULUS*    P_modulus(void) { return Shadow_moduli; }
static inline SWITCH_KEY* Swk(bool is_rot, int32_t rot_idx) { (void)is_rot, (void)rot_idx; return NULL; }
static inline POLY        Pk0_at(SWITCH_KEY* k, uint32_t part) { (void)k, (void)part; return NULL; }
static inline POLY        Pk1_at(SWITCH_KEY* k, uint32_t part) { (void)k, (void)part; return NULL; }
static inline void Decomp_modup(POLY res, POLY a, uint32_t part) { (void)res, (void)a, (void)part; }
static inline void Copy_limb(POLY res, POLY a) {
  if (!res->_data) Alloc_poly_data(res, a->_ring_degree, 1, 0);
  memcpy(res->_data, a->_data, a->_ring_degree * sizeof(double));
}
static inline POLY Mod_down(POLY res, POLY a) { Copy_limb(res, a); return res; }
static inline POLY Rescale(POLY res, POLY a) { Copy_limb(res, a); return res; }
int64_t* Auto_order(int32_t rot_idx);

/* ---- Hw_* on one limb: slot-wise ---- */
static inline void Hw_modadd(int64_t* r, int64_t* a, int64_t* b, MODULUS* m, uint32_t n) {
  (void)m;
  for (uint32_t i = 0; i < n; ++i) Sh(r)[i] = Sh(a)[i] + Sh(b)[i];
}
static inline void Hw_modmul(int64_t* r, int64_t* a, int64_t* b, MODULUS* m, uint32_t n) {
  (void)m;
  for (uint32_t i = 0; i < n; ++i) Sh(r)[i] = Sh(a)[i] * Sh(b)[i];
}
static inline void Hw_rotate(int64_t* r, int64_t* a, int64_t* order, MODULUS* m, uint32_t n) {
  (void)m;
  for (uint32_t i = 0; i < n; ++i) Sh(r)[i] = Sh(a)[order[i]];
}

/* ---- ciphertexts ---- */
static inline uint32_t Level(CIPHER c) { return c->_level; }
static inline uint32_t Sc_degree(CIPHER c) { return c->_sc_degree; }
static inline void Shape(POLY p) {
  if (!p->_data) Alloc_poly_data(p, Degree(), 1, 0);
}
static inline void Init_ciph_same_scale(CIPHER res, CIPHER a, CIPHER b) {
  CIPHER from = (a && a->_c0_poly._data) ? a : ((b && b->_c0_poly._data) ? b : a);
  uint32_t lv = from->_level, sd = from->_sc_degree;
  if (a && b && a->_c0_poly._data && b->_c0_poly._data && b->_level < lv) lv = b->_level;
  Shape(&res->_c0_poly), Shape(&res->_c1_poly);
  res->_level = lv, res->_sc_degree = sd;
}
static inline void Init_ciph_same_scale_plain(CIPHER res, CIPHER c, PLAIN p) {
  (void)p;
  uint32_t lv = c->_level, sd = c->_sc_degree;
  Shape(&res->_c0_poly), Shape(&res->_c1_poly);
  res->_level = lv, res->_sc_degree = sd;
}
static inline void Init_ciph_up_scale_plain(CIPHER res, CIPHER c, PLAIN p) {
  uint32_t lv = c->_level, sd = c->_sc_degree + p->_sc_degree;
  Shape(&res->_c0_poly), Shape(&res->_c1_poly);
  res->_level = lv, res->_sc_degree = sd;
}
static inline void Init_ciph_down_scale(CIPHER res, CIPHER c) {
  uint32_t lv = c->_level - 1, sd = c->_sc_degree - 1;
  Shape(&res->_c0_poly), Shape(&res->_c1_poly);
  res->_level = lv, res->_sc_degree = sd;
}
static inline void Init_ciph3_up_scale(CIPHER3 res, CIPHER a, CIPHER b) {
  uint32_t lv = a->_level < b->_level ? a->_level : b->_level, sd = a->_sc_degree + b->_sc_degree;
  Shape(&res->_c0_poly), Shape(&res->_c1_poly), Shape(&res->_c2_poly);
  res->_level = lv, res->_sc_degree = sd;
}
static inline void Init_ciph_same_scale_ciph3(CIPHER res, CIPHER3 c) {
  Shape(&res->_c0_poly), Shape(&res->_c1_poly);
  res->_level = c->_level, res->_sc_degree = c->_sc_degree;
}
static inline void Copy_ciph(CIPHER res, CIPHER c) {
  if (res == c) return;
  Copy_limb(&res->_c0_poly, &c->_c0_poly);
  Copy_limb(&res->_c1_poly, &c->_c1_poly);
  res->_level = c->_level, res->_sc_degree = c->_sc_degree;
}
static inline void Free_ciph_poly(CIPHER arr, uint32_t cnt) {
  for (uint32_t i = 0; i < cnt; ++i) Free_poly_data(&arr[i]._c0_poly), Free_poly_data(&arr[i]._c1_poly);
}
static inline CIPHER Bootstrap(CIPHER res, CIPHER c, uint32_t level_after) {
  Copy_ciph(res, c);
  res->_level     = level_after ? level_after : Shadow_top_level;
  res->_sc_degree = 1;
  return res;
}

/* ---- plaintexts ---- */
void Encode_double(PLAIN plain, double* input, size_t len, uint32_t sc_degree, uint32_t level);
void Encode_float(PLAIN plain, float* input, size_t len, uint32_t sc_degree, uint32_t level);
void* Pt_from_msg(void* pt, uint32_t index, size_t len, uint32_t scale, uint32_t level);

/* ---- named ciphertexts, timing marks ---- */
CIPHERTEXT Get_input_data(const char* name, size_t idx);
void       Set_output_data(const char* name, size_t idx, CIPHER data);
static inline void Tm_start(const char* msg) { (void)msg; }
static inline void Tm_taken(const char* msg) { (void)msg; }
#endif
