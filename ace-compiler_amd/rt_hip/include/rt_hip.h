/* rt_hip.h -- host-side C runtime with the ANT runtime's program-facing API,
 * whose polynomial data lives in HBM and whose arithmetic runs as HIP kernels
 * behind the C-ABI of ace_hip.h.
 *
 * A program written against the reference's `rt_ant/rt_ant.h` (the C emitted by
 * the FHE compiler: Main_graph, Rotate, Relinearize bodies) compiles against this
 * header instead: the struct layouts, function names, argument order and return
 * conventions are those of the reference (fhe-cmplr/rtlib/ant/include, cited per
 * declaration), the bodies are new.  What differs, by design:
 *
 *   - POLYNOMIAL._data is a DEVICE pointer.  Host code may do pointer arithmetic
 *     on it (Coeffs) and pass it back to the runtime; it must not dereference it.
 *   - Auto_order() returns a device table, consumed by Hw_rotate only.
 *   - The header inlines that malloc/memset/memcpy `_data` in the reference
 *     (Alloc_poly_data, Set_coeffs, Free_poly_data) call the device allocator.
 *   - Keys and inputs are supplied by the harness (Rt_load_switch_key,
 *     Rt_set_input): the reference's samplers are not reproducibly seedable, so
 *     bit-exact runs need the caller's own data.  Encode / encrypt / decrypt are
 *     not part of this layer.
 *
 * Errors follow the reference (include/common/error.h:17-32): print and abort.
 * One host thread; all work is enqueued on one HIP stream and is asynchronous
 * until Rt_get_output / Rt_download_poly.
 */
#ifndef RT_HIP_H
#define RT_HIP_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef TRUE
#define TRUE 1
#endif
#ifndef FALSE
#define FALSE 0
#endif

/* ---- program-provided hooks (include/common/common.h:40-92, rt_api.h:48-80) ---- */
typedef enum { LIB_ANT, LIB_SEAL, LIB_OPENFHE, LIB_PHANTOM, LIB_ACE } LIB_PROV;
typedef enum { NORMAL, CONV, CHANNEL, DIAGONAL } MAP_KIND;
typedef enum { DE_MSG_F32, DE_MSG_F64, DE_PLAINTEXT } DATA_ENTRY_TYPE;
typedef struct {
  MAP_KIND _kind;
  int      _count, _start, _pad, _stride;
} MAP_DESC;
typedef struct {
  size_t _n, _c, _h, _w;
} SHAPE;
typedef struct {
  const char* _name;
  SHAPE       _shape;
  int         _count;
  MAP_DESC*   _desc;
} DATA_SCHEME;
typedef struct {
  LIB_PROV _provider;
  uint32_t _poly_degree;
  size_t   _sec_level;
  size_t   _mul_depth;        /* number of Q primes = _mul_depth + 1 */
  size_t   _input_level;
  size_t   _first_mod_size;   /* bits of q_0 */
  size_t   _scaling_mod_size; /* bits of the other Q primes */
  size_t   _num_q_parts;      /* 0: by depth (1, 2 up to depth 3, else 3) */
  size_t   _hamming_weight;
  size_t   _num_rot_idx;
  int32_t  _rot_idxs[];
} CKKS_PARAMS;
typedef struct {
  const char*     _file_name;
  const char*     _file_uuid;
  DATA_ENTRY_TYPE _entry_type;
} RT_DATA_INFO;

CKKS_PARAMS*  Get_context_params(void) __attribute__((weak));
RT_DATA_INFO* Get_rt_data_info(void) __attribute__((weak));
int           Get_input_count(void) __attribute__((weak));
int           Get_output_count(void) __attribute__((weak));
DATA_SCHEME*  Get_encode_scheme(int idx) __attribute__((weak));
DATA_SCHEME*  Get_decode_scheme(int idx) __attribute__((weak));
bool          Main_graph(void) __attribute__((weak));

/* ---- MODULUS (include/util/modular.h:21-26): 48 bytes, arrays are contiguous ---- */
typedef struct {
  int64_t           _val;
  int64_t           _br_k;
  int64_t           _br_m;
  unsigned __int128 _prec128;
} MODULUS;

/* ---- POLYNOMIAL (include/poly/rns_poly.h:23-32) ---- */
typedef struct {
  uint32_t _ring_degree;
  size_t   _num_alloc_primes;
  size_t   _num_primes;
  size_t   _num_primes_p;
  bool     _is_ntt;
  int64_t* _data; /* device memory: limb-major, P limbs at (_num_alloc_primes - _num_primes_p) */
} POLYNOMIAL;
typedef POLYNOMIAL* POLY;
typedef POLYNOMIAL* POLY_ARR;

/* ---- ciphertexts (include/ckks/ciphertext.h:29-35, 260-267) ---- */
typedef struct {
  POLYNOMIAL _c0_poly, _c1_poly;
  uint32_t   _slots;
  double     _scaling_factor;
  uint32_t   _sf_degree;
} CIPHERTEXT;
typedef struct {
  POLYNOMIAL _c0_poly, _c1_poly, _c2_poly;
  uint32_t   _slots;
  double     _scaling_factor;
  uint32_t   _sf_degree;
} CIPHERTEXT3;
typedef CIPHERTEXT*  CIPHER;
typedef CIPHERTEXT3* CIPHER3;

/* ---- plaintext (include/ckks/plaintext.h:23-28) ---- */
typedef struct {
  POLYNOMIAL _poly;
  uint32_t   _slots;
  double     _scaling_factor;
  uint32_t   _sf_degree;
} PLAINTEXT;
typedef PLAINTEXT* PLAIN;
typedef double _Complex DCMPLX;

/* ---- tensors handed to Prepare_input (include/common/tensor.h:20-63) ---- */
typedef struct {
  SHAPE  _shape;
  double _vals[];
} TENSOR;
#define TENSOR_N(T) (T)->_shape._n
#define TENSOR_C(T) (T)->_shape._c
#define TENSOR_H(T) (T)->_shape._h
#define TENSOR_W(T) (T)->_shape._w
#define TENSOR_SIZE(T) TENSOR_N(T) * TENSOR_C(T) * TENSOR_H(T) * TENSOR_W(T)
static inline float* Slice(float* vec, size_t row_idx, size_t col) { return vec + row_idx * col; }
TENSOR* Alloc_tensor(size_t n, size_t c, size_t h, size_t w, const double* val);
void    Free_tensor(TENSOR* tensor);
void    Print_tensor(FILE* fp, TENSOR* tensor);

/* ---- keys (include/ckks/public_key.h:24-27, switch_key.h:27-29) ---- */
typedef struct {
  POLYNOMIAL _p0, _p1; /* views of one device buffer, (L+k) limbs each, NTT form */
} PUBLIC_KEY;
typedef struct rt_key_parts RT_KEY_PARTS;
typedef struct {
  RT_KEY_PARTS* _public_keys; /* one PUBLIC_KEY per digit */
} SWITCH_KEY;
typedef SWITCH_KEY* SW_KEY;
typedef PUBLIC_KEY* PUB_KEY;

/* ---- fatal errors ---- */
void Rt_fatal(const char* file, int line, const char* fmt, ...) __attribute__((noreturn, format(printf, 3, 4)));
#define FMT_ASSERT(cond, ...)                                \
  do {                                                       \
    if (!(cond)) Rt_fatal(__FILE__, __LINE__, __VA_ARGS__);  \
  } while (0)
#define IS_TRUE(cond, ...) FMT_ASSERT(cond, __VA_ARGS__)

/* ---- lifecycle (context/src/ckks_context.c:84-211, common/src/rt_lib.c:16-21) ---- */
void Prepare_context(void);  /* reads Get_context_params(); aborts if no HIP device is present */
void Finalize_context(void);
void Run_main_graph(void);

/* ---- context getters (context/src/ckks_context.c:213-274, util/src/crt.c:943-1144) ---- */
uint32_t Degree(void);
size_t   Get_q_cnt(void);
size_t   Get_p_cnt(void);
size_t   Get_q_parts(void);
MODULUS* Q_modulus(void);
MODULUS* P_modulus(void);
double   Get_default_sc(void);
size_t   Rt_num_decomp(size_t level); /* Get_num_decomp (util/src/crt.c:1135-1144) */

/* ---- device memory behind `_data` ---- */
int64_t* Rt_dev_alloc(size_t n_words); /* zero-filled */
void     Rt_dev_free(int64_t* p);
void     Rt_dev_copy(int64_t* dst, const int64_t* src, size_t n_words); /* no-op when dst == src */
void     Rt_upload_poly(POLY dst, const int64_t* host_words);   /* Get_num_pq(dst) limbs */
void     Rt_download_poly(int64_t* host_words, POLY src);       /* synchronises */

/* ---- polynomial accessors (include/poly/rns_poly.h:38-284) ---- */
static inline uint32_t Get_rdgree(POLY p) { return p->_ring_degree; }
static inline size_t   Poly_level(POLY p) { return p->_num_primes; }
static inline size_t   Num_p(POLY p) { return p->_num_primes_p; }
static inline size_t   Num_alloc(POLY p) { return p->_num_alloc_primes; }
static inline size_t   Get_num_pq(POLY p) { return p->_num_primes + p->_num_primes_p; }
static inline size_t   Get_poly_alloc_len(POLY p) { return (size_t)p->_ring_degree * p->_num_alloc_primes; }
static inline size_t   Get_poly_len(POLY p) { return (size_t)p->_ring_degree * Get_num_pq(p); }
static inline int64_t* Get_poly_coeffs(POLY p) { return p->_data; }
static inline int64_t* Get_p_coeffs(POLY p) {
  return p->_data + (p->_num_alloc_primes - p->_num_primes_p) * (size_t)p->_ring_degree;
}
static inline bool Is_ntt(POLY p) { return p->_is_ntt; }
static inline void Set_is_ntt(POLY p, bool v) { p->_is_ntt = v; }
static inline void Set_poly_level(POLY p, size_t level) {
  FMT_ASSERT(p->_num_alloc_primes >= level + p->_num_primes_p, "raised level exceed alloc_size");
  p->_num_primes = level;
}
static inline size_t Num_decomp(POLY p) { return Rt_num_decomp(p->_num_primes); }
static inline int64_t* Coeffs(POLY p, size_t limb, uint32_t degree) { return p->_data + limb * (size_t)degree; }
static inline void Set_coeffs(POLY dst, uint32_t limb, uint32_t degree, int64_t* src) {
  Rt_dev_copy(Coeffs(dst, limb, degree), src, degree);
}

/* allocation (include/poly/rns_poly.h:109-154, poly/src/rns_poly.c:18-72, 1319-1325) */
static inline void Alloc_poly_data(POLY p, uint32_t degree, size_t num_q, size_t num_p) {
  p->_ring_degree      = degree;
  p->_num_primes       = num_q;
  p->_num_primes_p     = num_p;
  p->_num_alloc_primes = num_q + num_p;
  p->_is_ntt           = false;
  p->_data             = Rt_dev_alloc((num_q + num_p) * (size_t)degree);
}
void Free_poly_data(POLY p);
/* Generated code passes the third argument as a flag (1 for an extended polynomial) whatever the
 * number of P primes is.  A polynomial with some but not all P limbs means nothing to hybrid key
 * switching (Mod_up, Mod_down assume the full P base), so any non-zero count allocates all of them. */
size_t Get_p_cnt(void);
static inline POLY Alloc_poly(uint32_t degree, size_t num_q, size_t num_p) {
  FMT_ASSERT(num_q > 0, "Alloc_poly: q primes should not be NULL");
  POLY p = (POLY)calloc(1, sizeof(POLYNOMIAL));
  Alloc_poly_data(p, degree, num_q, num_p ? Get_p_cnt() : 0);
  p->_is_ntt = true;
  return p;
}
static inline void Free_poly(POLY p) {
  Free_poly_data(p);
  free(p);
}
POLY_ARR Alloc_polys(uint32_t cnt, uint32_t degree, size_t num_q, size_t num_p); /* one slab */
void     Free_polys(POLY_ARR polys);
void     Init_poly(POLY res, POLY like);
void     Copy_poly(POLY res, POLY poly);
POLY     Init_poly_by_size(POLY res, size_t num_q, bool is_ext);
void     Derive_poly(POLY view, POLY poly, size_t q_cnt, size_t p_cnt); /* rns_poly.c:701-707: non-owning */

/* ---- key switching pieces (poly/src/rns_poly.c:74-529) ---- */
POLY     Decomp(POLY res, POLY poly, uint32_t q_part_idx);
POLY     Mod_up(POLY res, POLY digit, uint32_t q_part_idx);
POLY     Decomp_modup(POLY res, POLY poly, uint32_t q_part_idx);
POLY     Mod_down(POLY res, POLY poly);
POLY     Rescale(POLY res, POLY poly);
POLY     Modswitch(POLY res, POLY poly);
POLY     Mod_down_rescale(POLY res, POLY poly); /* poly is left in coefficient form, as in the reference */
void     Transform_values_from_level0(POLY res, POLY poly);
POLY_ARR Precomp(POLY_ARR res, size_t size, POLY input);
POLY_ARR Rt_alloc_precomp(POLY input, size_t* size); /* Alloc_precomp (rns_poly.c:471-481) without the VALUE_LIST box */
void     Rt_free_precomp(POLY_ARR digits);
POLY     Dot_prod(POLY res, POLY_ARR digits, POLY_ARR key, uint32_t size);
POLY     Extend(POLY res, POLY poly);
void     Conv_poly2ntt_inplace(POLY poly);
void     Conv_ntt2poly_inplace(POLY poly);
POLY     Add_poly(POLY res, POLY a, POLY b);
POLY     Sub_poly(POLY res, POLY a, POLY b);
POLY     Mul_poly(POLY res, POLY a, POLY b);

/* ---- HAL (include/hal/hal.h:24-111, hal/src/hal.c:15-160): return the advanced `res` ---- */
int64_t* Hw_modadd(int64_t* res, int64_t* a, int64_t* b, MODULUS* m, uint32_t degree);
int64_t* Hw_modadd_scalar(int64_t* res, int64_t* a, int64_t s, MODULUS* m, uint32_t degree);
int64_t* Hw_modsub(int64_t* res, int64_t* a, int64_t* b, MODULUS* m, uint32_t degree);
int64_t* Hw_modsub_scalar(int64_t* res, int64_t* a, int64_t s, MODULUS* m, uint32_t degree);
int64_t* Hw_modmul(int64_t* res, int64_t* a, int64_t* b, MODULUS* m, uint32_t degree);
int64_t* Hw_modmul_scalar(int64_t* res, int64_t* a, int64_t s, MODULUS* m, uint32_t degree);
int64_t* Hw_modmuladd(int64_t* res, int64_t* a, int64_t* b, MODULUS* m, uint32_t degree);
int64_t* Hw_modmuladd_scalar(int64_t* res, int64_t* a, int64_t s, MODULUS* m, uint32_t degree);
int64_t* Hw_rotate(int64_t* res, int64_t* a, int64_t* order, MODULUS* m, uint32_t degree);
void     Hw_ntt(int64_t* res, int64_t* a, size_t prime_idx, uint32_t degree);
void     Hw_intt(int64_t* res, int64_t* a, size_t prime_idx, uint32_t degree);

/* ---- keys (include/ckks/key.h:25-119) ---- */
uint32_t    Auto_idx(int32_t rot_idx);
int64_t*    Auto_order(int32_t rot_idx); /* device table of Degree() words */
SW_KEY      Swk(bool is_rot, int32_t rot_idx);
PUB_KEY     Get_swk_at(SW_KEY swk, size_t part);
size_t      Get_swk_size(SW_KEY swk);
static inline POLY Get_pk0(PUB_KEY pk) { return &pk->_p0; }
static inline POLY Get_pk1(PUB_KEY pk) { return &pk->_p1; }
static inline POLY Pk0_at(SW_KEY swk, uint32_t part) { return Get_pk0(Get_swk_at(swk, part)); }
static inline POLY Pk1_at(SW_KEY swk, uint32_t part) { return Get_pk1(Get_swk_at(swk, part)); }
POLY Swk_c0(POLY res, size_t size, bool is_rot, int32_t rot_idx); /* shallow copies of the structs */
POLY Swk_c1(POLY res, size_t size, bool is_rot, int32_t rot_idx);
/* Harness: install a key.  `host_words` is [digit][b | a][(L+k) limbs][N] in NTT
 * form (Generate_switching_key, ckks/src/key_gen.c:127-200).  is_rot false: the
 * relinearisation key; true: the key of rotation rot_idx (or of the conjugation
 * when rot_idx == 2N-1), whose index table is derived here. */
void Rt_load_switch_key(bool is_rot, int32_t rot_idx, const int64_t* host_words);

/* ---- ciphertext (include/ckks/cipher.h:28-251, ckks/src/cipher.c:27-489) ---- */
static inline POLY Get_c0(CIPHER c) { return &c->_c0_poly; }
static inline POLY Get_c1(CIPHER c) { return &c->_c1_poly; }
size_t   Level(CIPHER c);
uint32_t Sc_degree(CIPHER c);
uint32_t Get_slots(CIPHER c);
void     Set_slots(CIPHER c, uint32_t slots);
void     Init_ciph_same_scale(CIPHER res, CIPHER a, CIPHER b);
void     Init_ciph_up_scale(CIPHER res, CIPHER a, CIPHER b);
void     Init_ciph_down_scale(CIPHER res, CIPHER c);
void     Init_ciph_same_scale_ciph3(CIPHER res, CIPHER3 c);
void     Init_ciph3_same_scale_ciph3(CIPHER3 res, CIPHER3 a, CIPHER3 b);
void     Init_ciph3_up_scale(CIPHER3 res, CIPHER a, CIPHER b);
void     Copy_ciph(CIPHER res, CIPHER c);
void     Free_ciph_poly(CIPHER arr, uint32_t cnt);
void     Zero_ciph(CIPHER c);
CIPHER   Add_ciph(CIPHER res, CIPHER a, CIPHER b);
CIPHER   Sub_ciph(CIPHER res, CIPHER a, CIPHER b);
CIPHER3  Mul_ciph3(CIPHER3 res, CIPHER a, CIPHER b);
CIPHER   Relin(CIPHER res, CIPHER3 c);
CIPHER   Mul_ciph(CIPHER res, CIPHER a, CIPHER b);
CIPHER   Rescale_ciph(CIPHER res, CIPHER c);
CIPHER   Modswitch_ciph(CIPHER res, CIPHER c);
CIPHER   Rotate_ciph(CIPHER res, CIPHER c, int32_t rot_idx);
void     Rotate_batch_ciph(CIPHER res_arr, CIPHER c, const int32_t* rot_idx, uint32_t cnt);
CIPHER   Conjugate_ciph(CIPHER res, CIPHER c);

/* ---- plaintexts (include/ckks/plain.h:24-117, ckks/src/plain.c, cipher.c:58-84,373-396) ----
 * Vectors are encoded on the device (ace_encode); a single value (len == 1) becomes the constant
 * residues of Encode_val_at_level (ckks/src/encoder.c:473-575). */
static inline POLY Get_plain_poly(PLAIN p) { return &p->_poly; }
void   Encode_float(PLAIN plain, float* input, size_t len, uint32_t sc_degree, uint32_t level);
void   Encode_double(PLAIN plain, double* input, size_t len, uint32_t sc_degree, uint32_t level);
void   Encode_dcmplx(PLAIN plain, DCMPLX* input, size_t len, uint32_t sc_degree, uint32_t level);
void   Encode_float_mask(PLAIN plain, float cst, size_t len, uint32_t sc_degree, uint32_t level);
void   Encode_double_mask(PLAIN plain, double cst, size_t len, uint32_t sc_degree, uint32_t level);
void   Encode_dcmplx_ext(PLAIN plain, DCMPLX* input, size_t len, uint32_t level, uint32_t p_cnt);
void   Encode_single_float(int64_t* res, float input, uint32_t sc_degree, uint32_t level);   /* host words */
void   Encode_single_double(int64_t* res, double input, uint32_t sc_degree, uint32_t level); /* host words */
double* Get_msg_from_plain(PLAIN plain);        /* decoded real parts, _slots values; caller frees */
DCMPLX* Get_dcmplx_msg_from_plain(PLAIN plain); /* decoded slots; caller frees */
void   Free_plain_poly(PLAIN plain);
void   Init_ciph_same_scale_plain(CIPHER res, CIPHER c, PLAIN plain);
void   Init_ciph_up_scale_plain(CIPHER res, CIPHER c, PLAIN plain);
CIPHER Add_plain(CIPHER res, CIPHER c, PLAIN plain);
CIPHER Mul_plain(CIPHER res, CIPHER c, PLAIN plain);

/* ---- keys, encryption, decryption (ckks/src/key_gen.c:127-262, encryptor.c:19-75, decryptor.c, rtlib.c:164-229) ----
 * Rt_generate_keys: secret (ternary with the context's Hamming weight; uniform ternary when that is 0), public key,
 * relinearisation key and one "fast" rotation key per index of Get_context_params()->_rot_idxs, from a
 * generator seeded with `seed` (0: the environment's RT_HIP_SEED, else the clock).  Prepare_input and
 * Handle_output need it; programs that load their own keys (Rt_load_switch_key) do not. */
void    Rt_generate_keys(uint64_t seed);
void    Rt_generate_rotation_key(int32_t rot_idx);
CIPHER  Encrypt(CIPHER res, PLAIN plain);
void    Rt_decrypt(PLAIN res, CIPHER c);
void    Rt_decode(DCMPLX* res, PLAIN plain); /* plain->_slots values */
void    Prepare_input(TENSOR* input, const char* name);
double* Handle_output(const char* name); /* caller frees */

/* ---- program inputs / outputs (ckks/src/rtlib.c:231-244) ---- */
CIPHERTEXT Get_input_data(const char* name, size_t idx); /* by value; the program owns the polys */
void       Set_output_data(const char* name, size_t idx, CIPHER data); /* deep copy, then frees data's polys */
/* Harness: a ciphertext in NTT form at `level`, both polynomials `level*N` host words */
void Rt_set_input(const char* name, size_t idx, const int64_t* c0, const int64_t* c1, size_t level,
                  double scaling_factor, uint32_t sf_degree, uint32_t slots);
/* Harness: copies an output back (level*N words each); returns its level, 0 when absent */
size_t Rt_get_output(const char* name, size_t idx, int64_t* c0, int64_t* c1, CIPHERTEXT* meta);

/* ---- timing (include/common/rt_stat.h:20-23) ---- */
void Tm_start(const char* msg);
void Tm_taken(const char* msg);

#ifdef __cplusplus
}
#endif
#endif /* RT_HIP_H */
