/* rt_internal.h -- state shared by the files of the host-side runtime (not installed) */
#ifndef RT_INTERNAL_H
#define RT_INTERNAL_H

#include <time.h>

#include "ace_hip.h"
#include "rt_hip.h"

struct rt_key_parts {
  size_t     n;
  int64_t*   dev; /* [digit][b | a][(L+k) limbs][N] */
  PUBLIC_KEY pk[];
};

typedef struct {
  int32_t    rot_idx;
  uint32_t   auto_idx;
  SWITCH_KEY swk;
  int64_t*   order; /* device, NTT-form index table */
} ROT_KEY;

typedef struct {
  char*       name;
  size_t      idx;
  CIPHERTEXT* ct;
} IO_SLOT;

/* What the threads of a program share: the root context (tables in HBM), the parameters and the keys. */
struct rt_state {
  ace_ctx* root; /* made by Prepare_context; the thread that called it issues on it */
  uint64_t generation; /* counts Prepare_context calls: a thread's lane of an earlier context is stale */
  uint32_t N;
  size_t   L, K, parts, input_level;
  MODULUS *q, *p;
  double   sc;
  SWITCH_KEY relin;
  ROT_KEY**  rot; /* entries never move once made (Rt_find_rot is read by every thread) */
  size_t     n_rot;
  /* key material of Rt_generate_keys (rt_ckks.c); absent when the harness loads keys itself */
  int64_t* secret_small; /* host: N signed coefficients */
  int64_t* secret_ntt;   /* device: (L+k) limbs */
  int64_t *pk0, *pk1;    /* device: L limbs each */
};
extern struct rt_state G;

/* What every host thread has for itself, as the reference's OpenMP build keeps its I/O tables, timers and
 * generator per thread (common/src/io_lib.c:24-27, include/common/rtlib_timing.h:123-126, util/src/prng.c:13-16):
 * a context of the root's family (its own HIP stream, scratch arena, buffer pool and recorded calls), the named
 * input and output ciphertexts, the stopwatch of Tm_start.  A thread other than Prepare_context's gets its lane
 * the first time it calls into the runtime; Finalize_context destroys them all. */
struct rt_lane {
  ace_ctx* ctx;
  uint64_t generation;
  unsigned ordinal; /* 0: the thread of Prepare_context */
  IO_SLOT *in, *out;
  size_t   n_in, n_out;
  struct timespec t0;
};
extern __thread struct rt_lane* Rt_lane;
struct rt_lane* Rt_lane_slow(void);
size_t          Rt_lane_count(void); /* threads that have called into the runtime since Prepare_context */
static inline struct rt_lane* Rt_this_lane(void) {
  struct rt_lane* l = Rt_lane;
  return (l && l->generation == G.generation) ? l : Rt_lane_slow();
}
#define RT_CTX (Rt_this_lane()->ctx)
#define LANE (*Rt_this_lane())
/* setting up what all threads share after the first use (rotation keys made on demand, the bootstrap's plaintext
 * diagonals and monomials, kept weight plaintexts): one thread at a time, and what it built is complete on the
 * device (Rt_shared_publish) before the lock is released, because the other threads read it on their own streams */
void Rt_shared_lock(void);
void Rt_shared_unlock(void);
void Rt_shared_publish(void); /* waits for the calling thread's stream */

#define ACE_OK(call)                                                       \
  do {                                                                     \
    if ((call) != 0) Rt_fatal(__FILE__, __LINE__, "%s", ace_last_error()); \
  } while (0)
#define NEED_CTX() FMT_ASSERT(G.root, "Prepare_context() has not run")

size_t   Rt_p_offset(POLY p);
int64_t* Rt_dev_alloc_raw(size_t n_words);
IO_SLOT* Rt_find_slot(IO_SLOT* s, size_t n, const char* name, size_t idx);
IO_SLOT* Rt_add_slot(IO_SLOT** s, size_t* n, const char* name, size_t idx);
void     Rt_install_key(SWITCH_KEY* k, const int64_t* host);
void     Rt_install_key_dev(SWITCH_KEY* k, int64_t* dev); /* takes ownership of the buffer */
ROT_KEY* Rt_rot_entry(int32_t rot_idx);
ROT_KEY* Rt_find_rot(int32_t rot_idx);
void     Rt_shape_ciph(CIPHER res, CIPHER like, double sf, uint32_t deg); /* res shaped like `like`, NTT form */
void     Rt_sample_ternary(int64_t* v, size_t n, size_t hamming_weight);  /* the key generator's host stream */
#define RT_DATA_VERSION 1u /* RT_VERSION_FULL (fhe-cmplr/include/fhe/core/rt_version.h:15-22): 0.0.0 build 1 */
void     Rt_ckks_finalize(void);
void     Rt_bootstrap_finalize(void);
void     Rt_bootstrap_prepare(void);
size_t   Rt_sin_series(size_t hamming_weight, int even, double* coeff, uint32_t* k_bound, uint32_t* double_angle);
void     Rt_series_divide(double* q, size_t* n_q, double* r, size_t* n_r, const double* f, size_t n_f, const double* g, size_t n_g);
/* Encode_val: `level` residues of trunc(value * scale), large products through the approximation factor */
void     Rt_encode_val_words(int64_t* res, double value, uint32_t level, double scale);
void     Rt_copy_words(int64_t* dst, const int64_t* src, size_t n_words);
/* Mul_ciph (+ Add_ciph of the product with itself (+ Add_const of *then_add, if not NULL)) + Rescale_ciph: the same
 * words in fewer launches */
CIPHER   Rt_mul_rescale_ciph(CIPHER res, CIPHER a, CIPHER b, bool twice, const double* then_add);
void     Rt_plaintexts_settle(void); /* the run of weight plaintexts being encoded on the second stream has landed */
int64_t* Rt_plain_prepare(PLAIN plain, uint32_t sc_degree, uint32_t level);
void     Rt_encode_real(PLAIN plain, const void* values, int is_f32, size_t len, uint32_t sc_degree, uint32_t level);
void     Rt_encode_real_batch(int64_t* dev_base, size_t stride, const void* const* values, int is_f32, size_t len,
                              size_t n_vec, uint32_t sc_degree, uint32_t level);

#endif
