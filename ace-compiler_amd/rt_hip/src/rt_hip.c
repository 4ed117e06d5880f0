/* rt_hip.c -- the program-facing runtime of rt_hip.h over the C-ABI of
 * ace_hip.h.  Pure host C: metadata, ownership and argument checking live
 * here; every arithmetic step is one ace_* call that enqueues HIP kernels.
 */
#include "rt_hip.h"

#include <math.h>
#include <pthread.h>
#include <stdarg.h>
#include <time.h>


#include "rt_internal.h"

struct rt_state G;

/* ---- one lane per host thread ---------------------------------------------------------- */
__thread struct rt_lane* Rt_lane;
static pthread_mutex_t   Lanes_lock = PTHREAD_MUTEX_INITIALIZER;
static struct rt_lane**  Lanes; /* every lane made since Prepare_context, [0] = that thread's */
static size_t            N_lanes, Cap_lanes;

static struct rt_lane* new_lane(ace_ctx* ctx) {
  struct rt_lane* l = (struct rt_lane*)calloc(1, sizeof(*l));
  l->ctx            = ctx;
  l->generation     = G.generation;
  pthread_mutex_lock(&Lanes_lock);
  if (N_lanes == Cap_lanes) {
    Cap_lanes = Cap_lanes ? 2 * Cap_lanes : 8;
    Lanes     = (struct rt_lane**)realloc(Lanes, Cap_lanes * sizeof(*Lanes));
  }
  l->ordinal     = (unsigned)N_lanes;
  Lanes[N_lanes] = l;
  __atomic_store_n(&N_lanes, N_lanes + 1, __ATOMIC_RELAXED);
  pthread_mutex_unlock(&Lanes_lock);
  clock_gettime(CLOCK_MONOTONIC, &l->t0);
  return Rt_lane = l;
}
size_t Rt_lane_count(void) { return __atomic_load_n(&N_lanes, __ATOMIC_RELAXED); }
/* the calling thread has no lane of the current context yet */
struct rt_lane* Rt_lane_slow(void) {
  if (!G.root) Rt_fatal(__FILE__, __LINE__, "Prepare_context() has not run");
  ace_ctx* ctx = ace_ctx_share(G.root);
  if (!ctx) Rt_fatal(__FILE__, __LINE__, "no context for this thread: %s", ace_last_error());
  struct rt_lane* lane = new_lane(ctx);
  /* From here on Rt_shared_publish() waits (the count of lanes is above one); what the first thread built while it
   * was alone may still be on its way: wait for everything once. */
  ACE_OK(ace_sync_device(ctx));
  return lane;
}

static pthread_mutex_t Shared_lock;
static pthread_once_t  Shared_once = PTHREAD_ONCE_INIT;
static void            shared_init(void) {
  pthread_mutexattr_t a;
  pthread_mutexattr_init(&a);
  pthread_mutexattr_settype(&a, PTHREAD_MUTEX_RECURSIVE); /* key generation runs inside the bootstrap's set-up */
  pthread_mutex_init(&Shared_lock, &a);
}
void Rt_shared_lock(void) {
  pthread_once(&Shared_once, shared_init);
  pthread_mutex_lock(&Shared_lock);
}
void Rt_shared_unlock(void) { pthread_mutex_unlock(&Shared_lock); }
/* What a thread has built for all of them (keys, plaintexts, tables) on its own stream is complete before another
 * thread, on another stream, can find it; while there is only one thread there is nobody to wait for. */
void Rt_shared_publish(void) {
  if (Rt_lane_count() > 1) ACE_OK(ace_sync(RT_CTX));
}

void Rt_fatal(const char* file, int line, const char* fmt, ...) {
  va_list ap;
  fprintf(stderr, "rt_hip: %s:%d: ", file, line);
  va_start(ap, fmt);
  vfprintf(stderr, fmt, ap);
  va_end(ap);
  fputc('\n', stderr);
  fflush(stderr);
  abort();
}

/* ---- lifecycle ----------------------------------------------------------------- */
void Prepare_context(void) {
  FMT_ASSERT(!G.root, "Prepare_context() called twice");
  FMT_ASSERT(Get_context_params, "the program does not define Get_context_params()");
  CKKS_PARAMS* prm = Get_context_params();
  /* Get_default_num_q_parts (util/src/std_param.c:356-363) */
  size_t parts = prm->_num_q_parts ? prm->_num_q_parts : prm->_mul_depth > 3 ? 3 : prm->_mul_depth == 0 ? 1 : 2;
  G.root = ace_ctx_create(prm->_poly_degree, prm->_mul_depth + 1, prm->_first_mod_size, prm->_scaling_mod_size, parts);
  if (!G.root) Rt_fatal(__FILE__, __LINE__, "%s", ace_last_error());
  if (!ace_has_device(G.root)) Rt_fatal(__FILE__, __LINE__, "no HIP device: this runtime has no CPU path");
  ++G.generation;
  new_lane(G.root); /* this thread issues on the root context itself */
  G.N     = ace_degree(RT_CTX);
  G.L     = ace_num_q(RT_CTX);
  G.K     = ace_num_p(RT_CTX);
  G.parts = ace_num_parts(RT_CTX);
  G.input_level = prm->_input_level;
  G.sc    = ldexp(1.0, (int)prm->_scaling_mod_size);
  G.q     = (MODULUS*)aligned_alloc(16, sizeof(MODULUS) * (G.L + G.K));
  G.p     = G.q + G.L;
  for (size_t i = 0; i < G.L + G.K; ++i) {
    uint64_t f[5];
    ace_modulus(RT_CTX, i, f);
    G.q[i]._val     = (int64_t)f[0];
    G.q[i]._br_k    = (int64_t)f[1];
    G.q[i]._br_m    = (int64_t)f[2];
    G.q[i]._prec128 = ((unsigned __int128)f[4] << 64) | f[3];
  }
  if (Get_rt_data_info && Get_rt_data_info()) Pt_mgr_init(Get_rt_data_info()->_file_name);
}

static void free_key(SWITCH_KEY* k) {
  if (!k->_public_keys) return;
  ace_free(RT_CTX, k->_public_keys->dev);
  free(k->_public_keys);
  k->_public_keys = NULL;
}

static void free_slots(IO_SLOT* s, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    free(s[i].name);
    if (s[i].ct) {
      Free_ciph_poly(s[i].ct, 1);
      free(s[i].ct);
    }
  }
  free(s);
}

void Finalize_context(void) {
  if (!G.root) return;
  Pt_mgr_fini(); /* always: the kept plaintexts are device buffers of this context */
  Rt_bootstrap_finalize();
  Rt_ckks_finalize();
  free_key(&G.relin);
  for (size_t i = 0; i < G.n_rot; ++i) {
    free_key(&G.rot[i]->swk);
    ace_free(RT_CTX, G.rot[i]->order);
  }
  for (size_t i = 0; i < G.n_rot; ++i) free(G.rot[i]);
  free(G.rot);
  /* the other threads' lanes first: their contexts use the root's tables */
  for (size_t i = N_lanes; i-- > 0;) {
    struct rt_lane* l = Lanes[i];
    Rt_lane           = l; /* the slots' polynomials go back through the lane that holds them */
    free_slots(l->in, l->n_in);
    free_slots(l->out, l->n_out);
    if (l->ctx != G.root) ace_ctx_destroy(l->ctx);
    if (i) free(l);
  }
  Rt_lane = NULL;
  if (N_lanes) free(Lanes[0]);
  free(Lanes);
  Lanes   = NULL;
  N_lanes = Cap_lanes = 0;
  free(G.q);
  ace_ctx_destroy(G.root);
  uint64_t generation = G.generation;
  memset(&G, 0, sizeof(G));
  G.generation = generation;
  Report_rtlib_timing(); /* ckks_context.c:207-210: the table of times, if the environment asks for one */
  Close_trace_file();
}

void Run_main_graph(void) {
  NEED_CTX();
  FMT_ASSERT(Main_graph, "the program does not define Main_graph()");
  RTLIB_TM_START(RTM_MAIN_GRAPH, rtm);
  FMT_ASSERT(Main_graph(), "Main_graph() reported failure");
  RTLIB_TM_END(RTM_MAIN_GRAPH, rtm);
}

/* ---- context getters ----------------------------------------------------------- */
uint32_t Degree(void) { return G.N; }
size_t   Get_q_cnt(void) { return G.L; }
size_t   Get_p_cnt(void) { return G.K; }
size_t   Get_q_parts(void) { return G.parts; }
CRT_CONTEXT* Get_crt_context(void) { return G.root; }
NTT_CONTEXT* Get_ntt_ctx(void) { return G.root; }
size_t       Get_part_size(void) { return G.root ? ace_part_size(G.root) : 0; }
MODULUS* Q_modulus(void) { return G.q; }
MODULUS* P_modulus(void) { return G.p; }
double   Get_default_sc(void) { return G.sc; }
size_t   Rt_num_decomp(size_t level) {
  NEED_CTX();
  return ace_num_decomp(RT_CTX, level);
}

/* prime index of a MODULUS the program took from Q_modulus() / P_modulus() */
static size_t prime_of(const MODULUS* m) {
  FMT_ASSERT(m >= G.q && m < G.q + G.L + G.K, "modulus does not belong to this context");
  return (size_t)(m - G.q);
}

/* ---- device memory --------------------------------------------------------------- */
int64_t* Rt_dev_alloc(size_t n_words) {
  NEED_CTX();
  int64_t* p = ace_alloc(RT_CTX, n_words);
  if (!p) Rt_fatal(__FILE__, __LINE__, "device allocation of %zu words failed: %s", n_words, ace_last_error());
  return p;
}
void Rt_sync(void) {
  NEED_CTX();
  ACE_OK(ace_sync(RT_CTX));
}
int64_t* Rt_dev_alloc_raw(size_t n_words) { /* not zero-filled: for buffers written before they are read */
  NEED_CTX();
  int64_t* p = ace_alloc_uninit(RT_CTX, n_words);
  if (!p) Rt_fatal(__FILE__, __LINE__, "device allocation of %zu words failed: %s", n_words, ace_last_error());
  return p;
}
void Rt_copy_words(int64_t* dst, const int64_t* src, size_t n_words) { ACE_OK(ace_copy(RT_CTX, dst, src, n_words)); }
void Rt_dev_free(int64_t* p) {
  if (p && G.root) ace_free(RT_CTX, p);
}
void Rt_dev_copy(int64_t* dst, const int64_t* src, size_t n_words) { ACE_OK(ace_copy(RT_CTX, dst, src, n_words)); }

size_t Rt_p_offset(POLY p) { return (p->_num_alloc_primes - p->_num_primes_p) * (size_t)p->_ring_degree; }

void Rt_upload_poly(POLY dst, const int64_t* host) {
  size_t n = dst->_ring_degree;
  ACE_OK(ace_upload(RT_CTX, dst->_data, host, dst->_num_primes * n));
  if (dst->_num_primes_p)
    ACE_OK(ace_upload(RT_CTX, dst->_data + Rt_p_offset(dst), host + dst->_num_primes * n, dst->_num_primes_p * n));
}
void Rt_download_poly(int64_t* host, POLY src) {
  size_t n = src->_ring_degree;
  ACE_OK(ace_download(RT_CTX, host, src->_data, src->_num_primes * n));
  if (src->_num_primes_p)
    ACE_OK(ace_download(RT_CTX, host + src->_num_primes * n, src->_data + Rt_p_offset(src), src->_num_primes_p * n));
}

/* ---- polynomial containers --------------------------------------------------------- */
void Free_poly_data(POLY p) {
  if (p->_data) {
    Rt_dev_free(p->_data);
    p->_data = NULL;
  }
  p->_num_alloc_primes = 0;
}

POLY_ARR Alloc_polys(uint32_t cnt, uint32_t degree, size_t num_q, size_t num_p) {
  FMT_ASSERT(cnt > 0, "Alloc_polys: zero array size specified");
  POLY_ARR arr  = (POLY_ARR)calloc(cnt, sizeof(POLYNOMIAL));
  if (num_p) num_p = G.K; /* a flag in generated code, like Alloc_poly's */
  size_t   each = (num_q + num_p) * (size_t)degree;
  int64_t* slab = Rt_dev_alloc(each * cnt);
  for (uint32_t i = 0; i < cnt; ++i) {
    arr[i]._ring_degree      = degree;
    arr[i]._num_primes       = num_q;
    arr[i]._num_primes_p     = num_p;
    arr[i]._num_alloc_primes = num_q + num_p;
    arr[i]._is_ntt           = false;
    arr[i]._data             = slab + each * i;
  }
  return arr;
}
void Free_polys(POLY_ARR polys) {
  FMT_ASSERT(polys, "null polynomial array");
  Rt_dev_free(polys[0]._data); /* the slab starts at the first polynomial */
  free(polys);
}

/* res takes the shape of `like`; an existing buffer is kept (and cleared) when it is large enough */
void Init_poly(POLY res, POLY like) {
  if (res == like) return;
  uint32_t n  = like->_ring_degree;
  size_t   nq = like->_num_primes, np = like->_num_primes_p;
  if (res->_data && (res->_ring_degree != n || res->_num_alloc_primes < nq + np)) Free_poly_data(res);
  if (!res->_data) {
    Alloc_poly_data(res, n, nq, np);
  } else {
    ACE_OK(ace_zero(RT_CTX, res->_data, Get_poly_alloc_len(res)));
    res->_num_primes   = nq;
    res->_num_primes_p = np;
  }
  res->_is_ntt = like->_is_ntt;
}

void Copy_poly(POLY res, POLY poly) {
  FMT_ASSERT(res && poly && res->_ring_degree == poly->_ring_degree && res->_num_primes == poly->_num_primes,
             "unmatched primes");
  FMT_ASSERT(res->_num_primes_p >= poly->_num_primes_p, "unmatched p primes cnt");
  size_t n = res->_ring_degree;
  Rt_dev_copy(res->_data, poly->_data, res->_num_primes * n);
  if (poly->_num_primes_p) Rt_dev_copy(res->_data + Rt_p_offset(res), poly->_data + Rt_p_offset(poly), poly->_num_primes_p * n);
  res->_is_ntt = poly->_is_ntt;
}

POLY Init_poly_by_size(POLY res, size_t num_q, bool is_ext) {
  FMT_ASSERT(num_q > 0, "Init_poly_by_size: q primes should not be NULL");
  if (res->_num_alloc_primes) Free_poly_data(res);
  Alloc_poly_data(res, G.N, num_q, is_ext ? G.K : 0);
  res->_is_ntt = true;
  return res;
}

void Derive_poly(POLY view, POLY poly, size_t q_cnt, size_t p_cnt) {
  FMT_ASSERT(q_cnt <= poly->_num_primes && p_cnt <= poly->_num_primes_p, "Derive_poly: view larger than its source");
  *view               = *poly;
  view->_num_primes   = q_cnt;
  view->_num_primes_p = p_cnt;
}

/* an extended polynomial as the kernels address it: P limbs directly after the level's Q limbs */
static void need_packed_ext(POLY p, const char* who) {
  FMT_ASSERT(p->_num_primes_p == G.K && p->_num_alloc_primes == p->_num_primes + G.K,
             "%s: extended polynomial must be allocated at its level (alloc %zu, level %zu, p %zu)", who,
             p->_num_alloc_primes, p->_num_primes, p->_num_primes_p);
}

/* ---- key switching pieces ------------------------------------------------------------ */
static size_t digit_len(size_t level, uint32_t part) {
  size_t ps = ace_part_size(RT_CTX), nd = ace_num_decomp(RT_CTX, level);
  FMT_ASSERT(part < nd, "digit index %u out of range (%zu digits at level %zu)", part, nd, level);
  return part == nd - 1 ? level - ps * part : ps;
}

POLY Decomp(POLY res, POLY poly, uint32_t part) {
  size_t   level = poly->_num_primes, len = digit_len(level, part), start = ace_part_size(RT_CTX) * part;
  uint32_t n = poly->_ring_degree;
  if (res->_num_alloc_primes < len) {
    Free_poly_data(res);
    Alloc_poly_data(res, n, len, 0);
  } else {
    res->_num_primes   = len;
    res->_num_primes_p = 0;
  }
  Rt_dev_copy(res->_data, poly->_data + start * n, len * n);
  res->_is_ntt = poly->_is_ntt;
  return res;
}

POLY Mod_up(POLY res, POLY digit, uint32_t part) {
  need_packed_ext(res, "Mod_up");
  size_t level = res->_num_primes;
  FMT_ASSERT(digit->_ring_degree == res->_ring_degree && digit->_num_primes == digit_len(level, part),
             "Mod_up: digit size does not match part %u at level %zu", part, level);
  ACE_OK(ace_mod_up(RT_CTX, res->_data, digit->_data, level, part, digit->_is_ntt));
  res->_is_ntt = digit->_is_ntt;
  return res;
}

POLY Decomp_modup(POLY res, POLY poly, uint32_t part) {
  need_packed_ext(res, "Decomp_modup");
  FMT_ASSERT(res->_num_primes == poly->_num_primes && res->_ring_degree == poly->_ring_degree,
             "Decomp_modup: result size not match");
  ACE_OK(ace_decomp_modup(RT_CTX, res->_data, poly->_data, poly->_num_primes, part, poly->_is_ntt));
  res->_is_ntt = poly->_is_ntt;
  return res;
}

POLY Mod_down(POLY res, POLY poly) {
  if (!res->_data) Alloc_poly_data(res, poly->_ring_degree, poly->_num_primes, 0);
  need_packed_ext(poly, "Mod_down");
  FMT_ASSERT(res->_ring_degree == poly->_ring_degree && res->_num_primes == poly->_num_primes,
             "Mod_down: result size not match");
  ACE_OK(ace_mod_down(RT_CTX, res->_data, poly->_data, poly->_num_primes, poly->_is_ntt));
  res->_is_ntt = poly->_is_ntt;
  return res;
}

POLY Modswitch(POLY res, POLY poly) {
  size_t level = poly->_num_primes;
  FMT_ASSERT(level >= 2, "polynomial level is too small to support modswitch");
  Set_poly_level(res, level - 1);
  if (res != poly) Rt_dev_copy(res->_data, poly->_data, (level - 1) * (size_t)poly->_ring_degree);
  return res;
}

POLY Rescale(POLY res, POLY poly) {
  size_t level = poly->_num_primes;
  FMT_ASSERT(level >= 2, "Level of rescale opnd is too small");
  FMT_ASSERT(res->_num_primes == level && res->_ring_degree == poly->_ring_degree, "Rescale: primes not match");
  ACE_OK(ace_rescale(RT_CTX, res->_data, poly->_data, level, poly->_is_ntt));
  res->_is_ntt = poly->_is_ntt;
  Set_poly_level(res, level - 1); /* the dropped limb stays allocated, as in the reference */
  return res;
}

POLY Mod_down_rescale(POLY res, POLY poly) {
  need_packed_ext(poly, "Mod_down_rescale");
  size_t level = poly->_num_primes;
  FMT_ASSERT(res->_ring_degree == poly->_ring_degree && res->_num_primes == level && level > 1 && res->_num_primes_p == 0,
             "Reduce_and_rescale_rns: size not match");
  ACE_OK(ace_mod_down_rescale(RT_CTX, res->_data, poly->_data, level, poly->_is_ntt));
  poly->_is_ntt = false;
  Set_poly_level(res, level - 1);
  res->_is_ntt = true;
  return res;
}

void Transform_values_from_level0(POLY res, POLY poly) {
  FMT_ASSERT(res->_ring_degree == poly->_ring_degree, "unmatched ring degree");
  FMT_ASSERT(Get_poly_alloc_len(res) >= Get_poly_len(poly) && res->_num_alloc_primes <= G.L, "not enough memory");
  ACE_OK(ace_transform_from_level0(RT_CTX, res->_data, poly->_data, res->_num_primes));
}

POLY_ARR Precomp(POLY_ARR res, size_t size, POLY input) {
  size_t level = input->_num_primes, T = level + G.K;
  FMT_ASSERT(size == ace_num_decomp(RT_CTX, level), "length of precompute not match");
  bool slab = true;
  for (size_t d = 0; d < size; ++d) {
    need_packed_ext(&res[d], "Precomp");
    FMT_ASSERT(res[d]._num_primes == level, "Precomp: result level not match");
    if (res[d]._data != res[0]._data + d * T * (size_t)G.N) slab = false;
  }
  if (slab) {
    ACE_OK(ace_precomp(RT_CTX, res[0]._data, input->_data, level, input->_is_ntt));
  } else {
    for (size_t d = 0; d < size; ++d)
      ACE_OK(ace_decomp_modup(RT_CTX, res[d]._data, input->_data, level, d, input->_is_ntt));
  }
  for (size_t d = 0; d < size; ++d) res[d]._is_ntt = input->_is_ntt;
  return res;
}

POLY_ARR Rt_alloc_precomp(POLY input, size_t* size) {
  size_t   nd  = Num_decomp(input);
  POLY_ARR arr = Alloc_polys((uint32_t)nd, input->_ring_degree, input->_num_primes, G.K);
  Precomp(arr, nd, input);
  if (size) *size = nd;
  return arr;
}
void Rt_free_precomp(POLY_ARR digits) { Free_polys(digits); }

POLY Dot_prod(POLY res, POLY_ARR digits, POLY_ARR key, uint32_t size) {
  FMT_ASSERT(size > 0, "Dot_prod: no digits");
  Init_poly(res, &digits[0]);
  need_packed_ext(res, "Dot_prod");
  size_t level = res->_num_primes, T = level + G.K, n = G.N;
  bool   slab = true;
  for (uint32_t d = 0; d < size; ++d) {
    FMT_ASSERT(key[d]._num_alloc_primes == G.L + G.K && key[d]._num_primes_p == G.K, "Dot_prod: key size not match");
    if (digits[d]._data != digits[0]._data + d * T * n) slab = false;
    if (d && (key[d]._data - key[d - 1]._data) != (key[1]._data - key[0]._data)) slab = false;
  }
  if (slab) {
    size_t stride = size > 1 ? (size_t)(key[1]._data - key[0]._data) : 0;
    ACE_OK(ace_dot_prod(RT_CTX, res->_data, digits[0]._data, key[0]._data, stride, size, level));
  } else { /* operands scattered: accumulate digit by digit, limb by limb */
    ACE_OK(ace_zero(RT_CTX, res->_data, T * n));
    for (uint32_t d = 0; d < size; ++d) {
      for (size_t t = 0; t < T; ++t) {
        size_t kl = t < level ? t : G.L + (t - level), pi = kl; /* key limb == prime index */
        ACE_OK(ace_hw_modmuladd(RT_CTX, res->_data + t * n, digits[d]._data + t * n, key[d]._data + kl * n, pi, n));
      }
    }
  }
  res->_is_ntt = true;
  return res;
}

POLY Extend(POLY res, POLY poly) {
  FMT_ASSERT(res->_ring_degree == poly->_ring_degree && res->_num_primes == poly->_num_primes, "Extend: size not match");
  FMT_ASSERT(res->_num_alloc_primes == poly->_num_primes + G.K, "Extend: alloc_size not match");
  ACE_OK(ace_extend(RT_CTX, res->_data, poly->_data, poly->_num_primes));
  res->_num_primes_p = G.K;
  res->_is_ntt       = poly->_is_ntt;
  return res;
}

static void transform_inplace(POLY poly, bool inverse) {
  int32_t idx[128];
  size_t  l = poly->_num_primes, k = poly->_num_primes_p, n = poly->_ring_degree;
  FMT_ASSERT(l + k <= 128, "too many limbs");
  for (size_t i = 0; i < l; ++i) idx[i] = (int32_t)i;
  if (inverse)
    ACE_OK(ace_intt(RT_CTX, poly->_data, poly->_data, idx, l, 1, 0));
  else
    ACE_OK(ace_ntt(RT_CTX, poly->_data, poly->_data, idx, l, 1, 0));
  if (k) {
    for (size_t j = 0; j < k; ++j) idx[j] = (int32_t)(G.L + j);
    int64_t* p = poly->_data + Rt_p_offset(poly);
    if (inverse)
      ACE_OK(ace_intt(RT_CTX, p, p, idx, k, 1, 0));
    else
      ACE_OK(ace_ntt(RT_CTX, p, p, idx, k, 1, 0));
  }
  (void)n;
  poly->_is_ntt = !inverse;
}
void Conv_poly2ntt_inplace(POLY poly) {
  FMT_ASSERT(!poly->_is_ntt, "Conv_poly2ntt_inplace: already in NTT form");
  transform_inplace(poly, false);
}
void Conv_ntt2poly_inplace(POLY poly) {
  FMT_ASSERT(poly->_is_ntt, "Conv_ntt2poly_inplace: not in NTT form");
  transform_inplace(poly, true);
}

typedef int (*poly_ew_fn)(ace_ctx*, int64_t*, const int64_t*, const int64_t*, size_t, int);
static POLY poly_ew(poly_ew_fn fn, const char* who, POLY res, POLY a, POLY b) {
  FMT_ASSERT(a->_ring_degree == b->_ring_degree && a->_num_primes == b->_num_primes && res->_num_primes == a->_num_primes,
             "%s: size not match", who);
  FMT_ASSERT(a->_is_ntt == b->_is_ntt, "%s: operands in different forms", who);
  size_t level = a->_num_primes, n = a->_ring_degree, k = a->_num_primes_p < b->_num_primes_p ? a->_num_primes_p : b->_num_primes_p;
  ACE_OK(fn(RT_CTX, res->_data, a->_data, b->_data, level, 0));
  if (k) { /* P limbs of each operand sit at its own offset */
    FMT_ASSERT(k == G.K && res->_num_primes_p == G.K, "%s: p primes not match", who);
    for (size_t j = 0; j < k; ++j) {
      int64_t *r = res->_data + Rt_p_offset(res) + j * n, *x = a->_data + Rt_p_offset(a) + j * n, *y = b->_data + Rt_p_offset(b) + j * n;
      if (fn == ace_poly_add) ACE_OK(ace_hw_modadd(RT_CTX, r, x, y, G.L + j, n));
      else if (fn == ace_poly_sub) ACE_OK(ace_hw_modsub(RT_CTX, r, x, y, G.L + j, n));
      else ACE_OK(ace_hw_modmul(RT_CTX, r, x, y, G.L + j, n));
    }
  }
  res->_is_ntt = a->_is_ntt;
  return res;
}
POLY Add_poly(POLY res, POLY a, POLY b) { return poly_ew(ace_poly_add, "Add_poly", res, a, b); }
POLY Sub_poly(POLY res, POLY a, POLY b) { return poly_ew(ace_poly_sub, "Sub_poly", res, a, b); }
POLY Mul_poly(POLY res, POLY a, POLY b) {
  /* the reference converts coefficient-form operands in place first (rns_poly.c:952-957) */
  if (!a->_is_ntt) Conv_poly2ntt_inplace(a);
  if (!b->_is_ntt) Conv_poly2ntt_inplace(b);
  return poly_ew(ace_poly_mul, "Mul_poly", res, a, b);
}

/* ---- HAL ------------------------------------------------------------------------------- */
#define HW2(NAME, FN)                                                                       \
  int64_t* NAME(int64_t* res, int64_t* a, int64_t* b, MODULUS* m, uint32_t degree) {        \
    ACE_OK(FN(RT_CTX, res, a, b, prime_of(m), degree));                                      \
    return res + degree;                                                                    \
  }
#define HW1(NAME, FN)                                                                       \
  int64_t* NAME(int64_t* res, int64_t* a, int64_t s, MODULUS* m, uint32_t degree) {         \
    int64_t q = m->_val;                                                                    \
    s %= q;                                                                                 \
    if (s < 0) s += q;                                                                      \
    ACE_OK(FN(RT_CTX, res, a, s, prime_of(m), degree));                                      \
    return res + degree;                                                                    \
  }
HW2(Hw_modadd, ace_hw_modadd)
HW2(Hw_modsub, ace_hw_modsub)
HW2(Hw_modmul, ace_hw_modmul)
HW2(Hw_modmuladd, ace_hw_modmuladd)
HW1(Hw_modadd_scalar, ace_hw_modadd_scalar)
HW1(Hw_modsub_scalar, ace_hw_modsub_scalar)
HW1(Hw_modmul_scalar, ace_hw_modmul_scalar)
HW1(Hw_modmuladd_scalar, ace_hw_modmuladd_scalar)

int64_t* Hw_rotate(int64_t* res, int64_t* a, int64_t* order, MODULUS* m, uint32_t degree) {
  ACE_OK(ace_hw_rotate(RT_CTX, res, a, order, prime_of(m), degree));
  return res + degree;
}
void Hw_ntt(int64_t* res, int64_t* a, size_t prime_idx, uint32_t degree) {
  int32_t idx = (int32_t)prime_idx;
  FMT_ASSERT(degree == G.N, "Hw_ntt: degree not match");
  ACE_OK(ace_ntt(RT_CTX, res, a, &idx, 1, 1, 0));
}
void Hw_intt(int64_t* res, int64_t* a, size_t prime_idx, uint32_t degree) {
  int32_t idx = (int32_t)prime_idx;
  FMT_ASSERT(degree == G.N, "Hw_intt: degree not match");
  ACE_OK(ace_intt(RT_CTX, res, a, &idx, 1, 1, 0));
}

/* ---- keys --------------------------------------------------------------------------------- */
/* a switch key over a device buffer [digit][b | a][(L+k) limbs][N] that the key takes ownership of */
void Rt_install_key_dev(SWITCH_KEY* k, int64_t* dev) {
  size_t T = G.L + G.K, n = G.N;
  free_key(k);
  RT_KEY_PARTS* kp = (RT_KEY_PARTS*)calloc(1, sizeof(RT_KEY_PARTS) + G.parts * sizeof(PUBLIC_KEY));
  kp->n   = G.parts;
  kp->dev = dev;
  for (size_t d = 0; d < G.parts; ++d) {
    POLYNOMIAL v = {G.N, T, G.L, G.K, true, kp->dev + 2 * d * T * n};
    kp->pk[d]._p0 = v;
    v._data += T * n;
    kp->pk[d]._p1 = v;
  }
  Rt_shared_publish(); /* other threads read the key on their own streams as soon as they can see it */
  __atomic_store_n(&k->_public_keys, kp, __ATOMIC_RELEASE);
}
void Rt_install_key(SWITCH_KEY* k, const int64_t* host) {
  size_t   words = 2 * G.parts * (G.L + G.K) * G.N;
  int64_t* dev   = Rt_dev_alloc_raw(words);
  ACE_OK(ace_upload(RT_CTX, dev, host, words));
  Rt_install_key_dev(k, dev);
}

/* Entries are made one at a time (under the shared lock where threads may race for a key) and never move: the
 * table of pointers has a fixed size, an entry is complete before the count that makes it visible goes up. */
#define RT_MAX_ROT_KEYS 8192
ROT_KEY* Rt_find_rot(int32_t rot_idx) {
  size_t n = __atomic_load_n(&G.n_rot, __ATOMIC_ACQUIRE);
  for (size_t i = 0; i < n; ++i)
    if (G.rot[i]->rot_idx == rot_idx) return G.rot[i];
  return NULL;
}

/* the entry of a rotation index, created with its automorphism table when new */
ROT_KEY* Rt_rot_entry(int32_t rot_idx) {
  ROT_KEY* r = Rt_find_rot(rot_idx);
  if (r) return r;
  Rt_shared_lock();
  r = Rt_find_rot(rot_idx);
  if (!r) {
    if (!G.rot) G.rot = (ROT_KEY**)calloc(RT_MAX_ROT_KEYS, sizeof(ROT_KEY*));
    FMT_ASSERT(G.n_rot < RT_MAX_ROT_KEYS, "more than %d rotation keys", RT_MAX_ROT_KEYS);
    r           = (ROT_KEY*)calloc(1, sizeof(*r));
    r->rot_idx  = rot_idx;
    r->auto_idx = (uint32_t)rot_idx == 2 * G.N - 1 ? 2 * G.N - 1 : ace_find_automorphism_index(RT_CTX, rot_idx);
    r->order    = Rt_dev_alloc(G.N);
    ACE_OK(ace_automorphism_order(RT_CTX, r->order, r->auto_idx, 1)); /* waits for the upload */
    G.rot[G.n_rot] = r;
    __atomic_store_n(&G.n_rot, G.n_rot + 1, __ATOMIC_RELEASE);
  }
  Rt_shared_unlock();
  return r;
}

void Rt_load_switch_key(bool is_rot, int32_t rot_idx, const int64_t* host_words) {
  NEED_CTX();
  Rt_install_key(is_rot ? &Rt_rot_entry(rot_idx)->swk : &G.relin, host_words);
}

uint32_t Auto_idx(int32_t rot_idx) {
  ROT_KEY* r = Rt_find_rot(rot_idx);
  FMT_ASSERT(r, "cannot get precompute automorphism index of rotation %d", rot_idx);
  return r->auto_idx;
}
int64_t* Auto_order(int32_t rot_idx) {
  ROT_KEY* r = Rt_find_rot(rot_idx);
  FMT_ASSERT(r, "cannot find precomputed automorphism order of rotation %d", rot_idx);
  return r->order;
}
SW_KEY Swk(bool is_rot, int32_t rot_idx) {
  if (!is_rot) {
    FMT_ASSERT(G.relin._public_keys, "no relinearisation key loaded");
    return &G.relin;
  }
  ROT_KEY* r = Rt_find_rot(rot_idx);
  FMT_ASSERT(r, "cannot find auto key of rotation %d", rot_idx);
  return &r->swk;
}
PUB_KEY Get_swk_at(SW_KEY swk, size_t part) {
  FMT_ASSERT(swk && swk->_public_keys, "null swk");
  FMT_ASSERT(part < swk->_public_keys->n, "idx outof bound");
  return &swk->_public_keys->pk[part];
}
size_t Get_swk_size(SW_KEY swk) {
  FMT_ASSERT(swk && swk->_public_keys, "null swk");
  return swk->_public_keys->n;
}
POLY Swk_c0(POLY res, size_t size, bool is_rot, int32_t rot_idx) {
  SW_KEY k = Swk(is_rot, rot_idx);
  FMT_ASSERT(size <= Get_swk_size(k), "extra size provided");
  for (size_t d = 0; d < size; ++d) res[d] = k->_public_keys->pk[d]._p0;
  return res;
}
POLY Swk_c1(POLY res, size_t size, bool is_rot, int32_t rot_idx) {
  SW_KEY k = Swk(is_rot, rot_idx);
  FMT_ASSERT(size <= Get_swk_size(k), "extra size provided");
  for (size_t d = 0; d < size; ++d) res[d] = k->_public_keys->pk[d]._p1;
  return res;
}

/* ---- ciphertext metadata --------------------------------------------------------------------- */
size_t Level(CIPHER c) {
  FMT_ASSERT(c->_c0_poly._num_primes == c->_c1_poly._num_primes, "unmatched level in ciph");
  return c->_c0_poly._num_primes;
}
uint32_t Sc_degree(CIPHER c) { return c->_sf_degree; }
uint32_t Get_slots(CIPHER c) { return c->_slots; }
void     Set_slots(CIPHER c, uint32_t slots) { c->_slots = slots; }

/* shape res like `like` with the given scale; polynomials end up in NTT form at like's level */
void Rt_shape_ciph(CIPHER res, CIPHER like, double sf, uint32_t deg) {
  res->_scaling_factor = sf;
  res->_sf_degree      = deg;
  res->_slots          = like->_slots;
  if (res != like) {
    Init_poly(&res->_c0_poly, &like->_c0_poly);
    Init_poly(&res->_c1_poly, &like->_c1_poly);
  }
  res->_c0_poly._is_ntt = res->_c1_poly._is_ntt = true;
  Set_poly_level(&res->_c0_poly, Level(like));
  Set_poly_level(&res->_c1_poly, Level(like));
}
static void shape_ciph3(CIPHER3 res, POLY l0, POLY l1, POLY l2, double sf, uint32_t deg, uint32_t slots) {
  res->_scaling_factor = sf;
  res->_sf_degree      = deg;
  res->_slots          = slots;
  Init_poly(&res->_c0_poly, l0);
  Init_poly(&res->_c1_poly, l1);
  Init_poly(&res->_c2_poly, l2);
  res->_c0_poly._is_ntt = res->_c1_poly._is_ntt = res->_c2_poly._is_ntt = true;
}
/* the operand at the lower level; an empty first operand defers to the second (Adjust_level) */
static CIPHER lower_of(CIPHER a, CIPHER b) {
  FMT_ASSERT(a && b, "invalid ciph");
  if (!a->_c0_poly._data) return b;
  FMT_ASSERT(b->_c0_poly._data, "poly coeffs of input ciph is invalid");
  return Level(a) > Level(b) ? b : a;
}

void Init_ciph_same_scale(CIPHER res, CIPHER a, CIPHER b) {
  CIPHER pick = b ? lower_of(a, b) : a;
  if (pick == b && !a->_c0_poly._data) {
    /* accumulator idiom: an empty first operand becomes a zero ciphertext shaped like the second */
    Rt_shape_ciph(a, b, b->_scaling_factor, b->_sf_degree);
    a->_c0_poly._is_ntt = b->_c0_poly._is_ntt;
    a->_c1_poly._is_ntt = b->_c1_poly._is_ntt;
  } else if (!pick->_c0_poly._data) {
    memset(res, 0, sizeof(*res));
    return;
  }
  Rt_shape_ciph(res, pick, pick->_scaling_factor, pick->_sf_degree);
}
void Init_ciph_up_scale(CIPHER res, CIPHER a, CIPHER b) {
  Rt_shape_ciph(res, lower_of(a, b), a->_scaling_factor * b->_scaling_factor, a->_sf_degree + b->_sf_degree);
}
void Init_ciph_down_scale(CIPHER res, CIPHER c) {
  FMT_ASSERT(c->_sf_degree >= 2, "Scale degree of result dec to zero");
  Rt_shape_ciph(res, c, c->_scaling_factor / G.sc, c->_sf_degree - 1);
}
void Init_ciph_same_scale_ciph3(CIPHER res, CIPHER3 c) {
  FMT_ASSERT(res, "invalid ciphertext");
  res->_scaling_factor = c->_scaling_factor;
  res->_sf_degree      = c->_sf_degree;
  res->_slots          = c->_slots;
  Init_poly(&res->_c0_poly, &c->_c0_poly);
  Init_poly(&res->_c1_poly, &c->_c1_poly);
  res->_c0_poly._is_ntt = res->_c1_poly._is_ntt = true;
}
void Init_ciph3_same_scale_ciph3(CIPHER3 res, CIPHER3 a, CIPHER3 b) {
  CIPHER3 pick = a;
  if (b && a->_c0_poly._data && b->_c0_poly._data && b->_c0_poly._num_primes < a->_c0_poly._num_primes) pick = b;
  if (b && !a->_c0_poly._data) pick = b;
  if (res != pick)
    shape_ciph3(res, &pick->_c0_poly, &pick->_c1_poly, &pick->_c2_poly, pick->_scaling_factor, pick->_sf_degree,
                pick->_slots);
}
void Init_ciph3_up_scale(CIPHER3 res, CIPHER a, CIPHER b) {
  CIPHER pick = lower_of(a, b);
  shape_ciph3(res, &pick->_c0_poly, &pick->_c0_poly, &pick->_c0_poly, a->_scaling_factor * b->_scaling_factor,
              a->_sf_degree + b->_sf_degree, pick->_slots);
}

void Copy_ciph(CIPHER res, CIPHER c) {
  if (res == c) return;
  res->_scaling_factor = c->_scaling_factor;
  res->_sf_degree      = c->_sf_degree;
  res->_slots          = c->_slots;
  Init_poly(&res->_c0_poly, &c->_c0_poly);
  Init_poly(&res->_c1_poly, &c->_c1_poly);
  Copy_poly(&res->_c0_poly, &c->_c0_poly);
  Copy_poly(&res->_c1_poly, &c->_c1_poly);
}
void Free_ciph_poly(CIPHER arr, uint32_t cnt) {
  for (uint32_t i = 0; i < cnt; ++i) {
    Free_poly_data(&arr[i]._c0_poly);
    Free_poly_data(&arr[i]._c1_poly);
  }
}
void Zero_ciph(CIPHER c) {
  Free_ciph_poly(c, 1);
  memset(c, 0, sizeof(*c));
}

/* ---- ciphertext arithmetic (ckks/src/evaluator.c:46-595) ---------------------------------------- */
typedef POLY (*poly2_fn)(POLY, POLY, POLY);
static CIPHER ciph_ew(poly2_fn fn, CIPHER res, CIPHER a, CIPHER b) {
  FMT_ASSERT(a->_scaling_factor == b->_scaling_factor, "Scaling factors are not equal.");
  size_t la = Level(a), lb = Level(b), l = la < lb ? la : lb;
  CIPHER low = la <= lb ? a : b;
  if (res != a && res != b) Rt_shape_ciph(res, low, low->_scaling_factor, low->_sf_degree);
  /* the higher operand is viewed at the common level for the duration of the call */
  CIPHERTEXT va = *a, vb = *b;
  va._c0_poly._num_primes = va._c1_poly._num_primes = l;
  vb._c0_poly._num_primes = vb._c1_poly._num_primes = l;
  Set_poly_level(&res->_c0_poly, l);
  Set_poly_level(&res->_c1_poly, l);
  fn(&res->_c0_poly, &va._c0_poly, &vb._c0_poly);
  fn(&res->_c1_poly, &va._c1_poly, &vb._c1_poly);
  return res;
}
CIPHER Add_ciph(CIPHER res, CIPHER a, CIPHER b) { return ciph_ew(Add_poly, res, a, b); }
CIPHER Sub_ciph(CIPHER res, CIPHER a, CIPHER b) { return ciph_ew(Sub_poly, res, a, b); }

CIPHER3 Mul_ciph3(CIPHER3 res, CIPHER a, CIPHER b) {
  Init_ciph3_up_scale(res, a, b);
  size_t l = res->_c0_poly._num_primes;
  FMT_ASSERT(a->_c0_poly._is_ntt && b->_c0_poly._is_ntt, "Mul_ciph3: operands must be in NTT form");
  ACE_OK(ace_mul_ciph3(RT_CTX, res->_c0_poly._data, res->_c1_poly._data, res->_c2_poly._data, a->_c0_poly._data,
                       a->_c1_poly._data, b->_c0_poly._data, b->_c1_poly._data, l));
  return res;
}

CIPHER Relin(CIPHER res, CIPHER3 c) {
  FMT_ASSERT(G.relin._public_keys, "no relinearisation key loaded");
  Init_ciph_same_scale_ciph3(res, c);
  ACE_OK(ace_relin(RT_CTX, res->_c0_poly._data, res->_c1_poly._data, c->_c0_poly._data, c->_c1_poly._data,
                   c->_c2_poly._data, G.relin._public_keys->dev, c->_c0_poly._num_primes));
  return res;
}

CIPHER Mul_ciph(CIPHER res, CIPHER a, CIPHER b) {
  CIPHERTEXT3 t;
  memset(&t, 0, sizeof(t));
  Mul_ciph3(&t, a, b);
  Relin(res, &t);
  Free_poly_data(&t._c0_poly);
  Free_poly_data(&t._c1_poly);
  Free_poly_data(&t._c2_poly);
  return res;
}

/* Mul_ciph followed by Rescale_ciph on its result, in one set of launches: the key switch's Mod_down and the Rescale
 * share a forward transform there.  The words and the scale are those of the two calls one after the other
 * (evaluator.c:142-190, 288-306, 342-362).  twice: with Add_ciph of the product with itself between the two
 * (chebyshev_impl.c:563-565).  res may be one of the operands. */
CIPHER Rt_mul_rescale_ciph(CIPHER res, CIPHER a, CIPHER b, bool twice, const double* then_add) {
  FMT_ASSERT(G.relin._public_keys, "no relinearisation key loaded");
  CIPHER pick  = lower_of(a, b);
  size_t level = Level(pick);
  FMT_ASSERT(level > 1, "rescale: multiply level is not big enought for more operation");
  FMT_ASSERT(a->_c0_poly._is_ntt && b->_c0_poly._is_ntt, "Mul_ciph3: operands must be in NTT form");
  FMT_ASSERT(a->_sf_degree + b->_sf_degree >= 2, "Scale degree of result dec to zero");
  CIPHERTEXT t;
  memset(&t, 0, sizeof(t));
  Rt_shape_ciph(&t, pick, a->_scaling_factor * b->_scaling_factor / G.sc, a->_sf_degree + b->_sf_degree - 1);
  if (then_add) { /* Add_const of the doubled product, at the product's scale (evaluator.c:127-140) */
    int64_t w[128];
    FMT_ASSERT(twice && level <= 128, "Rt_mul_rescale_ciph: a constant goes with the doubled product");
    Rt_encode_val_words(w, *then_add, (uint32_t)level, a->_scaling_factor * b->_scaling_factor);
    ACE_OK(ace_mul_relin_double_add_rescale(RT_CTX, t._c0_poly._data, t._c1_poly._data, a->_c0_poly._data,
                                            a->_c1_poly._data, b->_c0_poly._data, b->_c1_poly._data,
                                            G.relin._public_keys->dev, w, level));
  } else {
    ACE_OK((twice ? ace_mul_relin_double_rescale : ace_mul_relin_rescale)(
        RT_CTX, t._c0_poly._data, t._c1_poly._data, a->_c0_poly._data, a->_c1_poly._data, b->_c0_poly._data,
        b->_c1_poly._data, G.relin._public_keys->dev, level));
  }
  Set_poly_level(&t._c0_poly, level - 1);
  Set_poly_level(&t._c1_poly, level - 1);
  Free_poly_data(&res->_c0_poly);
  Free_poly_data(&res->_c1_poly);
  *res = t;
  return res;
}

CIPHER Rescale_ciph(CIPHER res, CIPHER c) {
  size_t level = Level(c);
  FMT_ASSERT(level > 1, "rescale: multiply level is not big enought for more operation");
  double   sf  = c->_scaling_factor / G.sc;
  uint32_t deg = c->_sf_degree - 1;
  Rt_shape_ciph(res, c, sf, deg);
  ACE_OK(ace_rescale_ciph(RT_CTX, res->_c0_poly._data, res->_c1_poly._data, c->_c0_poly._data, c->_c1_poly._data, level));
  Set_poly_level(&res->_c0_poly, level - 1);
  Set_poly_level(&res->_c1_poly, level - 1);
  return res;
}

void Rotate_batch_ciph(CIPHER res_arr, CIPHER c, const int32_t* rot_idx, uint32_t cnt) {
  if (!cnt) return;
  size_t level = Level(c), n = G.N;
  /* results are gathered in two slabs, then handed to the caller's structs */
  const int64_t** keys   = (const int64_t**)malloc(cnt * sizeof(*keys));
  const int64_t** orders = (const int64_t**)malloc(cnt * sizeof(*orders));
  uint32_t*       where  = (uint32_t*)malloc(cnt * sizeof(*where));
  uint32_t        m      = 0;
  for (uint32_t i = 0; i < cnt; ++i) {
    if (rot_idx[i] == 0) {
      Copy_ciph(&res_arr[i], c);
      continue;
    }
    ROT_KEY* r = Rt_find_rot(rot_idx[i]);
    FMT_ASSERT(r, "cannot find auto key of rotation %d", rot_idx[i]);
    keys[m]   = r->swk._public_keys->dev;
    orders[m] = r->order;
    where[m++] = i;
  }
  if (m) {
    int64_t *s0 = Rt_dev_alloc(m * level * n), *s1 = Rt_dev_alloc(m * level * n);
    ACE_OK(ace_rotate_batch(RT_CTX, s0, s1, c->_c0_poly._data, c->_c1_poly._data, keys, orders, m, level));
    for (uint32_t j = 0; j < m; ++j) {
      CIPHER out = &res_arr[where[j]];
      Rt_shape_ciph(out, c, c->_scaling_factor, c->_sf_degree);
      Rt_dev_copy(out->_c0_poly._data, s0 + j * level * n, level * n);
      Rt_dev_copy(out->_c1_poly._data, s1 + j * level * n, level * n);
    }
    Rt_dev_free(s0);
    Rt_dev_free(s1);
  }
  free(keys);
  free(orders);
  free(where);
}

/* res may be c: the rotated polynomials are formed apart and copied over the operand afterwards, as Fast_rotate
 * assigns its result last (evaluator.c:503-522) */
CIPHER Rotate_ciph(CIPHER res, CIPHER c, int32_t rot_idx) {
  Rotate_batch_ciph(res, c, &rot_idx, 1);
  return res;
}
CIPHER Conjugate_ciph(CIPHER res, CIPHER c) { return Rotate_ciph(res, c, (int32_t)(2 * G.N - 1)); }

/* ---- program inputs / outputs -------------------------------------------------------------------- */
IO_SLOT* Rt_find_slot(IO_SLOT* s, size_t n, const char* name, size_t idx) {
  for (size_t i = 0; i < n; ++i)
    if (s[i].idx == idx && strcmp(s[i].name, name) == 0) return &s[i];
  return NULL;
}
IO_SLOT* Rt_add_slot(IO_SLOT** s, size_t* n, const char* name, size_t idx) {
  IO_SLOT* f = Rt_find_slot(*s, *n, name, idx);
  if (f) {
    if (f->ct) {
      Free_ciph_poly(f->ct, 1);
      free(f->ct);
    }
    f->ct = NULL;
    return f;
  }
  *s = (IO_SLOT*)realloc(*s, (*n + 1) * sizeof(IO_SLOT));
  f  = &(*s)[(*n)++];
  f->name = strdup(name);
  f->idx  = idx;
  f->ct   = NULL;
  return f;
}

void Rt_set_input(const char* name, size_t idx, const int64_t* c0, const int64_t* c1, size_t level, double sf,
                  uint32_t sf_degree, uint32_t slots) {
  NEED_CTX();
  FMT_ASSERT(level >= 1 && level <= G.L, "Rt_set_input: level out of range");
  IO_SLOT*    s  = Rt_add_slot(&LANE.in, &LANE.n_in, name, idx);
  CIPHERTEXT* ct = (CIPHERTEXT*)calloc(1, sizeof(CIPHERTEXT));
  Alloc_poly_data(&ct->_c0_poly, G.N, level, 0);
  Alloc_poly_data(&ct->_c1_poly, G.N, level, 0);
  ct->_c0_poly._is_ntt = ct->_c1_poly._is_ntt = true;
  Rt_upload_poly(&ct->_c0_poly, c0);
  Rt_upload_poly(&ct->_c1_poly, c1);
  ct->_scaling_factor = sf;
  ct->_sf_degree      = sf_degree;
  ct->_slots          = slots;
  s->ct               = ct;
}

CIPHERTEXT Get_input_data(const char* name, size_t idx) {
  IO_SLOT* s = Rt_find_slot(LANE.in, LANE.n_in, name, idx);
  FMT_ASSERT(s && s->ct, "not find data: input \"%s\"[%zu]", name, idx);
  CIPHERTEXT ret = *s->ct; /* ownership of the polynomials moves to the program */
  free(s->ct);
  s->ct = NULL;
  return ret;
}

void Set_output_data(const char* name, size_t idx, CIPHER data) {
  IO_SLOT*    s  = Rt_add_slot(&LANE.out, &LANE.n_out, name, idx);
  CIPHERTEXT* ct = (CIPHERTEXT*)calloc(1, sizeof(CIPHERTEXT));
  Copy_ciph(ct, data);
  Free_ciph_poly(data, 1);
  s->ct = ct;
}

size_t Rt_get_output(const char* name, size_t idx, int64_t* c0, int64_t* c1, CIPHERTEXT* meta) {
  IO_SLOT* s = Rt_find_slot(LANE.out, LANE.n_out, name, idx);
  if (!s || !s->ct) return 0;
  if (c0) Rt_download_poly(c0, &s->ct->_c0_poly);
  if (c1) Rt_download_poly(c1, &s->ct->_c1_poly);
  if (meta) {
    *meta = *s->ct;
    meta->_c0_poly._data = meta->_c1_poly._data = NULL;
  }
  return Level(s->ct);
}

/* ---- timing ------------------------------------------------------------------------------------------ */
static double since_start(void) {
  struct timespec t;
  clock_gettime(CLOCK_MONOTONIC, &t);
  return (double)(t.tv_sec - LANE.t0.tv_sec) + 1e-9 * (double)(t.tv_nsec - LANE.t0.tv_nsec);
}
void Tm_start(const char* msg) {
  clock_gettime(CLOCK_MONOTONIC, &LANE.t0);
  if (msg) printf("[RT_STAT] %s: timer started\n", msg);
}
void Tm_taken(const char* msg) {
  if (G.root) (void)ace_sync(RT_CTX); /* the stream is asynchronous: wait, so the figure covers the work */
  printf("[RT_STAT] %s: %.6f s\n", msg ? msg : "", since_start());
}
