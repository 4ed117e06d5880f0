// C-ABI of the MI355X CKKS polynomial runtime (include/ace_hip.h): context
// life cycle, device memory, and the host-side sequencing of kernels for each
// reference operation.  One HIP stream per context; every call only enqueues.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/ace_hip.h"
#include "ace_context.h"
#include "ace_kernels.h"

using namespace ace;

namespace {

thread_local std::string g_err;

int fail(const std::string& msg) {
  g_err = msg;
  return 1;
}

#define HIP_OK(expr)                                                                     \
  do {                                                                                   \
    hipError_t _e = (expr);                                                              \
    if (_e != hipSuccess) throw std::runtime_error(std::string(#expr) + ": " + hipGetErrorString(_e)); \
  } while (0)

// per-(level, digit) constants of Decomp_modup, resident in HBM
struct ModUpDev {
  ModUpTable t;
  u64* hat = nullptr;         // [nd][nc]
  u64* scale_ntt = nullptr;   // [nd][2]: (1/N * hat_inv, Shoup)
  u64* scale_coef = nullptr;  // [nd][2]: (hat_inv, Shoup)
  LimbMap digit_lm{}, compl_lm{}, compl_pos{};
  ConvMap conv{};
};

struct RescaleDev {
  u64* sw = nullptr;    // [level-1][3]: K, K', diff
  u64* tail = nullptr;  // [level-1][2]: q_l^-1, Shoup
};

}  // namespace

struct ace_ctx {
  HostContext h;
  bool device_ok = false;  // false: host tables only (no GPU present), every compute call is rejected
  hipStream_t stream = nullptr;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  DevCtx d{};
  std::vector<void*> owned;  // device allocations freed with the context
  std::map<std::pair<size_t, size_t>, ModUpDev> modup;
  std::map<size_t, RescaleDev> rescale;
  // Mod_down / Extend constants
  u64* phat = nullptr;        // [K][L]
  u64* pscale_ntt = nullptr;  // [K][2]
  u64* pscale_coef = nullptr; // [K][2]
  u64* pinv = nullptr;        // [L][2]
  u64* pmodq = nullptr;       // [L][2]
  LimbMap q_lm{}, p_lm{};     // identity maps: limb t -> prime t / prime L+t
  // scratch arena
  u64* ws = nullptr;
  size_t ws_words = 0, ws_used = 0;

  template <class T>
  T* upload_vec(const std::vector<T>& v) {
    T* p = nullptr;
    HIP_OK(hipMalloc((void**)&p, std::max<size_t>(v.size(), 1) * sizeof(T)));
    HIP_OK(hipMemcpy(p, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
    owned.push_back(p);
    return p;
  }
  ShoupConst sc(u64 w, size_t prime) const { return {w, shoup(w, h.primes[prime].q)}; }

  void ensure_ws(size_t words) {
    if (words <= ws_words) return;
    HIP_OK(hipStreamSynchronize(stream));
    if (ws) HIP_OK(hipFree(ws));
    ws = nullptr;
    ws_words = 0;
    HIP_OK(hipMalloc((void**)&ws, words * sizeof(u64)));
    ws_words = words;
  }
  u64* take(size_t words) {
    if (ws_used + words > ws_words) throw std::runtime_error("internal: scratch arena too small");
    u64* p = ws + ws_used;
    ws_used += words;
    return p;
  }
  size_t std_ws(size_t level) const {  // enough for every composite op at `level`
    return (h.num_decomp(level) + 10) * (level + h.K + 1) * (size_t)h.N;
  }

  const ModUpDev& modup_at(size_t level, size_t part) {
    auto key = std::make_pair(level, part);
    auto it = modup.find(key);
    if (it != modup.end()) return it->second;
    ModUpDev m;
    m.t = h.modup_table(level, part);
    size_t nd = m.t.digit.size(), nc = m.t.compl_idx.size(), start = h.part_size * part;
    m.hat = upload_vec(m.t.hat);
    std::vector<u64> sn(2 * nd), scf(2 * nd);
    for (size_t i = 0; i < nd; ++i) {
      size_t pi = m.t.digit[i];
      u64 q = h.primes[pi].q;
      u64 a = mul_mod(h.primes[pi].ninv, m.t.hat_inv[i], q);
      sn[2 * i] = a;              sn[2 * i + 1] = shoup(a, q);
      scf[2 * i] = m.t.hat_inv[i]; scf[2 * i + 1] = shoup(m.t.hat_inv[i], q);
      m.digit_lm.prime[i] = (uint8_t)pi;
    }
    m.scale_ntt = upload_vec(sn);
    m.scale_coef = upload_vec(scf);
    for (size_t j = 0; j < nc; ++j) {
      size_t pos = j < start ? j : j + nd;
      m.compl_lm.prime[j] = (uint8_t)m.t.compl_idx[j];
      m.compl_pos.prime[j] = (uint8_t)pos;
      m.conv.prime[j] = (uint8_t)m.t.compl_idx[j];
      m.conv.out_limb[j] = (uint8_t)pos;
    }
    return modup.emplace(key, std::move(m)).first->second;
  }

  const RescaleDev& rescale_at(size_t level) {
    auto it = rescale.find(level);
    if (it != rescale.end()) return it->second;
    std::vector<u64> qi, nqi;
    h.rescale_table(level, qi, nqi);
    u64 ql = h.primes[level - 1].q;
    std::vector<u64> sw(3 * (level - 1)), tl(2 * (level - 1));
    for (size_t i = 0; i + 1 < level; ++i) {
      u64 q = h.primes[i].q;
      sw[3 * i] = nqi[i]; sw[3 * i + 1] = shoup(nqi[i], q); sw[3 * i + 2] = q - (ql % q);
      tl[2 * i] = qi[i];  tl[2 * i + 1] = shoup(qi[i], q);
    }
    RescaleDev r;
    r.sw = upload_vec(sw);
    r.tail = upload_vec(tl);
    return rescale.emplace(level, r).first->second;
  }

  void init_device() {
    HIP_OK(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    HIP_OK(hipEventCreate(&ev0));
    HIP_OK(hipEventCreate(&ev1));
    size_t T = h.L + h.K;
    std::vector<DevPrime> dp(T);
    for (size_t i = 0; i < T; ++i) {
      const PrimeInfo& p = h.primes[i];
      dp[i] = DevPrime{p.q, p.mu_lo, p.mu_hi, p.mu_sh, p.shift, 0, p.ninv, shoup(p.ninv, p.q)};
    }
    d.primes = upload_vec(dp);
    d.rou = upload_vec(h.rou);
    d.rou_p = upload_vec(h.rou_p);
    d.irou = upload_vec(h.irou);
    d.irou_p = upload_vec(h.irou_p);
    d.N = h.N;
    d.logN = h.logN;
    {
      // FP64 twiddles for the primes the FP64 NTT back end can take
      const char* force_int = std::getenv("ACE_NTT_FORCE_INT");
      bool use_fp = !(force_int && force_int[0] == '1') && h.logN > 12;
      std::vector<double> w(T * h.N, 0.0), iw(T * h.N, 0.0);
      for (size_t i = 0; i < T; ++i) {
        d.fp_ok[i] = (use_fp && h.primes[i].q < kFpPrimeLimit) ? 1 : 0;
        if (!d.fp_ok[i]) continue;
        for (size_t k = 0; k < h.N; ++k) {
          size_t o = i * h.N + k;
          w[o] = (double)h.rou[o];
          iw[o] = (double)h.irou[o];
        }
      }
      if (use_fp) {
        d.roud = upload_vec(w);
        d.iroud = upload_vec(iw);
      }
    }
    for (size_t i = 0; i < h.L && i < (size_t)kMaxPrimes; ++i) q_lm.prime[i] = (uint8_t)i;
    for (size_t j = 0; j < h.K; ++j) p_lm.prime[j] = (uint8_t)(h.L + j);
    // P -> Q tables, transposed to [K][L] so that targets are contiguous
    std::vector<u64> ph(h.K * h.L), sn(2 * h.K), scf(2 * h.K), pi(2 * h.L), pm(2 * h.L);
    for (size_t j = 0; j < h.K; ++j) {
      for (size_t i = 0; i < h.L; ++i) ph[j * h.L + i] = h.phat_modq[i * h.K + j];
      u64 q = h.primes[h.L + j].q;
      u64 a = mul_mod(h.primes[h.L + j].ninv, h.phat_inv[j], q);
      sn[2 * j] = a;               sn[2 * j + 1] = shoup(a, q);
      scf[2 * j] = h.phat_inv[j];  scf[2 * j + 1] = shoup(h.phat_inv[j], q);
    }
    for (size_t i = 0; i < h.L; ++i) {
      u64 q = h.primes[i].q;
      pi[2 * i] = h.pinv_modq[i]; pi[2 * i + 1] = shoup(h.pinv_modq[i], q);
      pm[2 * i] = h.pmodq[i];     pm[2 * i + 1] = shoup(h.pmodq[i], q);
    }
    phat = upload_vec(ph);
    pscale_ntt = upload_vec(sn);
    pscale_coef = upload_vec(scf);
    pinv = upload_vec(pi);
    pmodq = upload_vec(pm);
  }

  ~ace_ctx() {
    if (stream) (void)hipStreamSynchronize(stream);
    for (void* p : owned) (void)hipFree(p);
    if (ws) (void)hipFree(ws);
    if (ev0) (void)hipEventDestroy(ev0);
    if (ev1) (void)hipEventDestroy(ev1);
    if (stream) (void)hipStreamDestroy(stream);
  }
};

namespace {

inline u64* U(int64_t* p) { return reinterpret_cast<u64*>(p); }
inline const u64* U(const int64_t* p) { return reinterpret_cast<const u64*>(p); }

// limb map of a polynomial at `level`, optionally extended by the P limbs
LimbMap poly_lm(const ace_ctx* c, size_t level, bool with_p) {
  LimbMap lm{};
  for (size_t t = 0; t < level; ++t) lm.prime[t] = (uint8_t)t;
  if (with_p)
    for (size_t j = 0; j < c->h.K; ++j) lm.prime[level + j] = (uint8_t)(c->h.L + j);
  return lm;
}

bool level_ok(const ace_ctx* c, size_t level) { return level >= 1 && level <= c->h.L; }

// ---- internal sequencers: scratch comes from the arena, already sized ------

// Decomp_modup (rns_poly.c:160-258): copy the digit, INTT it scaled by the
// inverse cofactors, convert to the complement basis, NTT the new limbs.
void do_decomp_modup(ace_ctx* c, u64* res, const u64* src, size_t level, size_t part, bool is_ntt) {
  const ModUpDev& m = c->modup_at(level, part);
  const size_t N = c->h.N, nd = m.t.digit.size(), nc = m.t.compl_idx.size(), start = c->h.part_size * part;
  if (res + start * N != src + start * N)
    HIP_OK(hipMemcpyAsync(res + start * N, src + start * N, nd * N * sizeof(u64), hipMemcpyDeviceToDevice, c->stream));
  size_t mark = c->ws_used;
  u64* t = c->take(nd * N);
  if (is_ntt) launch_ntt(c->stream, c->d, t, src + start * N, m.digit_lm, nullptr, (u32)nd, 1, 0, true, m.scale_ntt);
  else        launch_mul_const(c->stream, c->d, t, src + start * N, m.scale_coef, m.digit_lm, (u32)nd);
  launch_baseconv(c->stream, c->d, res, t, m.hat, (u32)nc, (u32)nd, (u32)nc, m.conv);
  if (is_ntt) launch_ntt(c->stream, c->d, res, res, m.compl_lm, &m.compl_pos, (u32)nc, 1, 0, false, nullptr);
  c->ws_used = mark;
}

// Mod_down (rns_poly.c:260-308); addend (optional) is added to the result
void do_mod_down(ace_ctx* c, u64* res, const u64* src, size_t level, bool is_ntt, const u64* addend) {
  const size_t N = c->h.N, K = c->h.K, L = c->h.L;
  size_t mark = c->ws_used;
  u64* t = c->take(K * N);
  u64* y = c->take(level * N);
  if (is_ntt) launch_ntt(c->stream, c->d, t, src + level * N, c->p_lm, nullptr, (u32)K, 1, 0, true, c->pscale_ntt);
  else        launch_mul_const(c->stream, c->d, t, src + level * N, c->pscale_coef, c->p_lm, (u32)K);
  ConvMap cm{};
  for (size_t i = 0; i < level; ++i) { cm.prime[i] = (uint8_t)i; cm.out_limb[i] = (uint8_t)i; }
  launch_baseconv(c->stream, c->d, y, t, c->phat, (u32)L, (u32)K, (u32)level, cm);
  if (is_ntt) launch_ntt(c->stream, c->d, y, y, c->q_lm, nullptr, (u32)level, 1, 0, false, nullptr);
  launch_moddown_tail(c->stream, c->d, res, src, y, addend, c->pinv, c->q_lm, (u32)level);
  c->ws_used = mark;
}

// Rescale (rns_poly.c:310-404)
void do_rescale(ace_ctx* c, u64* res, const u64* src, size_t level, bool is_ntt) {
  const size_t N = c->h.N;
  const RescaleDev& r = c->rescale_at(level);
  if (!is_ntt) {
    launch_rescale_coef(c->stream, c->d, res, src, src + (level - 1) * N, r.tail, c->q_lm, (u32)(level - 1));
    return;
  }
  size_t mark = c->ws_used;
  u64* last = c->take(N);
  u64* u = c->take((level - 1) * N);
  LimbMap one{};
  one.prime[0] = (uint8_t)(level - 1);
  launch_ntt(c->stream, c->d, last, src + (level - 1) * N, one, nullptr, 1, 1, 0, true, nullptr);
  launch_rescale_switch(c->stream, c->d, u, last, (u32)(level - 1), r.sw, c->q_lm, (u32)(level - 1));
  launch_ntt(c->stream, c->d, u, u, c->q_lm, nullptr, (u32)(level - 1), 1, 0, false, nullptr);
  launch_rescale_tail(c->stream, c->d, res, src, u, r.tail, c->q_lm, (u32)(level - 1));
  c->ws_used = mark;
}

void do_precomp(ace_ctx* c, u64* res, const u64* src, size_t level, bool is_ntt) {
  size_t nd = c->h.num_decomp(level), stride = (level + c->h.K) * (size_t)c->h.N;
  for (size_t part = 0; part < nd; ++part) do_decomp_modup(c, res + part * stride, src, level, part, is_ntt);
}

// key limb positions of a polynomial viewed at `level` (Derive_poly, rns_poly.c:701-707)
LimbMap key_pos(const ace_ctx* c, size_t level) {
  LimbMap kp{};
  for (size_t t = 0; t < level; ++t) kp.prime[t] = (uint8_t)t;
  for (size_t j = 0; j < c->h.K; ++j) kp.prime[level + j] = (uint8_t)(c->h.L + j);
  return kp;
}

// Fast_switch_key (evaluator.c:411-462); add0/add1 are fused into the Mod_down tails
void do_switch_key(ace_ctx* c, u64* out0, u64* out1, const u64* digits, const u64* swk, size_t level,
                   const u64* add0, const u64* add1) {
  const size_t N = c->h.N, T = level + c->h.K, kpoly = (c->h.L + c->h.K) * N, nd = c->h.num_decomp(level);
  size_t mark = c->ws_used;
  u64* e0 = c->take(T * N);
  u64* e1 = c->take(T * N);
  LimbMap lm = poly_lm(c, level, true), kp = key_pos(c, level);
  launch_dotprod(c->stream, c->d, e0, e1, digits, T * N, swk, swk + kpoly, 2 * kpoly, (u32)nd, lm, kp, (u32)T);
  do_mod_down(c, out0, e0, level, true, add0);
  do_mod_down(c, out1, e1, level, true, add1);
  c->ws_used = mark;
}

}  // namespace

// ===========================================================================
extern "C" {

#define ACE_TRY try {                                                          \
  if (!c) return fail("null context");                                         \
  if (!c->device_ok) return fail("no HIP device: this context holds host tables only");
#define ACE_CATCH_INT                      \
  }                                        \
  catch (const std::exception& e) {        \
    return fail(e.what());                 \
  }                                        \
  return 0;

const char* ace_last_error(void) { return g_err.c_str(); }

static ace_ctx* make_ctx(uint32_t degree, const std::vector<i64>& q, size_t parts) {
  try {
    std::unique_ptr<ace_ctx> c(new ace_ctx());
    c->h.build(degree, q, parts);
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) == hipSuccess && ndev > 0) {
      c->init_device();
      c->device_ok = true;
    }
    return c.release();
  } catch (const std::exception& e) {
    g_err = e.what();
    return nullptr;
  }
}

ace_ctx* ace_ctx_create(uint32_t degree, size_t num_q, size_t q0_bits, size_t sf_bits, size_t num_parts) {
  if (degree < 2 || (degree & (degree - 1)) || num_q == 0 || q0_bits > 61 || sf_bits > 61 || q0_bits < 2 ||
      sf_bits < 2 || num_parts == 0) {
    g_err = "ace_ctx_create: invalid parameters";
    return nullptr;
  }
  std::vector<i64> q;
  try {
    q = generate_q_primes(degree, num_q, q0_bits, sf_bits);
  } catch (const std::exception& e) {
    g_err = e.what();
    return nullptr;
  }
  return make_ctx(degree, q, num_parts);
}

ace_ctx* ace_ctx_create_with_primes(uint32_t degree, size_t num_q, const int64_t* q_primes, size_t num_parts) {
  if (!q_primes || num_q == 0 || num_parts == 0) {
    g_err = "ace_ctx_create_with_primes: invalid parameters";
    return nullptr;
  }
  return make_ctx(degree, std::vector<i64>(q_primes, q_primes + num_q), num_parts);
}

void ace_ctx_destroy(ace_ctx* ctx) { delete ctx; }

uint32_t ace_degree(const ace_ctx* c) { return c->h.N; }
size_t ace_num_q(const ace_ctx* c) { return c->h.L; }
size_t ace_num_p(const ace_ctx* c) { return c->h.K; }
size_t ace_num_parts(const ace_ctx* c) { return c->h.parts; }
size_t ace_part_size(const ace_ctx* c) { return c->h.part_size; }
size_t ace_num_decomp(const ace_ctx* c, size_t level) { return c->h.num_decomp(level); }
int64_t ace_prime(const ace_ctx* c, size_t i) { return i < c->h.primes.size() ? (int64_t)c->h.primes[i].q : 0; }
int64_t ace_root(const ace_ctx* c, size_t i) { return i < c->h.primes.size() ? (int64_t)c->h.primes[i].root : 0; }
void ace_modulus(const ace_ctx* c, size_t i, uint64_t out[5]) {
  const PrimeInfo& p = c->h.primes[i];
  out[0] = p.q; out[1] = (u64)p.br_k; out[2] = (u64)p.br_m; out[3] = p.mu_lo; out[4] = p.mu_hi;
}

// ---- memory -----------------------------------------------------------------
int64_t* ace_alloc(ace_ctx* c, size_t n_words) {
  try {
    if (!c || !c->device_ok) throw std::runtime_error("no HIP device: this context holds host tables only");
    u64* p = nullptr;
    HIP_OK(hipMalloc((void**)&p, std::max<size_t>(n_words, 1) * sizeof(u64)));
    launch_fill_zero(c->stream, p, n_words);
    return reinterpret_cast<int64_t*>(p);
  } catch (const std::exception& e) {
    g_err = e.what();
    return nullptr;
  }
}
void ace_free(ace_ctx* c, int64_t* p) {
  if (!p || !c || !c->device_ok) return;
  (void)hipStreamSynchronize(c->stream);
  (void)hipFree(p);
}
int ace_upload(ace_ctx* c, int64_t* dst, const int64_t* src, size_t n) {
  ACE_TRY
  HIP_OK(hipMemcpyAsync(dst, src, n * sizeof(u64), hipMemcpyHostToDevice, c->stream));
  HIP_OK(hipStreamSynchronize(c->stream));
  ACE_CATCH_INT
}
int ace_download(ace_ctx* c, int64_t* dst, const int64_t* src, size_t n) {
  ACE_TRY
  HIP_OK(hipMemcpyAsync(dst, src, n * sizeof(u64), hipMemcpyDeviceToHost, c->stream));
  HIP_OK(hipStreamSynchronize(c->stream));
  ACE_CATCH_INT
}
int ace_copy(ace_ctx* c, int64_t* dst, const int64_t* src, size_t n) {
  ACE_TRY
  if (dst != src) HIP_OK(hipMemcpyAsync(dst, src, n * sizeof(u64), hipMemcpyDeviceToDevice, c->stream));
  ACE_CATCH_INT
}
int ace_zero(ace_ctx* c, int64_t* dst, size_t n) {
  ACE_TRY
  launch_fill_zero(c->stream, U(dst), n);
  ACE_CATCH_INT
}
int ace_sync(ace_ctx* c) {
  ACE_TRY
  HIP_OK(hipStreamSynchronize(c->stream));
  ACE_CATCH_INT
}
int ace_timer_start(ace_ctx* c) {
  ACE_TRY
  HIP_OK(hipEventRecord(c->ev0, c->stream));
  ACE_CATCH_INT
}
float ace_timer_stop_ms(ace_ctx* c) {
  try {
    if (!c || !c->device_ok) throw std::runtime_error("no HIP device");
    HIP_OK(hipEventRecord(c->ev1, c->stream));
    HIP_OK(hipEventSynchronize(c->ev1));
    float ms = 0;
    HIP_OK(hipEventElapsedTime(&ms, c->ev0, c->ev1));
    return ms;
  } catch (const std::exception& e) {
    g_err = e.what();
    return -1.0f;
  }
}

// ---- NTT ---------------------------------------------------------------------
static int ntt_common(ace_ctx* c, int64_t* dst, const int64_t* src, const int32_t* prime_idx, size_t n_limbs,
                      size_t n_polys, size_t stride_limbs, bool inverse, int passes = 3) {
  ACE_TRY
  if (n_limbs == 0 || n_polys == 0) return 0;
  if (!dst || !src || !prime_idx) return fail("ace_ntt: null argument");
  if (n_limbs > (size_t)kMaxPrimes) return fail("ace_ntt: more than 96 limbs per polynomial");
  if (n_polys > 65535) return fail("ace_ntt: more than 65535 polynomials per call");
  if (n_polys > 1 && stride_limbs < n_limbs) return fail("ace_ntt: polynomial stride smaller than limb count");
  LimbMap lm{};
  for (size_t t = 0; t < n_limbs; ++t) {
    if (prime_idx[t] < 0 || (size_t)prime_idx[t] >= c->h.L + c->h.K) return fail("ace_ntt: prime index out of range");
    lm.prime[t] = (uint8_t)prime_idx[t];
  }
  if (!launch_ntt(c->stream, c->d, U(dst), U(src), lm, nullptr, (u32)n_limbs, (u32)n_polys,
                  (u64)stride_limbs * c->h.N, inverse, nullptr, passes))
    return fail("ace_ntt: ring degree not supported");
  ACE_CATCH_INT
}
int ace_ntt(ace_ctx* c, int64_t* dst, const int64_t* src, const int32_t* prime_idx, size_t n_limbs, size_t n_polys,
            size_t stride) {
  return ntt_common(c, dst, src, prime_idx, n_limbs, n_polys, stride, false);
}
int ace_intt(ace_ctx* c, int64_t* dst, const int64_t* src, const int32_t* prime_idx, size_t n_limbs, size_t n_polys,
             size_t stride) {
  return ntt_common(c, dst, src, prime_idx, n_limbs, n_polys, stride, true);
}

int ace_ntt_pass(ace_ctx* c, int64_t* dst, const int64_t* src, const int32_t* prime_idx, size_t n_limbs,
                 size_t n_polys, size_t stride, int inverse, int pass) {
  if (pass != 1 && pass != 2) return fail("ace_ntt_pass: pass must be 1 or 2");
  if (c && c->h.logN <= 12) return fail("ace_ntt_pass: ring degrees up to 4096 are a single kernel");
  return ntt_common(c, dst, src, prime_idx, n_limbs, n_polys, stride, inverse != 0, pass);
}

// ---- Hw_* ---------------------------------------------------------------------
static int hw_common(ace_ctx* c, EwOp op, int64_t* r, const int64_t* a, const int64_t* b, int64_t s, size_t pi,
                     size_t n) {
  ACE_TRY
  if (n == 0) return 0;
  if (!r || !a || (op < EW_ADD_S && !b)) return fail("ace_hw: null argument");
  if (pi >= c->h.L + c->h.K) return fail("ace_hw: prime index out of range");
  if ((op == EW_MUL_S || op == EW_MULADD_S) && (s < 0 || (u64)s >= c->h.primes[pi].q))
    return fail("ace_hw: scalar multiplier must be a residue in [0, q)");
  LimbMap lm{};
  lm.prime[0] = (uint8_t)pi;
  launch_ew(c->stream, c->d, op, U(r), U(a), U(b), (u64)s, lm, 1, n);
  ACE_CATCH_INT
}
int ace_hw_modadd(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t pi, size_t n) { return hw_common(c, EW_ADD, r, a, b, 0, pi, n); }
int ace_hw_modsub(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t pi, size_t n) { return hw_common(c, EW_SUB, r, a, b, 0, pi, n); }
int ace_hw_modmul(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t pi, size_t n) { return hw_common(c, EW_MUL, r, a, b, 0, pi, n); }
int ace_hw_modmuladd(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t pi, size_t n) { return hw_common(c, EW_MULADD, r, a, b, 0, pi, n); }
int ace_hw_modadd_scalar(ace_ctx* c, int64_t* r, const int64_t* a, int64_t s, size_t pi, size_t n) { return hw_common(c, EW_ADD_S, r, a, nullptr, s, pi, n); }
int ace_hw_modsub_scalar(ace_ctx* c, int64_t* r, const int64_t* a, int64_t s, size_t pi, size_t n) { return hw_common(c, EW_SUB_S, r, a, nullptr, s, pi, n); }
int ace_hw_modmul_scalar(ace_ctx* c, int64_t* r, const int64_t* a, int64_t s, size_t pi, size_t n) { return hw_common(c, EW_MUL_S, r, a, nullptr, s, pi, n); }
int ace_hw_modmuladd_scalar(ace_ctx* c, int64_t* r, const int64_t* a, int64_t s, size_t pi, size_t n) { return hw_common(c, EW_MULADD_S, r, a, nullptr, s, pi, n); }

int ace_hw_rotate(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* order, size_t pi, size_t n) {
  ACE_TRY
  if (n == 0) return 0;
  if (!r || !a || !order) return fail("ace_hw_rotate: null argument");
  if (r == a) return fail("ace_hw_rotate: in-place gather is not supported");
  if (pi >= c->h.L + c->h.K) return fail("ace_hw_rotate: prime index out of range");
  LimbMap lm{};
  lm.prime[0] = (uint8_t)pi;
  launch_gather(c->stream, c->d, U(r), U(a), order, lm, 1, n);
  ACE_CATCH_INT
}

// ---- automorphism tables --------------------------------------------------------
uint32_t ace_find_automorphism_index(const ace_ctx* c, int32_t rot_idx) {
  return find_automorphism_index(rot_idx, c->h.N);
}
int ace_host_automorphism_order(const ace_ctx* c, int64_t* host_order, uint32_t k, int is_ntt) {
  if (!c || !host_order) return fail("ace_host_automorphism_order: null argument");
  if (!(k & 1) || k >= 2 * c->h.N) return fail("ace_host_automorphism_order: index must be odd and below 2N");
  automorphism_order(host_order, k, c->h.N, is_ntt != 0);
  return 0;
}

int ace_has_device(const ace_ctx* c) { return c && c->device_ok ? 1 : 0; }

// host copies of the tables, for inspection and parity tests
int ace_host_twiddles(const ace_ctx* c, size_t prime_idx, int which, uint64_t* out) {
  if (!c || !out || prime_idx >= c->h.L + c->h.K || which < 0 || which > 3) return fail("ace_host_twiddles: bad argument");
  const std::vector<u64>* t[4] = {&c->h.rou, &c->h.rou_p, &c->h.irou, &c->h.irou_p};
  std::memcpy(out, t[which]->data() + prime_idx * c->h.N, c->h.N * sizeof(u64));
  return 0;
}
int ace_host_tbl_modup(const ace_ctx* c, size_t level, size_t part, int64_t* hat_inv, int64_t* hat,
                       int32_t* compl_idx, size_t* n_digit, size_t* n_compl) {
  try {
    if (!c || !hat_inv || !hat || !compl_idx || !n_digit || !n_compl) return fail("ace_host_tbl_modup: null argument");
    if (!level_ok(c, level)) return fail("ace_host_tbl_modup: level out of range");
    ModUpTable t = c->h.modup_table(level, part);
    *n_digit = t.digit.size();
    *n_compl = t.compl_idx.size();
    for (size_t i = 0; i < t.hat_inv.size(); ++i) hat_inv[i] = (int64_t)t.hat_inv[i];
    for (size_t i = 0; i < t.hat.size(); ++i) hat[i] = (int64_t)t.hat[i];
    for (size_t j = 0; j < t.compl_idx.size(); ++j) compl_idx[j] = t.compl_idx[j];
  } catch (const std::exception& e) {
    return fail(e.what());
  }
  return 0;
}
int ace_host_tbl_moddown(const ace_ctx* c, int64_t* phat_inv, int64_t* phat_modq, int64_t* pinv_modq, int64_t* pmodq) {
  if (!c || !phat_inv || !phat_modq || !pinv_modq || !pmodq) return fail("ace_host_tbl_moddown: null argument");
  for (size_t j = 0; j < c->h.K; ++j) phat_inv[j] = (int64_t)c->h.phat_inv[j];
  for (size_t i = 0; i < c->h.L * c->h.K; ++i) phat_modq[i] = (int64_t)c->h.phat_modq[i];
  for (size_t i = 0; i < c->h.L; ++i) { pinv_modq[i] = (int64_t)c->h.pinv_modq[i]; pmodq[i] = (int64_t)c->h.pmodq[i]; }
  return 0;
}
int ace_host_tbl_rescale(const ace_ctx* c, size_t level, int64_t* ql_inv, int64_t* neg_ql_inv) {
  if (!c || !ql_inv || !neg_ql_inv) return fail("ace_host_tbl_rescale: null argument");
  if (level < 2 || level > c->h.L) return fail("ace_host_tbl_rescale: level out of range");
  std::vector<u64> a, b;
  c->h.rescale_table(level, a, b);
  for (size_t i = 0; i + 1 < level; ++i) { ql_inv[i] = (int64_t)a[i]; neg_ql_inv[i] = (int64_t)b[i]; }
  return 0;
}

int ace_automorphism_order(ace_ctx* c, int64_t* dev_order, uint32_t k, int is_ntt) {
  ACE_TRY
  if (!dev_order) return fail("ace_automorphism_order: null argument");
  if (!(k & 1) || k >= 2 * c->h.N) return fail("ace_automorphism_order: index must be odd and below 2N");
  std::vector<i64> ord(c->h.N);
  automorphism_order(ord.data(), k, c->h.N, is_ntt != 0);
  HIP_OK(hipMemcpyAsync(dev_order, ord.data(), ord.size() * sizeof(i64), hipMemcpyHostToDevice, c->stream));
  HIP_OK(hipStreamSynchronize(c->stream));
  ACE_CATCH_INT
}

// ---- polynomial ops ---------------------------------------------------------------
static int poly_ew(ace_ctx* c, EwOp op, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p) {
  ACE_TRY
  if (!r || !a || !b) return fail("ace_poly: null argument");
  if (!level_ok(c, level)) return fail("ace_poly: level out of range");
  LimbMap lm = poly_lm(c, level, with_p != 0);
  launch_ew(c->stream, c->d, op, U(r), U(a), U(b), 0, lm, (u32)(level + (with_p ? c->h.K : 0)), c->h.N);
  ACE_CATCH_INT
}
int ace_poly_add(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p) { return poly_ew(c, EW_ADD, r, a, b, level, with_p); }
int ace_poly_sub(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p) { return poly_ew(c, EW_SUB, r, a, b, level, with_p); }
int ace_poly_mul(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p) { return poly_ew(c, EW_MUL, r, a, b, level, with_p); }

int ace_poly_automorphism(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* order, size_t level, int with_p) {
  ACE_TRY
  if (!r || !a || !order) return fail("ace_poly_automorphism: null argument");
  if (r == a) return fail("ace_poly_automorphism: in-place gather is not supported");
  if (!level_ok(c, level)) return fail("ace_poly_automorphism: level out of range");
  LimbMap lm = poly_lm(c, level, with_p != 0);
  launch_gather(c->stream, c->d, U(r), U(a), order, lm, (u32)(level + (with_p ? c->h.K : 0)), c->h.N);
  ACE_CATCH_INT
}

int ace_decomp_modup(ace_ctx* c, int64_t* res, const int64_t* src, size_t level, size_t part, int is_ntt) {
  ACE_TRY
  if (!res || !src) return fail("ace_decomp_modup: null argument");
  if (!level_ok(c, level)) return fail("ace_decomp_modup: level out of range");
  if (part >= c->h.num_decomp(level)) return fail("ace_decomp_modup: digit index out of range");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_decomp_modup(c, U(res), U(src), level, part, is_ntt != 0);
  ACE_CATCH_INT
}

int ace_precomp(ace_ctx* c, int64_t* res, const int64_t* src, size_t level, int is_ntt) {
  ACE_TRY
  if (!res || !src) return fail("ace_precomp: null argument");
  if (!level_ok(c, level)) return fail("ace_precomp: level out of range");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_precomp(c, U(res), U(src), level, is_ntt != 0);
  ACE_CATCH_INT
}

int ace_mod_down(ace_ctx* c, int64_t* res, const int64_t* src, size_t level, int is_ntt) {
  ACE_TRY
  if (!res || !src) return fail("ace_mod_down: null argument");
  if (!level_ok(c, level)) return fail("ace_mod_down: level out of range");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_mod_down(c, U(res), U(src), level, is_ntt != 0, nullptr);
  ACE_CATCH_INT
}

int ace_rescale(ace_ctx* c, int64_t* res, const int64_t* src, size_t level, int is_ntt) {
  ACE_TRY
  if (!res || !src) return fail("ace_rescale: null argument");
  if (level < 2 || level > c->h.L) return fail("Level of rescale opnd is too small");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_rescale(c, U(res), U(src), level, is_ntt != 0);
  ACE_CATCH_INT
}

int ace_extend(ace_ctx* c, int64_t* res, const int64_t* src, size_t level) {
  ACE_TRY
  if (!res || !src) return fail("ace_extend: null argument");
  if (!level_ok(c, level)) return fail("ace_extend: level out of range");
  launch_mul_const(c->stream, c->d, U(res), U(src), c->pmodq, c->q_lm, (u32)level);
  launch_fill_zero(c->stream, U(res) + level * (size_t)c->h.N, c->h.K * (size_t)c->h.N);
  ACE_CATCH_INT
}

int ace_dot_prod(ace_ctx* c, int64_t* res, const int64_t* digits, const int64_t* key, size_t key_stride,
                 size_t n_parts, size_t level) {
  ACE_TRY
  if (!res || !digits || !key) return fail("ace_dot_prod: null argument");
  if (!level_ok(c, level)) return fail("ace_dot_prod: level out of range");
  if (n_parts == 0 || n_parts > c->h.parts) return fail("ace_dot_prod: number of digits out of range");
  size_t T = level + c->h.K;
  LimbMap lm = poly_lm(c, level, true), kp = key_pos(c, level);
  launch_dotprod(c->stream, c->d, U(res), nullptr, U(digits), T * (size_t)c->h.N, U(key), nullptr, key_stride,
                 (u32)n_parts, lm, kp, (u32)T);
  ACE_CATCH_INT
}

// ---- ciphertext level ------------------------------------------------------------
int ace_mul_ciph3(ace_ctx* c, int64_t* d0, int64_t* d1, int64_t* d2, const int64_t* a0, const int64_t* a1,
                  const int64_t* b0, const int64_t* b1, size_t level) {
  ACE_TRY
  if (!d0 || !d1 || !d2 || !a0 || !a1 || !b0 || !b1) return fail("ace_mul_ciph3: null argument");
  if (!level_ok(c, level)) return fail("ace_mul_ciph3: level out of range");
  launch_tensor(c->stream, c->d, U(d0), U(d1), U(d2), U(a0), U(a1), U(b0), U(b1), c->q_lm, (u32)level);
  ACE_CATCH_INT
}

int ace_fast_switch_key(ace_ctx* c, int64_t* out0, int64_t* out1, const int64_t* digits, const int64_t* swk,
                        size_t level) {
  ACE_TRY
  if (!out0 || !out1 || !digits || !swk) return fail("ace_fast_switch_key: null argument");
  if (!level_ok(c, level)) return fail("ace_fast_switch_key: level out of range");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_switch_key(c, U(out0), U(out1), U(digits), U(swk), level, nullptr, nullptr);
  ACE_CATCH_INT
}

int ace_relin(ace_ctx* c, int64_t* r0, int64_t* r1, const int64_t* d0, const int64_t* d1, const int64_t* d2,
              const int64_t* swk, size_t level) {
  ACE_TRY
  if (!r0 || !r1 || !d0 || !d1 || !d2 || !swk) return fail("ace_relin: null argument");
  if (!level_ok(c, level)) return fail("ace_relin: level out of range");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  size_t nd = c->h.num_decomp(level), T = level + c->h.K;
  u64* digits = c->take(nd * T * c->h.N);
  do_precomp(c, digits, U(d2), level, true);
  do_switch_key(c, U(r0), U(r1), digits, U(swk), level, U(d0), U(d1));
  ACE_CATCH_INT
}

int ace_rescale_ciph(ace_ctx* c, int64_t* r0, int64_t* r1, const int64_t* c0, const int64_t* c1, size_t level) {
  ACE_TRY
  if (!r0 || !r1 || !c0 || !c1) return fail("ace_rescale_ciph: null argument");
  if (level < 2 || level > c->h.L) return fail("Level of rescale opnd is too small");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_rescale(c, U(r0), U(c0), level, true);
  do_rescale(c, U(r1), U(c1), level, true);
  ACE_CATCH_INT
}

int ace_mul_relin_rescale(ace_ctx* c, int64_t* r0, int64_t* r1, const int64_t* a0, const int64_t* a1,
                          const int64_t* b0, const int64_t* b1, const int64_t* swk, size_t level) {
  ACE_TRY
  if (!r0 || !r1 || !a0 || !a1 || !b0 || !b1 || !swk) return fail("ace_mul_relin_rescale: null argument");
  if (level < 2 || level > c->h.L) return fail("ace_mul_relin_rescale: level out of range");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  const size_t N = c->h.N, nd = c->h.num_decomp(level), T = level + c->h.K;
  u64* d0 = c->take(level * N);
  u64* d1 = c->take(level * N);
  u64* d2 = c->take(level * N);
  u64* digits = c->take(nd * T * N);
  launch_tensor(c->stream, c->d, d0, d1, d2, U(a0), U(a1), U(b0), U(b1), c->q_lm, (u32)level);
  do_precomp(c, digits, d2, level, true);
  do_switch_key(c, d0, d1, digits, U(swk), level, d0, d1);  // relinearised ciphertext replaces d0, d1
  do_rescale(c, U(r0), d0, level, true);
  do_rescale(c, U(r1), d1, level, true);
  ACE_CATCH_INT
}

static void do_fast_rotate(ace_ctx* c, u64* r0, u64* r1, const u64* c0, const u64* digits, const u64* swk,
                           const i64* order, size_t level) {
  const size_t N = c->h.N;
  size_t mark = c->ws_used;
  u64* t0 = c->take(level * N);
  u64* t1 = c->take(level * N);
  do_switch_key(c, t0, t1, digits, swk, level, c0, nullptr);
  launch_gather2(c->stream, c->d, r0, r1, t0, t1, order, c->q_lm, (u32)level, N);
  c->ws_used = mark;
}

int ace_fast_rotate(ace_ctx* c, int64_t* r0, int64_t* r1, const int64_t* c0, const int64_t* digits,
                    const int64_t* swk, const int64_t* order, size_t level) {
  ACE_TRY
  if (!r0 || !r1 || !c0 || !digits || !swk || !order) return fail("ace_fast_rotate: null argument");
  if (!level_ok(c, level)) return fail("ace_fast_rotate: level out of range");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_fast_rotate(c, U(r0), U(r1), U(c0), U(digits), U(swk), order, level);
  ACE_CATCH_INT
}

int ace_rotate_batch(ace_ctx* c, int64_t* r0s, int64_t* r1s, const int64_t* c0, const int64_t* c1,
                     const int64_t* const* swks, const int64_t* const* orders, size_t count, size_t level) {
  ACE_TRY
  if (count == 0) return 0;
  if (!r0s || !r1s || !c0 || !c1 || !swks || !orders) return fail("ace_rotate_batch: null argument");
  if (!level_ok(c, level)) return fail("ace_rotate_batch: level out of range");
  for (size_t i = 0; i < count; ++i)
    if (!swks[i] || !orders[i]) return fail("ace_rotate_batch: null key or order table");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  const size_t N = c->h.N, nd = c->h.num_decomp(level), T = level + c->h.K;
  u64* digits = c->take(nd * T * N);
  do_precomp(c, digits, U(c1), level, true);
  for (size_t i = 0; i < count; ++i)
    do_fast_rotate(c, U(r0s) + i * level * N, U(r1s) + i * level * N, U(c0), digits, U(swks[i]), orders[i], level);
  ACE_CATCH_INT
}

}  // extern "C"
