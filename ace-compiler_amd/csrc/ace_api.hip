// C-ABI of the MI355X CKKS polynomial runtime (include/ace_hip.h): context
// life cycle, device memory, and the host-side sequencing of kernels for each
// reference operation.  One HIP stream per context; every call only enqueues.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <map>
#include <set>
#include <unordered_set>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <tuple>
#include <unordered_map>
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
  ConvJob job{};  // the digit's conversion, offsets zero
};

// all digits of a level at once (Precomp)
struct PrecompDev {
  u64* scale_ntt = nullptr;   // [level][2]: 1/N * hat_inv of the limb's own digit
  u64* scale_coef = nullptr;  // [level][2]
  std::vector<ConvJob> jobs;  // one per digit; t_off / out_off filled for one operand
  LimbMap tgt_lm{}, tgt_pos{};  // every converted limb of every digit: prime, position in the digits block
  u32 n_tgt = 0;
  bool one_ntt_launch = false;  // positions fit a byte and n_tgt <= kMaxPrimes
};

struct RescaleDev {
  u64* sw = nullptr;    // [level-1][3]: K, K', diff
  u64* tail = nullptr;  // [level-1][2]: q_l^-1, Shoup
};

// Constants of a Mod_down and a Rescale that share one forward transform (do_switch_key_rescale)
struct ModDownRescaleDev {
  u64* inv_scale = nullptr;  // [1 + K][2]: (1/N * P^-1 mod q_last) for the dropped limb, then the P limbs' Mod_down scales
  u64* tail = nullptr;       // [level-1][2]: (P q_last)^-1 mod q_t
  LimbMap inv_lm{};          // the dropped limb, then the P limbs
  std::vector<u64> ql_inv;   // host copy: q_last^-1 mod q_t, t < level - 1
  // P -> Q conversion onto the level's limbs with a constant folded into each target's column of the matrix:
  // -(P q_last)^-1 mod q_t for t < level - 1, P^-1 mod q_last for the dropped limb
  ConvJob job{};
};

// Scratch of ace_mod_down_noalloc: the intermediates of one Mod_down (the scaled inverse transform of the P limbs
// and their conversion to the Q basis), held in a device array that exists from the moment the library is loaded.
// Each GPU has its own copy at its own address; host code reaches it only through the pointer that
// hipGetSymbolAddress returned for that GPU (static_scratch_of).
constexpr size_t kStaticScratchWords = (size_t)1 << 21;  // 16 MiB
static __device__ __align__(256) __attribute__((used)) unsigned long long scratch[kStaticScratchWords];
constexpr int kMaxDevices = 64;
u64* g_static_scratch[kMaxDevices] = {nullptr};

// the address of `scratch` on the current device, looked up once per device
u64* static_scratch_of_current_device() {
  int dev = -1;
  HIP_OK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) throw std::runtime_error("device ordinal out of range");
  if (!g_static_scratch[dev]) {
    void* ptr = nullptr;
    HIP_OK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) throw std::runtime_error("hipGetSymbolAddress returned no address for the static scratch");
    g_static_scratch[dev] = static_cast<u64*>(ptr);
  }
  return g_static_scratch[dev];
}

}  // namespace

// Hw_* calls recorded for one launch (see flush_run)
struct PendingRun {
  std::vector<BatchOp> ops;
  u64 n = 0;                                  // words per operand, the same for the whole run
  std::set<uintptr_t> touched;                // start of every operand and result of the run
  std::unordered_set<uintptr_t> written;      // starts written by elementwise entries
  std::unordered_set<uintptr_t> rot_res, rot_src;  // results / sources (and index tables) of rotates
};

// What the contexts of one family share (a context made by ace_ctx_create and those made from it by ace_ctx_share):
// the host tables, and the record of the buffers ace_alloc has handed out, so that a buffer may be freed through
// another context of the family than the one that made it.
struct Family {
  HostContext h;
  std::mutex mu;  // guards `live` and `order_fits`
  std::unordered_map<void*, size_t> live;
  std::atomic<size_t> pooled_words{0};  // freed buffers kept for reuse by all contexts of the family together
  size_t pool_limit_words = (size_t)4 << 30;  // at most this much of it: a third of the GPU's memory, or ACE_POOL_LIMIT_GB (set by the root)
  // Index tables of rotations seen so far -> whether the forward chunk pass may apply them on the way out (every
  // 4096-word block of the table draws on one block of the source, and the blocks' sources are a permutation:
  // true of Precompute_automorphism_order's NTT-form tables, number_theory.c:211-222).  Tables made by
  // ace_automorphism_order are entered as they are made, a caller's own table is examined on the device when a
  // rotation first uses it; writing to a table through this library (upload, copy, zero, free) forgets the verdict.
  std::map<uintptr_t, bool> order_fits;  // by address: forgetting the tables a write overlaps is a range query
};

struct ace_ctx {
  std::shared_ptr<Family> family;
  HostContext& h;
  std::unordered_map<void*, size_t>& live;  // sizes of the buffers handed out (guarded by family->mu)
  ace_ctx* parent = nullptr;  // the context whose device tables this one uses (null: its own)
  ace_ctx() : family(std::make_shared<Family>()), h(family->h), live(family->live) {}
  explicit ace_ctx(ace_ctx* from) : family(from->family), h(family->h), live(family->live), parent(from) {}
  bool device_ok = false;  // false: host tables only (no GPU present), every compute call is rejected
  hipStream_t stream = nullptr;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  DevCtx d{};
  std::vector<void*> owned;  // device allocations freed with the context
  // host-to-device copies of small host arrays whose lifetime ends with the call: staged through pinned
  // buffers that are reused only after the copy out of them has finished
  struct Stage {
    void* host = nullptr;
    size_t cap = 0;
    hipEvent_t done = nullptr;
    bool pending = false;
  };
  static constexpr int kStages = 256;
  Stage stages[kStages];
  int next_stage = 0;
  static constexpr int kGatherStages = 8;
  Stage gather_stages[kGatherStages];
  int next_gather = 0;
  void h2d(void* dev_dst, const void* src, size_t bytes) {
    if (!bytes) return;
    Stage& st = stages[next_stage];
    next_stage = (next_stage + 1) % kStages;
    if (st.pending) {
      HIP_OK(hipEventSynchronize(st.done));
      st.pending = false;
    }
    if (st.cap < bytes) {
      if (st.host) HIP_OK(hipHostFree(st.host));
      st.host = nullptr;
      st.cap = std::max<size_t>(bytes, 64 * 1024);
      HIP_OK(hipHostMalloc(&st.host, st.cap, hipHostMallocDefault));
    }
    if (!st.done) HIP_OK(hipEventCreateWithFlags(&st.done, hipEventDisableTiming));
    std::memcpy(st.host, src, bytes);
    HIP_OK(hipMemcpyAsync(dev_dst, st.host, bytes, hipMemcpyHostToDevice, stream));
    HIP_OK(hipEventRecord(st.done, stream));
    st.pending = true;
  }
  // n host arrays of `bytes` each to consecutive places of the device: one staging block, one copy
  void h2d_gather(void* dev_dst, const void* const* srcs, size_t n, size_t bytes) {
    if (!bytes || !n) return;
    if (n == 1) return h2d(dev_dst, srcs[0], bytes);
    // (blocks of their own: the ring above keeps many small blocks, and pinned memory is slow to allocate)
    Stage& st = gather_stages[next_gather];
    next_gather = (next_gather + 1) % kGatherStages;
    if (st.pending) {
      HIP_OK(hipEventSynchronize(st.done));
      st.pending = false;
    }
    if (st.cap < n * bytes) {
      if (st.host) HIP_OK(hipHostFree(st.host));
      st.host = nullptr;
      st.cap = std::max<size_t>(n * bytes, 64 * 1024);
      HIP_OK(hipHostMalloc(&st.host, st.cap, hipHostMallocDefault));
    }
    if (!st.done) HIP_OK(hipEventCreateWithFlags(&st.done, hipEventDisableTiming));
    for (size_t v = 0; v < n; ++v) std::memcpy(static_cast<char*>(st.host) + v * bytes, srcs[v], bytes);
    HIP_OK(hipMemcpyAsync(dev_dst, st.host, n * bytes, hipMemcpyHostToDevice, stream));
    HIP_OK(hipEventRecord(st.done, stream));
    st.pending = true;
  }
  PendingRun run;
  bool batching = true;      // record Hw_* calls and launch them together
  BatchOpDev* run_dev = nullptr;
  static constexpr size_t kMaxRun = 2048;
  void flush_run();
  // A Mod_down or Rescale of one polynomial waits for the next call: generated code issues them in pairs (c0, then
  // c1), and two polynomials through one set of launches take little longer than one, the launches of a single
  // polynomial being far too small for the machine.  Anything else that arrives first sends it off alone.
  struct PendingPoly {
    int kind = 0;  // 0 none, 1 Mod_down, 2 Rescale
    u64* res = nullptr;
    const u64* src = nullptr;
    size_t level = 0;
    bool is_ntt = false;
  } ppoly;
  void flush_poly();
  void submit_poly(int kind, u64* res, const u64* src, size_t level, bool is_ntt);
  void flush_pending() {
    flush_poly();
    flush_run();
  }
  // The same for an entry point that names everything it touches: `writes` are ranges it fills completely without
  // reading them, `reads` everything else it reads or writes.  A recorded zero fill that nothing recorded after it
  // touches (the fill of a fresh buffer, which Alloc_poly promises) is then dropped if it lies inside a range the
  // entry point overwrites, and moved behind the entry point's own launches, into the next run, if the entry point
  // does not touch it at all; only a fill it reads is carried out now.
  struct Span {
    uintptr_t lo, hi;
  };
  static Span span(const void* p, size_t words) { return Span{(uintptr_t)p, (uintptr_t)p + words * sizeof(u64)}; }
  std::vector<Span> decl_writes, decl_reads;
  bool decl_active = false;
  void flush_pending_declared(std::initializer_list<Span> writes, std::initializer_list<Span> reads,
                              bool keep_poly = false) {
    if (!keep_poly) flush_poly();
    decl_writes.assign(writes.begin(), writes.end());
    decl_reads.assign(reads.begin(), reads.end());
    decl_active = true;
    flush_run();
    decl_active = false;
  }
  void flush_pending_overwriting(const void* out, size_t out_words, const void* in, size_t in_words,
                                 bool keep_poly = false) {
    flush_pending_declared({span(out, out_words)}, {span(in, in_words)}, keep_poly);
  }
  bool run_accepts(const BatchOp& o, u64 n) const;
  void run_append(const BatchOp& o, u64 n);
  void drop_untouched_fills(const void* p, size_t words);
  std::map<std::pair<size_t, size_t>, ModUpDev> modup;
  std::map<size_t, RescaleDev> rescale;
  std::map<size_t, PrecompDev> precomp;
  std::map<size_t, ModDownRescaleDev> moddown_rescale;
  // Mod_down / Extend constants
  u64* phat = nullptr;        // [K][L]
  u64* pscale_ntt = nullptr;  // [K][2]
  u64* pscale_coef = nullptr; // [K][2]
  u64* pinv = nullptr;        // [L][2]
  u64* pmodq = nullptr;       // [L][2]
  ConvJob p2q_job{};          // P -> Q conversion onto all L limbs (callers lower nc to their level)
  // encoder
  size_t q0_bits = 0, sf_bits = 0;  // 0: the primes were given explicitly, no scaling factor is known
  double2* fft_rou = nullptr;       // [2N] exp(2 pi i k / 2N)
  u32* rot_group = nullptr;         // [N/2] 5^k mod 2N
  int* d_err = nullptr;             // sticky device flag of checks that run inside kernels
  // decoder: inv[L] then garner[L][L] (see crt_to_double), built on first use; Q = q0..q(level-1) per level
  u64* decode_tab = nullptr;
  std::map<size_t, u64*> decode_q;
  void check_deferred() {
    int e = 0;
    HIP_OK(hipMemcpyAsync(&e, d_err, sizeof(int), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    if (e) {
      HIP_OK(hipMemsetAsync(d_err, 0, sizeof(int), stream));
      throw std::runtime_error(
          "encode vector out of range, please increase encoding level or increase first_mod_size & "
          "scale_mod_size or decrease scale of msg");
    }
  }
  u32* order_report = nullptr;  // [1 + N / 4096] on the device: what order_check_kernel found (see Family::order_fits)
  void forget_orders(const void* dst, size_t words) {
    std::lock_guard<std::mutex> lock(family->mu);
    auto& fits = family->order_fits;
    if (fits.empty()) return;
    // a table at address a (N words) overlaps [lo, hi) when a < hi and lo < a + span
    const uintptr_t lo = (uintptr_t)dst, hi = lo + words * sizeof(u64), span = (uintptr_t)h.N * sizeof(i64);
    auto it = fits.lower_bound(lo >= span ? lo - span + 1 : 0);
    while (it != fits.end() && it->first < hi) it = fits.erase(it);
  }
  void note_order(const void* order, bool ok) {
    std::lock_guard<std::mutex> lock(family->mu);
    family->order_fits[(uintptr_t)order] = ok;
  }
  bool order_fits_chunks(const i64* order) {
    {
      std::lock_guard<std::mutex> lock(family->mu);
      auto it = family->order_fits.find((uintptr_t)order);
      if (it != family->order_fits.end()) return it->second;
    }
    bool ok = false;
    if (d.logN > 12) {
      const u32 nb = h.N >> 12;
      std::vector<u32> rep(1 + nb, 0);
      HIP_OK(hipMemsetAsync(order_report, 0, rep.size() * sizeof(u32), stream));
      launch_order_check(stream, d, order, order_report);
      HIP_OK(hipMemcpyAsync(rep.data(), order_report, rep.size() * sizeof(u32), hipMemcpyDeviceToHost, stream));
      HIP_OK(hipStreamSynchronize(stream));
      ok = rep[0] == 0;
      std::vector<char> seen(nb, 0);
      for (u32 b = 0; ok && b < nb; ++b) {
        if (rep[1 + b] >= nb || seen[rep[1 + b]]) ok = false;
        else seen[rep[1 + b]] = 1;
      }
    }
    note_order(order, ok);
    return ok;
  }
  LimbMap q_lm{}, p_lm{};     // identity maps: limb t -> prime t / prime L+t
  // ace_alloc / ace_free: sizes of the buffers handed out, and freed buffers kept for reuse
  std::multimap<size_t, void*> pool;
  size_t pooled_words = 0;
  void drop_pool() {
    if (stream) (void)hipStreamSynchronize(stream);
    for (auto& kv : pool) (void)hipFree(kv.second);
    pool.clear();
    family->pooled_words -= pooled_words;
    pooled_words = 0;
  }
  // scratch arena
  u64* ws = nullptr;
  size_t ws_words = 0, ws_used = 0;
  u64* static_scratch = nullptr;  // this GPU's copy of the device array `scratch` (ace_mod_down_noalloc)
  // A second lane for calls that may overlap with those of the first (ace_fork / ace_fork_switch / ace_join): its
  // own stream (same priority), scratch arena, buffer pool and run image; everything else (tables, the map of live
  // buffers) is shared.  `idle` holds the lane that is not in use; swapping makes every entry point work on the other
  // lane without knowing.  A buffer freed on a lane joins that lane's pool, so its next use is ordered on the stream
  // that last touched it (or on one that has waited for it at the fork or the join).
  struct Lane {
    hipStream_t stream = nullptr;
    u64* ws = nullptr;
    size_t ws_words = 0, ws_used = 0;
    std::multimap<size_t, void*> pool;
    size_t pooled_words = 0;
    BatchOpDev* run_dev = nullptr;
  } idle;
  int fork_state = 0;  // 0 one lane; 1 issuing on the second lane; 2 back on the first, the second's work in flight
  hipEvent_t fork_ev = nullptr, join_ev = nullptr;
  void swap_lanes() {
    std::swap(stream, idle.stream);
    std::swap(ws, idle.ws);
    std::swap(ws_words, idle.ws_words);
    std::swap(ws_used, idle.ws_used);
    std::swap(pool, idle.pool);
    std::swap(pooled_words, idle.pooled_words);
    std::swap(run_dev, idle.run_dev);
  }

  template <class T>
  T* upload_vec(const std::vector<T>& v) {
    T* p = nullptr;
    HIP_OK(hipMalloc((void**)&p, std::max<size_t>(v.size(), 1) * sizeof(T)));
    HIP_OK(hipMemcpy(p, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
    owned.push_back(p);
    return p;
  }
  ShoupConst sc(u64 w, size_t prime) const { return {w, shoup(w, h.primes[prime].q)}; }

  // FP64 tables of a base conversion (ConvJob::fw / fq) for the targets below kFpConvTargetLimit
  bool conv_fp = true;
  bool conv_matrix = true;  // base conversions on the matrix cores (ACE_CONV_MATRIX=0 in the environment: off)
  // Mod_down followed by Rescale through one forward transform where an entry point knows both
  // (ACE_SHARE_TRANSFORM=0 in the environment: the two one after the other; same words)
  bool share_transform = true;
  // an HMult's d2 formed as the inverse transform of Mod_up reads its factors (ACE_PRODUCT_ON_LOAD=0: as a kernel of
  // its own; same words)
  bool product_on_load = true;
  void conv_fp_tables(ConvJob& j, const std::vector<size_t>& src, const std::vector<size_t>& tgt, const u64* hat,
                      size_t hat_stride) {
    j.fw = j.fq = nullptr;
    j.fw_stride = 0;
    std::memset(j.fp_target, 0, sizeof(j.fp_target));
    if (!conv_fp || src.size() > 16) return;  // 48 products at most in a sum
    bool any = false;
    for (size_t jj = 0; jj < tgt.size(); ++jj) {
      j.fp_target[jj] = h.primes[tgt[jj]].q < kFpConvTargetLimit ? 1 : 0;
      any |= j.fp_target[jj] != 0;
    }
    if (!any) return;
    const size_t nd = src.size(), nc = tgt.size();
    std::vector<double> fw(3 * nd * nc * 2 + 8, 0.0), fq(nc * 2, 0.0);  // a margin of four entries for grouped reads
    for (size_t jj = 0; jj < nc; ++jj) {
      const u64 q = h.primes[tgt[jj]].q;
      fq[2 * jj] = (double)q;
      fq[2 * jj + 1] = (double)(1.0L / (long double)q);
      if (!j.fp_target[jj]) continue;
      for (size_t k = 0; k < nd; ++k) {
        const u64 w = hat[k * hat_stride + jj];
        for (size_t i = 0; i < 3; ++i) {
          const u64 wi = mul_mod(w, ((u64)1 << (21 * i)) % q, q);
          fw[2 * ((3 * k + i) * nc + jj)] = (double)(wi >> 26);
          fw[2 * ((3 * k + i) * nc + jj) + 1] = (double)(wi & (((u64)1 << 26) - 1));
        }
      }
    }
    j.fw = upload_vec(fw);
    j.fq = upload_vec(fq);
    j.fw_stride = (u32)nc;
  }

  // Operands of a base conversion on the matrix cores (ConvJob::mx / mq): for targets j, source k and byte a of
  // a source word the constant hat_kj * 2^(8a) mod m_j in signed bytes, laid out as the MFMA's A operand: lane l of
  // (quad, step) holds row l % 32 and inner indices 16 (l / 32) .. + 15, inner index t of step s being byte t % 8 of
  // source 4 s + t / 8; row rho is byte 4 (rho / 8) + rho % 4 (below 8: the first, from 8: the second) of the two
  // targets lane half (rho / 4) % 2 finds in its result registers.
  void conv_matrix_tables(ConvJob& j, const std::vector<size_t>& tgt, const u64* hat, size_t hat_stride, size_t nd) {
    j.mx = nullptr;
    j.mt = nullptr;
    if (nd > 4 * kMxSteps) return;
    for (size_t p : tgt)
      if (h.primes[p].q >> 61) return;
    const size_t nc = tgt.size(), quads = (nc + 3) / 4;
    std::vector<ConvTarget> mt((quads + 1) * 4, ConvTarget{1, 1.0, 0, 0});  // a spare quad: the kernel reads one ahead
    std::vector<u64> signed_bytes(nc * nd * 8);
    for (size_t jj = 0; jj < nc; ++jj) {
      const u64 q = h.primes[tgt[jj]].q;
      mt[jj] = ConvTarget{q, (double)(1.0L / (long double)q), (u64)j.map.out_limb[jj] * h.N, 0};
      for (size_t k = 0; k < nd; ++k) {
        u64 cst = hat[k * hat_stride + jj] % q;
        for (size_t a = 0; a < 8; ++a) {
          signed_bytes[(jj * nd + k) * 8 + a] = (cst + 0x8080808080808080ull) ^ 0x8080808080808080ull;
          cst = mul_mod(cst, 256 % q, q);
        }
      }
    }
    std::vector<uint8_t> tab((quads + 1) * kMxSteps * 64 * 16, 0);
    for (size_t quad = 0; quad < quads; ++quad)
      for (size_t s = 0; s < kMxSteps; ++s)
        for (size_t lane = 0; lane < 64; ++lane) {
          const size_t rho = lane % 32, kb = lane / 32, half = (rho / 4) % 2, r = (rho / 8) * 4 + rho % 4;
          const size_t jj = quad * 4 + 2 * half + r / 8, byte = r % 8;
          if (jj >= nc) continue;
          for (size_t t = 0; t < 16; ++t) {
            const size_t k = 4 * s + 2 * kb + t / 8, a = t % 8;
            if (k >= nd) continue;
            tab[((quad * kMxSteps + s) * 64 + lane) * 16 + t] = (uint8_t)(signed_bytes[(jj * nd + k) * 8 + a] >> (8 * byte));
          }
        }
    j.mx = reinterpret_cast<const uint4*>(upload_vec(tab));
    j.mt = upload_vec(mt);
  }

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
    m.job.hat = m.hat;
    m.job.hat_stride = (u32)nc;
    m.job.nd = (u32)nd;
    m.job.nc = (u32)nc;
    m.job.map = m.conv;
    conv_fp_tables(m.job, std::vector<size_t>(m.t.digit.begin(), m.t.digit.end()),
                   std::vector<size_t>(m.t.compl_idx.begin(), m.t.compl_idx.end()), m.t.hat.data(), nc);
    conv_matrix_tables(m.job, std::vector<size_t>(m.t.compl_idx.begin(), m.t.compl_idx.end()), m.t.hat.data(), nc, nd);
    return modup.emplace(key, std::move(m)).first->second;
  }

  const PrecompDev& precomp_at(size_t level) {
    auto it = precomp.find(level);
    if (it != precomp.end()) return it->second;
    PrecompDev pd;
    const size_t nd = h.num_decomp(level), T = level + h.K, N = h.N;
    std::vector<u64> sn(2 * level), scf(2 * level);
    pd.one_ntt_launch = nd * T <= 256;
    for (size_t d = 0; d < nd; ++d) {
      const ModUpDev& m = modup_at(level, d);
      const size_t start = h.part_size * d, len = m.t.digit.size(), nc = m.t.compl_idx.size();
      for (size_t i = 0; i < len; ++i) {
        size_t pi = m.t.digit[i];
        u64 q = h.primes[pi].q;
        u64 a = mul_mod(h.primes[pi].ninv, m.t.hat_inv[i], q);
        sn[2 * pi] = a;                 sn[2 * pi + 1] = shoup(a, q);
        scf[2 * pi] = m.t.hat_inv[i];   scf[2 * pi + 1] = shoup(m.t.hat_inv[i], q);
      }
      ConvJob j = m.job;
      j.t_off = start * N;
      j.out_off = d * T * N;
      pd.jobs.push_back(j);
      for (size_t k = 0; k < nc; ++k) {
        if (pd.n_tgt < (u32)kMaxPrimes) {
          pd.tgt_lm.prime[pd.n_tgt] = m.compl_lm.prime[k];
          pd.tgt_pos.prime[pd.n_tgt] = (uint8_t)(d * T + m.compl_pos.prime[k]);
        }
        ++pd.n_tgt;
      }
    }
    if (pd.n_tgt > (u32)kMaxPrimes) pd.one_ntt_launch = false;
    pd.scale_ntt = upload_vec(sn);
    pd.scale_coef = upload_vec(scf);
    return precomp.emplace(level, std::move(pd)).first->second;
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

  const ModDownRescaleDev& moddown_rescale_at(size_t level) {
    auto it = moddown_rescale.find(level);
    if (it != moddown_rescale.end()) return it->second;
    std::vector<u64> qi, nqi;
    h.rescale_table(level, qi, nqi);
    const size_t last = level - 1;
    const u64 ql = h.primes[last].q;
    ModDownRescaleDev m;
    std::vector<u64> sc(2 * (1 + h.K)), tl(2 * last), colc(level);
    const u64 a = mul_mod(h.primes[last].ninv, h.pinv_modq[last], ql);
    sc[0] = a; sc[1] = shoup(a, ql);
    m.inv_lm.prime[0] = (uint8_t)last;
    for (size_t j = 0; j < h.K; ++j) {
      const u64 q = h.primes[h.L + j].q, b = mul_mod(h.primes[h.L + j].ninv, h.phat_inv[j], q);
      sc[2 * (1 + j)] = b; sc[2 * (1 + j) + 1] = shoup(b, q);
      m.inv_lm.prime[1 + j] = (uint8_t)(h.L + j);
    }
    for (size_t i = 0; i < last; ++i) {
      const u64 q = h.primes[i].q;
      const u64 t = mul_mod(h.pinv_modq[i], qi[i], q);
      colc[i] = mul_mod(h.pinv_modq[i], nqi[i], q);
      tl[2 * i] = t; tl[2 * i + 1] = shoup(t, q);
    }
    colc[last] = h.pinv_modq[last];
    m.ql_inv.assign(qi.begin(), qi.begin() + last);
    m.inv_scale = upload_vec(sc);
    m.tail = upload_vec(tl);
    {
      std::vector<u64> ph(h.K * level);
      std::vector<size_t> src, tgt;
      for (size_t j = 0; j < h.K; ++j) {
        src.push_back(h.L + j);
        for (size_t i = 0; i < level; ++i)
          ph[j * level + i] = mul_mod(h.phat_modq[i * h.K + j], colc[i], h.primes[i].q);
      }
      for (size_t i = 0; i < level; ++i) {
        tgt.push_back(i);
        m.job.map.prime[i] = (uint8_t)i;
        m.job.map.out_limb[i] = (uint8_t)i;
      }
      m.job.hat = upload_vec(ph);
      m.job.hat_stride = (u32)level;
      m.job.nd = (u32)h.K;
      m.job.nc = (u32)level;
      conv_fp_tables(m.job, src, tgt, ph.data(), level);
      conv_matrix_tables(m.job, tgt, ph.data(), level, h.K);
    }
    return moddown_rescale.emplace(level, m).first->second;
  }

  // A context that shares `from`'s device tables (twiddles, per-prime constants, P -> Q conversion, encoder tables)
  // and has its own stream, scratch arena, buffer pool, recorded run and lazily built per-level tables.
  void init_shared(const ace_ctx& from) {
    static_scratch = static_scratch_of_current_device();
    HIP_OK(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    HIP_OK(hipEventCreate(&ev0));
    HIP_OK(hipEventCreate(&ev1));
    d = from.d;
    conv_fp = from.conv_fp;
    conv_matrix = from.conv_matrix;
    share_transform = from.share_transform;
    product_on_load = from.product_on_load;
    q_lm = from.q_lm;
    p_lm = from.p_lm;
    phat = from.phat;
    p2q_job = from.p2q_job;
    pscale_ntt = from.pscale_ntt;
    pscale_coef = from.pscale_coef;
    pinv = from.pinv;
    pmodq = from.pmodq;
    fft_rou = from.fft_rou;
    rot_group = from.rot_group;
    q0_bits = from.q0_bits;
    sf_bits = from.sf_bits;
    batching = from.batching;
    std::vector<int> z(1, 0);
    d_err = upload_vec(z);
    std::vector<u32> rep(1 + (h.N >> 12) + 1, 0);
    order_report = upload_vec(rep);
  }

  void init_device() {
    static_scratch = static_scratch_of_current_device();
    {
      // A ResNet-20 image leaves about 10 GiB of freed polynomials behind for the next one, per thread that runs
      // images; beyond the limit a freed buffer goes back to the driver, which waits for the stream each time.
      size_t free_b = 0, total_b = 0;
      if (hipMemGetInfo(&free_b, &total_b) == hipSuccess && total_b) family->pool_limit_words = total_b / 3 / sizeof(u64);
      if (const char* gb = std::getenv("ACE_POOL_LIMIT_GB")) family->pool_limit_words = (size_t)(atof(gb) * (double)(1 << 27));
    }
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
      conv_fp = !(force_int && force_int[0] == '1');
      const char* no_matrix = std::getenv("ACE_CONV_MATRIX");
      conv_matrix = !(no_matrix && no_matrix[0] == '0');
      const char* no_share = std::getenv("ACE_SHARE_TRANSFORM");
      share_transform = !(no_share && no_share[0] == '0');
      const char* no_product = std::getenv("ACE_PRODUCT_ON_LOAD");
      product_on_load = !(no_product && no_product[0] == '0');
      bool use_fp = conv_fp && h.logN > 12;
      std::vector<double> w(T * h.N, 0.0), iw(T * h.N, 0.0);
      for (size_t i = 0; i < T; ++i) {
        d.fp_ok[i] = (use_fp && h.primes[i].q < kFpPrimeLimit) ? 1 : 0;
        if (!d.fp_ok[i]) continue;
        for (size_t k = 0; k < h.N; ++k) {
          size_t o = i * h.N + k;
          // centred on zero: |w| <= q/2 halves the error of the quotient estimate in a twiddle product, which is
          // what lets six forward stages run between two reductions (ace_ntt.hip)
          const i64 q = (i64)h.primes[i].q, a = (i64)h.rou[o], b = (i64)h.irou[o];
          w[o] = (double)(a > q / 2 ? a - q : a);
          iw[o] = (double)(b > q / 2 ? b - q : b);
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
    {
      std::vector<double> rou_d;
      std::vector<u32> rot;
      fft_tables(h.N, rou_d, rot);
      std::vector<double2> rou(rou_d.size() / 2);
      for (size_t i = 0; i < rou.size(); ++i) rou[i] = make_double2(rou_d[2 * i], rou_d[2 * i + 1]);
      fft_rou = upload_vec(rou);
      rot_group = upload_vec(rot);
      std::vector<int> z(1, 0);
      d_err = upload_vec(z);
    }
    phat = upload_vec(ph);
    {
      std::vector<size_t> src, tgt;
      for (size_t j = 0; j < h.K; ++j) src.push_back(h.L + j);
      for (size_t i = 0; i < h.L && i < (size_t)kMaxPrimes; ++i) {
        tgt.push_back(i);
        p2q_job.map.prime[i] = (uint8_t)i;
        p2q_job.map.out_limb[i] = (uint8_t)i;
      }
      p2q_job.hat = phat;
      p2q_job.hat_stride = (u32)h.L;
      p2q_job.nd = (u32)h.K;
      p2q_job.nc = (u32)h.L;
      conv_fp_tables(p2q_job, src, tgt, ph.data(), h.L);
      conv_matrix_tables(p2q_job, tgt, ph.data(), h.L, h.K);
    }
    {
      std::vector<u32> rep(1 + (h.N >> 12) + 1, 0);
      order_report = upload_vec(rep);
    }
    pscale_ntt = upload_vec(sn);
    pscale_coef = upload_vec(scf);
    pinv = upload_vec(pi);
    pmodq = upload_vec(pm);
  }

  ~ace_ctx() {
    try {
      flush_pending();
    } catch (...) {
    }
    if (std::getenv("ACE_HIP_PROFILE"))
      std::fprintf(stderr, "[ace_hip] context %p: arena %.2f GiB, %zu freed buffers kept (%.2f GiB), second lane %.2f GiB\n",
                   (void*)this, (double)ws_words / (double)(1 << 27), pool.size(), (double)pooled_words / (double)(1 << 27),
                   (double)(idle.ws_words + idle.pooled_words) / (double)(1 << 27));
    if (stream) (void)hipStreamSynchronize(stream);
    for (Stage& st : stages) {
      if (st.host) (void)hipHostFree(st.host);
      if (st.done) (void)hipEventDestroy(st.done);
    }
    if (fork_state == 1) swap_lanes();  // destroyed in the middle of a fork: back to the first lane
    if (idle.stream) (void)hipStreamSynchronize(idle.stream);
    for (Stage& st : gather_stages) {
      if (st.host) (void)hipHostFree(st.host);
      if (st.done) (void)hipEventDestroy(st.done);
    }
    for (void* p : owned) (void)hipFree(p);
    drop_pool();
    for (auto& kv : idle.pool) (void)hipFree(kv.second);
    family->pooled_words -= idle.pooled_words;
    if (idle.ws) (void)hipFree(idle.ws);
    if (idle.stream) (void)hipStreamDestroy(idle.stream);
    if (fork_ev) (void)hipEventDestroy(fork_ev);
    if (join_ev) (void)hipEventDestroy(join_ev);
    if (ws) (void)hipFree(ws);
    if (ev0) (void)hipEventDestroy(ev0);
    if (ev1) (void)hipEventDestroy(ev1);
    if (stream) (void)hipStreamDestroy(stream);
  }
};

// ---- recorded Hw_* calls --------------------------------------------------------------------------
// A run is launched as one kernel in which the thread of element i carries out its chain's entries in order.
// That equals issuing the calls one by one as long as (1) ranges that overlap are the same range, so element i
// of one entry is element i of the other, and (2) a rotate, which reads other elements than its own, neither
// reads nor overwrites anything else the run touches.  An entry that would break this starts a new run.
bool ace_ctx::run_accepts(const BatchOp& o, u64 n) const {
  if (run.ops.empty()) return true;
  if (n != run.n || run.ops.size() >= kMaxRun) return false;
  const uintptr_t bytes = (uintptr_t)n * sizeof(u64);
  auto misaligned = [&](const void* p) {  // overlaps a range of the run without being that range
    const uintptr_t x = (uintptr_t)p;
    auto it = run.touched.lower_bound(x);
    if (it != run.touched.end() && *it != x && *it - x < bytes) return true;
    if (it != run.touched.begin()) {
      --it;
      if (*it != x && x - *it < bytes) return true;
    }
    return false;
  };
  const bool rotate = o.op == BATCH_ROTATE;
  const uintptr_t r = (uintptr_t)o.r, a = (uintptr_t)o.a, b = (uintptr_t)o.b;
  if (misaligned(o.r) || (o.a && misaligned(o.a)) || (o.b && misaligned(o.b))) return false;
  if (rotate) {
    if (run.touched.count(r)) return false;                       // its result is anything the run used
    if (run.written.count(a) || run.rot_res.count(a)) return false;  // its source or table was written by the run
    if (run.written.count(b) || run.rot_res.count(b)) return false;
    return true;
  }
  // an elementwise entry may not read a rotate's result (other threads wrote it) nor overwrite its sources
  if ((o.a && run.rot_res.count(a)) || (o.b && run.rot_res.count(b)) || run.rot_res.count(r)) return false;
  if (run.rot_src.count(r)) return false;
  return true;
}

void ace_ctx::run_append(const BatchOp& o, u64 n) {
  if (!run_accepts(o, n)) flush_run();
  run.n = n;
  run.ops.push_back(o);
  run.touched.insert((uintptr_t)o.r);
  if (o.a) run.touched.insert((uintptr_t)o.a);
  if (o.b) run.touched.insert((uintptr_t)o.b);
  if (o.op == BATCH_ROTATE) {
    run.rot_res.insert((uintptr_t)o.r);
    run.rot_src.insert((uintptr_t)o.a);
    run.rot_src.insert((uintptr_t)o.b);
  } else {
    run.written.insert((uintptr_t)o.r);
  }
}

// Recorded zero fills inside [p, p + words) that no later entry of the run reads or writes are taken out (the
// buffer is being released: nobody will see them).
void ace_ctx::drop_untouched_fills(const void* p, size_t words) {
  if (run.ops.empty()) return;
  const uintptr_t lo = (uintptr_t)p, hi = lo + words * sizeof(u64);
  auto in_span = [&](const void* x) { return (uintptr_t)x >= lo && (uintptr_t)x < hi; };
  std::unordered_set<uintptr_t> later;  // ranges of the buffer that entries behind the current one touch
  std::vector<uint8_t> gone(run.ops.size(), 0);
  bool any = false;
  for (size_t k = run.ops.size(); k-- > 0;) {
    const BatchOp& o = run.ops[k];
    if (o.op == BATCH_ZERO && in_span(o.r) && !later.count((uintptr_t)o.r)) {
      gone[k] = 1;
      any = true;
      continue;
    }
    if (in_span(o.r)) later.insert((uintptr_t)o.r);
    if (o.a && in_span(o.a)) later.insert((uintptr_t)o.a);
    if (o.b && in_span(o.b)) later.insert((uintptr_t)o.b);
  }
  if (!any) return;
  size_t w = 0;
  for (size_t k = 0; k < run.ops.size(); ++k)
    if (!gone[k]) run.ops[w++] = run.ops[k];
  run.ops.resize(w);  // (the sets of touched ranges keep the fills' addresses: they only make the run more careful)
}

void ace_ctx::flush_run() {
  if (run.ops.empty()) return;
  // Zero fills that nobody can see yet: the range is written by a later entry of the run before any entry reads it
  // (dropped), or the rest of the run leaves it alone and the flushing entry point, having named its operands,
  // overwrites it (dropped) or does not touch it (moved into the next run).  Ranges of a run that overlap are
  // identical, so the start address names the range.
  std::vector<BatchOp> carried;
  {
    const uintptr_t bytes = (uintptr_t)run.n * sizeof(u64);
    auto overlaps = [&](const std::vector<Span>& v, uintptr_t r) {
      for (const Span& x : v)
        if (r < x.hi && x.lo < r + bytes) return true;
      return false;
    };
    auto inside = [&](const std::vector<Span>& v, uintptr_t r) {
      for (const Span& x : v)
        if (r >= x.lo && r + bytes <= x.hi) return true;
      return false;
    };
    std::vector<BatchOp> kept;
    kept.reserve(run.ops.size());
    for (size_t k = 0; k < run.ops.size(); ++k) {
      const BatchOp& o = run.ops[k];
      bool dead = false, carry = false;
      if (o.op == BATCH_ZERO) {
        const uintptr_t r = (uintptr_t)o.r;
        bool touched = run.ops.size() - k > 512;  // a longer look ahead is not worth its time: the fill stays
        for (size_t j = k + 1; j < run.ops.size() && !touched; ++j) {
          BatchOp& n = run.ops[j];
          const bool reads_b = !(n.op == BATCH_COPY || n.op == BATCH_ZERO || (n.op >= EW_ADD_S && n.op <= EW_MULADD_S));
          const bool reads_r = n.op == EW_MULADD || n.op == EW_MULADD_S;
          const bool a_is_r = n.op != BATCH_ZERO && (uintptr_t)n.a == r, b_is_r = reads_b && (uintptr_t)n.b == r;
          if (reads_r && (uintptr_t)n.r == r && !a_is_r && !b_is_r) {
            // the first thing that happens to the zeros is a product added to them: the product alone
            n.op = n.op == EW_MULADD ? (u32)EW_MUL : (u32)EW_MUL_S;
            touched = dead = true;
          } else if (n.op == EW_ADD && (uintptr_t)n.r == r && a_is_r != b_is_r) {
            // ... or a sum with them: a copy of the other operand (residues are canonical, 0 + x = x)
            n = BatchOp{n.r, a_is_r ? n.b : n.a, nullptr, 0, (u32)BATCH_COPY, n.prime};
            touched = dead = true;
          } else if (a_is_r || b_is_r || (reads_r && (uintptr_t)n.r == r)) {
            touched = true;  // read first: the zeros are needed
          } else if ((uintptr_t)n.r == r) {
            touched = dead = true;  // written first
          }
        }
        if (!touched && decl_active && !overlaps(decl_reads, r)) {
          if (inside(decl_writes, r)) dead = true;
          else if (!overlaps(decl_writes, r)) carry = true;
        }
      }
      if (carry) carried.push_back(o);
      else if (!dead) kept.push_back(o);
    }
    run.ops.swap(kept);
  }
  const u64 carried_n = run.n;
  auto recarry = [&]() {  // the fills that wait: first entries of the next run
    for (const BatchOp& o : carried) run_append(o, carried_n);
  };
  if (run.ops.empty()) {
    run.touched.clear();
    run.written.clear();
    run.rot_res.clear();
    run.rot_src.clear();
    recarry();
    return;
  }
  size_t count = run.ops.size();
  // Scratch results: entry k's range is read by entry k+1 (which the kernel serves from a register), by nothing
  // else before a later entry overwrites it.  Such a store is dropped, and the range then ties k to k+1 only:
  // the limb-by-limb products of an inner product (Hw_modmul into one scratch limb, Hw_modadd from it) become
  // chains of their own instead of one long chain through the scratch limb.
  auto reads_of = [](const BatchOp& o, uintptr_t out[3]) {
    const u32 op = o.op & ~kBatchDeadStore;
    out[0] = op == BATCH_ZERO ? 0 : (uintptr_t)o.a;
    out[1] = (op == BATCH_ROTATE || op == BATCH_COPY || op == BATCH_ZERO || (op >= EW_ADD_S && op <= EW_MULADD_S))
                 ? 0 : (uintptr_t)o.b;
    out[2] = (op == EW_MULADD || op == EW_MULADD_S) ? (uintptr_t)o.r : 0;
  };
  std::vector<uint8_t> scratch_read(count, 0);  // entry reads its predecessor's dropped result
  for (u32 k = 0; k + 1 < count; ++k) {
    BatchOp& o = run.ops[k];
    if (o.op == BATCH_ROTATE || run.ops[k + 1].op == BATCH_ROTATE) continue;
    const uintptr_t r = (uintptr_t)o.r;
    uintptr_t rd[3];
    reads_of(run.ops[k + 1], rd);
    if (rd[0] != r && rd[1] != r && rd[2] != r) continue;
    bool dead = false;
    for (u32 j = k + 1; j < count && j <= k + 16; ++j) {
      const BatchOp& n = run.ops[j];
      if (j > k + 1) {
        reads_of(n, rd);
        const bool rot_touch = n.op == BATCH_ROTATE && ((uintptr_t)n.a == r || (uintptr_t)n.b == r);
        if (rd[0] == r || rd[1] == r || rd[2] == r || rot_touch) break;
      }
      if ((uintptr_t)n.r == r) {
        dead = true;
        break;
      }
    }
    if (dead) {
      o.op |= kBatchDeadStore;
      scratch_read[k + 1] = 1;
    }
  }
  // A product into such a scratch limb followed by the sum that adds it to its own destination is one
  // multiply-add entry (the same canonical value): half the entries, so more runs travel as kernel arguments.
  {
    std::vector<BatchOp> merged;
    std::vector<uint8_t> merged_read;
    merged.reserve(count);
    for (u32 k = 0; k < count; ++k) {
      const BatchOp& o = run.ops[k];
      const u32 op = o.op & ~kBatchDeadStore;
      if ((o.op & kBatchDeadStore) && (op == EW_MUL || op == EW_MUL_S) && !scratch_read[k] && k + 1 < count) {
        const BatchOp& n = run.ops[k + 1];
        const bool sum_to_self = n.op == EW_ADD && n.prime == o.prime && n.r != o.r &&
                                 ((n.a == n.r && n.b == o.r) || (n.b == n.r && n.a == o.r));
        if (sum_to_self) {
          merged.push_back(BatchOp{n.r, o.a, o.b, o.scalar, (u32)(op == EW_MUL ? EW_MULADD : EW_MULADD_S), o.prime});
          merged_read.push_back(0);
          ++k;
          continue;
        }
        if (n.op == BATCH_COPY && n.a == o.r && n.r != o.r) {  // ... or by its copy: the product goes there
          merged.push_back(BatchOp{n.r, o.a, o.b, o.scalar, op, o.prime});
          merged_read.push_back(0);
          ++k;
          continue;
        }
      }
      merged.push_back(o);
      merged_read.push_back(scratch_read[k]);
    }
    run.ops.swap(merged);
    scratch_read.swap(merged_read);
    count = run.ops.size();
  }
  // chains: entries joined whenever one writes a range the other reads or writes (union-find over entries)
  std::vector<u32> parent(count);
  for (u32 k = 0; k < count; ++k) parent[k] = k;
  auto find = [&](u32 x) {
    while (parent[x] != x) x = parent[x] = parent[parent[x]];
    return x;
  };
  auto join = [&](u32 x, u32 y) {
    x = find(x), y = find(y);
    if (x != y) parent[std::max(x, y)] = std::min(x, y);
  };
  std::unordered_map<uintptr_t, u32> writer;                // last entry that wrote the range
  std::unordered_map<uintptr_t, std::vector<u32>> readers;  // entries that read it since
  for (u32 k = 0; k < count; ++k) {
    const BatchOp& o = run.ops[k];
    const bool dead = (o.op & kBatchDeadStore) != 0;
    uintptr_t reads[3];
    reads_of(o, reads);
    for (uintptr_t x : reads) {
      if (!x) continue;
      if (scratch_read[k] && x == (uintptr_t)run.ops[k - 1].r) continue;  // comes in a register
      auto w = writer.find(x);
      if (w != writer.end()) join(k, w->second);
      readers[x].push_back(k);
    }
    if (scratch_read[k]) join(k, k - 1);
    if (dead) continue;  // writes nothing
    const uintptr_t r = (uintptr_t)o.r;
    auto w = writer.find(r);
    if (w != writer.end()) join(k, w->second);
    auto rd = readers.find(r);
    if (rd != readers.end()) {
      for (u32 j : rd->second) join(k, j);
      rd->second.clear();
    }
    writer[r] = k;
  }
  // entries sorted by chain, order inside a chain kept
  std::vector<u32> order(count);
  for (u32 k = 0; k < count; ++k) order[k] = k;
  std::stable_sort(order.begin(), order.end(), [&](u32 x, u32 y) { return find(x) < find(y); });
  std::vector<BatchOp> sorted(count);
  std::vector<u32> chain_start;
  for (u32 k = 0; k < count; ++k) {
    if (k == 0 || find(order[k]) != find(order[k - 1])) chain_start.push_back(k);
    sorted[k] = run.ops[order[k]];
  }
  const u32 n_chains = (u32)chain_start.size();
  chain_start.push_back((u32)count);
  const u64 n = run.n;
  run.ops.clear();
  run.touched.clear();
  run.written.clear();
  run.rot_res.clear();
  run.rot_src.clear();
  recarry();
  auto compact = [](const BatchOp& o) {
    const u32 op = o.op & ~kBatchDeadStore;
    const bool scalar = op >= EW_ADD_S && op <= EW_MULADD_S;
    return BatchOpDev{o.r, o.a, scalar ? o.scalar : (u64)(uintptr_t)o.b, o.op, o.prime};
  };
  // two elements per thread when every range of the run allows 16-byte accesses
  bool pairs = n % 2 == 0;
  for (u32 k = 0; k < count && pairs; ++k) {
    const BatchOp& o = sorted[k];
    uintptr_t rd[3];
    reads_of(o, rd);
    const uintptr_t table = o.op == BATCH_ROTATE ? (uintptr_t)o.b : 0;
    pairs = (((uintptr_t)o.r | rd[0] | rd[1] | table) & 15) == 0;
  }
  if (count <= kSmallRun) {
    SmallRun small{};
    for (u32 k = 0; k < count; ++k) small.ops[k] = compact(sorted[k]);
    for (size_t k = 0; k < chain_start.size(); ++k) small.chain_start[k] = (uint16_t)chain_start[k];
    launch_ew_batch_small(stream, d, small, n_chains, n, pairs);
    return;
  }
  // entries and chain starts travel in one copy: [entries | chain starts]
  if (!run_dev) {
    HIP_OK(hipMalloc((void**)&run_dev, kMaxRun * sizeof(BatchOpDev) + (kMaxRun + 1) * sizeof(u32)));
    owned.push_back(run_dev);
  }
  const size_t ops_bytes = count * sizeof(BatchOpDev), chain_bytes = chain_start.size() * sizeof(u32);
  std::vector<unsigned char> image(ops_bytes + chain_bytes);
  for (u32 k = 0; k < count; ++k) reinterpret_cast<BatchOpDev*>(image.data())[k] = compact(sorted[k]);
  std::memcpy(image.data() + ops_bytes, chain_start.data(), chain_bytes);
  h2d(run_dev, image.data(), image.size());
  launch_ew_batch(stream, d, run_dev, reinterpret_cast<const u32*>(reinterpret_cast<const unsigned char*>(run_dev) + ops_bytes),
                  n_chains, n, pairs);
}

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
// Every sequencer works on a batch: n polynomials (or operands) per launch.

PolySeq shifted(const PolySeq& s, u64 words) {
  PolySeq r = s;
  r.b[0] += words;
  r.b[1] += words;
  return r;
}

// Decomp_modup (rns_poly.c:160-258), one digit of one polynomial: copy the
// digit, INTT it scaled by the inverse cofactors, convert to the complement
// basis, NTT the new limbs.  `digit` points at the digit's first limb (inside
// the source polynomial for the fused call, a compact copy for Mod_up).
void do_decomp_modup(ace_ctx* c, u64* res, const u64* digit, size_t level, size_t part, bool is_ntt) {
  const ModUpDev& m = c->modup_at(level, part);
  const size_t N = c->h.N, nd = m.t.digit.size(), nc = m.t.compl_idx.size(), start = c->h.part_size * part;
  // the digit's own limbs pass through; the inverse transform of a large ring drops that copy as it reads them
  const bool pass_through = res + start * N != digit, by_transform = pass_through && is_ntt && c->d.logN > 12;
  if (pass_through && !by_transform)
    HIP_OK(hipMemcpyAsync(res + start * N, digit, nd * N * sizeof(u64), hipMemcpyDeviceToDevice, c->stream));
  size_t mark = c->ws_used;
  u64* t = c->take(nd * N);
  if (is_ntt) {
    const CopyThrough through{seq_strided(res + start * N, 0), 0, ~0u};
    if (!launch_ntt(c->stream, c->d, seq_strided(t, 0), seq_strided(digit, 0), m.digit_lm, nullptr, (u32)nd, 1, true,
                    m.scale_ntt, 3, nullptr, by_transform ? &through : nullptr))
      throw std::runtime_error("internal: Mod_up transform rejected");
  } else {
    launch_mul_const(c->stream, c->d, t, digit, m.scale_coef, m.digit_lm, (u32)nd);
  }
  ConvBatch b{};
  b.matrix = c->conv_matrix;
  b.n_jobs = 1;
  b.job[0] = m.job;
  launch_baseconv(c->stream, c->d, res, t, b, 1);
  if (is_ntt)
    launch_ntt(c->stream, c->d, seq_strided(res, 0), seq_strided(res, 0), m.compl_lm, &m.compl_pos, (u32)nc, 1, false,
               nullptr);
  c->ws_used = mark;
}

// Precomp (rns_poly.c:416-481) for nb polynomials: operand o reads
// src + o*src_stride (level limbs) and writes res + o*res_stride
// (num_decomp x (level+K) limbs).  One INTT over all limbs (each scaled by its
// own digit's inverse cofactor), one base-conversion launch per 4 digits, one
// NTT over every converted limb.
// skip_own: the digits' own limbs are not copied into the raised polynomials (the caller's inner product reads them
// from src: OwnLimbs)
// times (with skip_own, NTT form): the polynomial raised is the limb-wise product of src and times (same stride), formed
// as the inverse transform reads them; false, with nothing launched, where that transform cannot do so.
bool do_precomp(ace_ctx* c, u64* res, u64 res_stride, const u64* src, u64 src_stride, size_t nb, size_t level,
                bool is_ntt, bool skip_own = false, const u64* times = nullptr) {
  const PrecompDev& pd = c->precomp_at(level);
  const size_t N = c->h.N, nd = c->h.num_decomp(level), T = level + c->h.K;
  size_t mark = c->ws_used;
  u64* t = c->take(nb * level * N);
  // the digits' own limbs pass through; the inverse transform of a large ring drops that copy as it reads them
  const bool by_transform = is_ntt && c->d.logN > 12 && !skip_own;
  if (times) {
    const PolySeq ts = seq_strided(times, src_stride);
    if (!is_ntt || !skip_own ||
        !launch_ntt(c->stream, c->d, seq_strided(t, level * N), seq_strided(src, src_stride), c->q_lm, nullptr,
                    (u32)level, (u32)nb, true, pd.scale_ntt, 3, nullptr, nullptr, &ts)) {
      c->ws_used = mark;
      return false;
    }
  } else if (is_ntt) {
    const CopyThrough through{seq_strided(res, res_stride), (u64)(T * N), (u32)c->h.part_size};
    if (!launch_ntt(c->stream, c->d, seq_strided(t, level * N), seq_strided(src, src_stride), c->q_lm, nullptr,
                    (u32)level, (u32)nb, true, pd.scale_ntt, 3, nullptr, by_transform ? &through : nullptr))
      throw std::runtime_error("internal: Mod_up transform rejected");
  } else {
    for (size_t o = 0; o < nb; ++o)
      launch_mul_const(c->stream, c->d, t + o * level * N, src + o * src_stride, pd.scale_coef, c->q_lm, (u32)level);
  }
  if (!by_transform && !skip_own)
    launch_digit_copy(c->stream, c->d, res, src, (u32)level, (u32)c->h.part_size, (u32)nd, T * N, res_stride,
                      src_stride, (u32)nb);
  // (large launches of N = 2^16 whose digits fit one conversion launch: conversion and strided pass of the transform
  // in one kernel)
  bool strided_done = false;
  for (size_t j0 = 0; j0 < nd; j0 += kMaxConvJobs) {
    ConvBatch b{};
    b.matrix = c->conv_matrix;
    b.n_jobs = (u32)std::min<size_t>(kMaxConvJobs, nd - j0);
    for (u32 k = 0; k < b.n_jobs; ++k) b.job[k] = pd.jobs[j0 + k];
    b.t_stride = level * N;
    b.out_stride = res_stride;
    if (is_ntt && pd.one_ntt_launch && nd <= (size_t)kMaxConvJobs)
      strided_done = launch_baseconv_fwd_strided(c->stream, c->d, res, t, b, (u32)nb);
    if (!strided_done) launch_baseconv(c->stream, c->d, res, t, b, (u32)nb);
  }
  if (is_ntt) {
    PolySeq rs = seq_strided(res, res_stride);
    if (pd.one_ntt_launch) {
      launch_ntt(c->stream, c->d, rs, rs, pd.tgt_lm, &pd.tgt_pos, pd.n_tgt, (u32)nb, false, nullptr,
                 strided_done ? 2 : 3);
    } else {
      for (size_t d = 0; d < nd; ++d) {
        const ModUpDev& m = c->modup_at(level, d);
        PolySeq ds = shifted(rs, d * T * N);
        launch_ntt(c->stream, c->d, ds, ds, m.compl_lm, &m.compl_pos, (u32)m.t.compl_idx.size(), (u32)nb, false,
                   nullptr);
      }
    }
  }
  c->ws_used = mark;
  return true;
}

// Mod_down (rns_poly.c:260-308) of np polynomials; addend_mode: 0 none,
// 1 add addend.at(p) to every polynomial, 2 only to even p
void do_mod_down(ace_ctx* c, const PolySeq& res, const PolySeq& src, size_t np, size_t level, bool is_ntt,
                 const PolySeq* addend, int addend_mode, const OrderSet* orders = nullptr) {
  const size_t N = c->h.N, K = c->h.K;
  size_t mark = c->ws_used;
  u64* t = c->take(np * K * N);
  u64* y = c->take(np * level * N);
  if (is_ntt) {
    launch_ntt(c->stream, c->d, seq_strided(t, K * N), shifted(src, level * N), c->p_lm, nullptr, (u32)K, (u32)np, true,
               c->pscale_ntt);
  } else {
    for (size_t p = 0; p < np; ++p)
      launch_mul_const(c->stream, c->d, t + p * K * N, src.at((u32)p) + level * N, c->pscale_coef, c->p_lm, (u32)K);
  }
  ConvBatch b{};
  b.matrix = c->conv_matrix;
  b.n_jobs = 1;
  b.job[0] = c->p2q_job;
  b.job[0].nc = (u32)level;
  b.t_stride = K * N;
  b.out_stride = level * N;
  // (large launches of N = 2^16: conversion and strided pass of the transform in one kernel)
  const bool strided_done = is_ntt && launch_baseconv_fwd_strided(c->stream, c->d, y, t, b, (u32)np);
  if (!strided_done) launch_baseconv(c->stream, c->d, y, t, b, (u32)np);
  if (is_ntt) {
    PolySeq ys = seq_strided(y, level * N);
    bool fits = true;  // index tables of another make go through the separate tail, which takes any table
    if (orders && c->d.logN > 12)
      for (u32 k = 0; k < orders->n; ++k) fits = fits && c->order_fits_chunks(orders->p[k]);
    if (c->d.logN > 12 && fits) {  // the tail, and with `orders` the automorphism, ride on the transform's last kernel
      FwdFuse f{};
      f.epi = 1;
      if (orders) f.orders = *orders;
      f.out = res;
      f.src = src;
      f.addend = addend_mode ? *addend : res;
      f.addend_mode = addend_mode;
      f.cst = c->pinv;
      if (!launch_ntt(c->stream, c->d, ys, ys, c->q_lm, nullptr, (u32)level, (u32)np, false, nullptr,
                      strided_done ? 2 : 3, &f))
        throw std::runtime_error("internal: fused Mod_down transform rejected");
      c->ws_used = mark;
      return;
    }
    launch_ntt(c->stream, c->d, ys, ys, c->q_lm, nullptr, (u32)level, (u32)np, false, nullptr, strided_done ? 2 : 3);
  }
  launch_moddown_tail(c->stream, c->d, res, src, y, level * N, addend_mode ? addend : nullptr, addend_mode, c->pinv,
                      c->q_lm, (u32)level, (u32)np, orders);
  c->ws_used = mark;
}

// Rescale (rns_poly.c:310-404) of np polynomials
void do_rescale(ace_ctx* c, const PolySeq& res, const PolySeq& src, size_t np, size_t level, bool is_ntt) {
  const size_t N = c->h.N;
  const RescaleDev& r = c->rescale_at(level);
  if (!is_ntt) {
    for (size_t p = 0; p < np; ++p)
      launch_rescale_coef(c->stream, c->d, res.at((u32)p), src.at((u32)p), src.at((u32)p) + (level - 1) * N, r.tail,
                          c->q_lm, (u32)(level - 1));
    return;
  }
  size_t mark = c->ws_used;
  u64* last = c->take(np * N);
  u64* u = c->take(np * (level - 1) * N);
  LimbMap one{};
  one.prime[0] = (uint8_t)(level - 1);
  PolySeq ls = seq_strided(last, N), us = seq_strided(u, (level - 1) * N);
  // the inverse transform reads the last limb where it lies
  launch_ntt(c->stream, c->d, ls, shifted(src, (level - 1) * N), one, nullptr, 1, (u32)np, true, nullptr);
  if (c->d.logN > 12) {  // modulus switch and tail ride on the transform's first and last kernels
    FwdFuse f{};
    f.pro = 1;
    f.last = last;
    f.last_stride = N;
    f.last_prime = (u32)(level - 1);
    f.sw = r.sw;
    f.epi = 2;
    f.out = res;
    f.src = src;
    f.addend = res;
    f.cst = r.tail;
    if (!launch_ntt(c->stream, c->d, us, us, c->q_lm, nullptr, (u32)(level - 1), (u32)np, false, nullptr, 3, &f))
      throw std::runtime_error("internal: fused Rescale transform rejected");
    c->ws_used = mark;
    return;
  }
  launch_rescale_switch(c->stream, c->d, u, (level - 1) * N, last, N, (u32)(level - 1), r.sw, c->q_lm,
                        (u32)(level - 1), (u32)np);
  launch_ntt(c->stream, c->d, us, us, c->q_lm, nullptr, (u32)(level - 1), (u32)np, false, nullptr);
  launch_rescale_tail(c->stream, c->d, res, src, u, (level - 1) * N, r.tail, c->q_lm, (u32)(level - 1), (u32)np);
  c->ws_used = mark;
}

// Shared front of Mod_down_rescale and Reduce_and_rescale_modup: poly (level+K
// limbs) goes to coefficient form in place, y = its P part in the Q basis
// (level limbs), x = the fused Mod_down + rescale value (level-1 limbs,
// coefficient form); last_out, when given, receives the reduced last limb.
void do_moddown_rescale_core(ace_ctx* c, u64* x, u64* y, u64* last_out, u64* poly, size_t level, bool is_ntt) {
  const size_t N = c->h.N, K = c->h.K;
  if (is_ntt) {
    LimbMap lm = poly_lm(c, level, true);
    PolySeq ps = seq_strided(poly, 0);
    launch_ntt(c->stream, c->d, ps, ps, lm, nullptr, (u32)(level + K), 1, true, nullptr);
  }
  size_t mark = c->ws_used;
  u64* t = c->take(K * N);
  launch_mul_const(c->stream, c->d, t, poly + level * N, c->pscale_coef, c->p_lm, (u32)K);
  ConvBatch b{};
  b.matrix = c->conv_matrix;
  b.n_jobs = 1;
  b.job[0] = c->p2q_job;
  b.job[0].nc = (u32)level;
  launch_baseconv(c->stream, c->d, y, t, b, 1);
  const RescaleDev& r = c->rescale_at(level);
  launch_moddown_rescale(c->stream, c->d, x, poly, y, last_out, c->pinv, r.tail, (u32)level);
  c->ws_used = mark;
}

// key limb positions of a polynomial viewed at `level` (Derive_poly, rns_poly.c:701-707)
LimbMap key_pos(const ace_ctx* c, size_t level) {
  LimbMap kp{};
  for (size_t t = 0; t < level; ++t) kp.prime[t] = (uint8_t)t;
  for (size_t j = 0; j < c->h.K; ++j) kp.prime[level + j] = (uint8_t)(c->h.L + j);
  return kp;
}

// Fast_switch_key (evaluator.c:411-462) for nb operands.  Operand o reads the
// digits at digits + o*digits_op_stride (0: all share one set) and key
// keys.p[o] (or keys.p[0] when keys.n == 1); its two results are polynomials
// 2o and 2o+1 of `out`.  The addend, and with `orders` the automorphism of
// operand o (table o), are fused into the Mod_down tail.
void do_switch_key(ace_ctx* c, const PolySeq& out, const u64* digits, u64 digits_op_stride, const KeySet& keys,
                   size_t nb, size_t level, const PolySeq* addend, int addend_mode, const OrderSet* orders = nullptr,
                   const OwnLimbs* own = nullptr) {
  const size_t N = c->h.N, T = level + c->h.K, kpoly = (c->h.L + c->h.K) * N, nd = c->h.num_decomp(level);
  size_t mark = c->ws_used;
  u64* e = c->take(nb * 2 * T * N);  // [operand][b|a][T limbs]
  LimbMap lm = poly_lm(c, level, true), kp = key_pos(c, level);
  launch_dotprod(c->stream, c->d, e, e + T * N, 2 * T * N, digits, T * N, digits_op_stride, keys, kpoly, 2 * kpoly,
                 (u32)nd, lm, kp, (u32)T, (u32)nb, own);
  do_mod_down(c, out, seq_strided(e, T * N), 2 * nb, level, true, addend, addend_mode, orders);
  c->ws_used = mark;
}

KeySet one_key(const u64* swk);
// Fast_switch_key with the addend, followed by Rescale_ciphertext (evaluator.c:411-462, 342-362), for nb operands on
// a ring of more than 4096 coefficients: results 2o and 2o+1 of `out` (level - 1 limbs) are
// Rescale(Mod_down(inner product of operand o) + addend.at(2o), .at(2o+1)).  Mod_down ends and Rescale begins with a
// forward transform over the same limbs; the transform is linear modulo each prime, so one transform of
// w = -(conv * (P q_l)^-1 + Switch_modulus(last) * q_l^-1) serves both: out_t = e'_t * (P q_l)^-1 + NTT(w)_t with
// e' = inner product + P * addend (the inner product kernel adds the lifted addend) and conv the P part of e'
// converted to the Q basis (the factor -(P q_l)^-1 is folded into the conversion's matrix).  The dropped limb's
// coefficient form, which Rescale switches to the other primes, is INTT(e'_last) * P^-1 - conv_last * P^-1: the
// inverse transform that serves the P limbs takes that limb along.
// Every step is exact modulo its prime and Switch_modulus sees the same canonical word, so the results are the words
// of do_switch_key followed by do_rescale.
// Rescale(Mod_down(e_p)) for np polynomials of the extended basis (es.at(p): level + K limbs, NTT form) through the one
// forward transform described above; twice: Rescale(2 Mod_down(e_p)).  Scratch from the arena.
// constant: `level` residues of an integer C that is added to polynomial 0 as a constant polynomial before the Rescale
// (Add_const between the Mod_down and the Rescale: every word of limb t in NTT form + C mod q_t), or null:
// Rescale(Mod_down(e_0) [* 2] + C).  Only coefficient 0 of the sum's coefficient form differs, so the dropped limb's
// coefficient 0 gets C mod q_l before it is switched to the other primes (half of it where the kernel doubles
// afterwards: the primes are odd), and every word of limb t of the result gets (C mod q_t) * q_l^-1.
void do_moddown_rescale_shared(ace_ctx* c, const PolySeq& out, const PolySeq& es, size_t np, size_t level, bool twice,
                               const u64* constant = nullptr) {
  const size_t N = c->h.N, K = c->h.K;
  const ModDownRescaleDev& m = c->moddown_rescale_at(level);
  const RescaleDev& r = c->rescale_at(level);
  size_t mark = c->ws_used;
  u64* t = c->take(np * (K + 1) * N);  // per polynomial: the dropped limb's z, then the scaled P limbs
  u64* y = c->take(np * level * N);
  launch_ntt(c->stream, c->d, seq_strided(t, (K + 1) * N), shifted(es, (level - 1) * N), m.inv_lm, nullptr,
             (u32)(K + 1), (u32)np, true, m.inv_scale);
  const u64 ql = c->h.primes[level - 1].q;
  if (constant) {
    LimbScalars s{};
    LimbMap last{};
    last.prime[0] = (u32)(level - 1);
    const u64 cl = constant[level - 1];
    s.v[0] = !twice ? cl : (cl & 1) ? (cl + ql) >> 1 : cl >> 1;  // C / 2 modulo the odd q_l (q_l < 2^63)
    launch_limb_scalars(c->stream, c->d, false, t, t, s, last, 1, 1);  // one word: z[0] of polynomial 0
  }
  ConvBatch b{};
  b.matrix = c->conv_matrix;
  b.n_jobs = 1;
  b.job[0] = m.job;
  b.t_stride = (K + 1) * N;
  b.out_stride = level * N;
  FwdFuse f{};
  f.pro = 2;
  f.last_prime = (u32)(level - 1);
  f.sw = r.sw;
  f.z = t;
  f.z_stride = (K + 1) * N;
  f.ylast = y + (level - 1) * N;
  f.ylast_stride = level * N;
  f.epi = 2;
  f.out = out;
  f.src = es;
  f.addend = out;
  f.cst = m.tail;
  f.twice = twice ? 1u : 0u;  // Rescale(2 (Mod_down(e) + d)): see FwdFuse
  PolySeq ys = seq_strided(y, level * N);
  // (large launches of N = 2^16: conversion, prologue and strided pass of the transform in one kernel)
  const bool strided_done = launch_baseconv_fwd_strided(c->stream, c->d, y, t + N, b, (u32)np, &f);
  if (!strided_done) launch_baseconv(c->stream, c->d, y, t + N, b, (u32)np);
  if (!launch_ntt(c->stream, c->d, ys, ys, c->q_lm, nullptr, (u32)(level - 1), (u32)np, false, nullptr,
                  strided_done ? 2 : 3, &f))
    throw std::runtime_error("internal: fused Mod_down + Rescale transform rejected");
  if (constant) {
    LimbScalars s{};
    for (size_t i = 0; i + 1 < level; ++i) {
      const u64 q = c->h.primes[i].q;
      s.v[i] = mul_mod(constant[i], m.ql_inv[i], q);
    }
    u64* o = const_cast<u64*>(out.at(0));
    launch_limb_scalars(c->stream, c->d, false, o, o, s, poly_lm(c, level - 1, false), (u32)(level - 1), N);
  }
  c->ws_used = mark;
}

void do_switch_key_rescale(ace_ctx* c, const PolySeq& out, const u64* digits, u64 digits_op_stride, const u64* swk,
                           size_t nb, size_t level, const Lift& lift, const OwnLimbs* own, bool twice = false,
                           const u64* constant = nullptr) {
  const size_t N = c->h.N, K = c->h.K, T = level + K, kpoly = (c->h.L + K) * N, nd = c->h.num_decomp(level);
  const size_t np = 2 * nb;
  size_t mark = c->ws_used;
  u64* e = c->take(np * T * N);  // [operand][b|a][T limbs], the addend lifted in
  LimbMap lm = poly_lm(c, level, true), kp = key_pos(c, level);
  launch_dotprod(c->stream, c->d, e, e + T * N, 2 * T * N, digits, T * N, digits_op_stride, one_key(swk), kpoly,
                 2 * kpoly, (u32)nd, lm, kp, (u32)T, (u32)nb, own, &lift);
  do_moddown_rescale_shared(c, out, seq_strided(e, T * N), np, level, twice, constant);
  c->ws_used = mark;
}

KeySet one_key(const u64* swk) {
  KeySet k{};
  k.n = 1;
  k.p[0] = swk;
  return k;
}

// Mul_ciphertext + Rescale_ciphertext for nb ciphertext pairs (evaluator.c:142-190, 342-362)
// twice: the relinearised product is added to itself before the Rescale (Add_ciph between the two)
// constant (nb == 1): `level` residues of an integer added to c0 as a constant polynomial after that (Add_const)
void do_mul_relin_rescale(ace_ctx* c, u64* r0, u64* r1, u64 out_stride, const u64* a0, const u64* a1, const u64* b0,
                          const u64* b1, u64 in_stride, const u64* swk, size_t nb, size_t level, bool twice = false,
                          const u64* constant = nullptr) {
  const size_t N = c->h.N, nd = c->h.num_decomp(level), T = level + c->h.K;
  // where the inner product can read the digits' own limbs from d2 itself, Mod_up does not copy them
  const bool from_d2 = c->d.logN > 12 && dotprod_reads_own(1, (u32)nb, true, (u32)nd);
  const bool shared = c->d.logN > 12 && level >= 2 && c->share_transform;
  // the same kernel can form the first two terms of the tensor product where it adds them, lifted, to its sums:
  // they are then neither written nor read back
  const bool on_the_way = shared && from_d2;
  u64* d01 = on_the_way ? nullptr : c->take(nb * 2 * level * N);  // [operand][c0|c1][level limbs]
  u64* d2 = c->take(nb * level * N);
  u64* digits = c->take(nb * nd * T * N);
  // With the terms formed on the way, d2 = a1 b1 need not exist in NTT form either where every limb's sums have room
  // for the lifted terms (the inner product then has a1 and b1 at hand for the digits' own limbs) and the inverse
  // transform that starts Mod_up can multiply as it reads (large launches of FP64-capable limbs).
  bool product_on_load = on_the_way && c->product_on_load;
  for (size_t t = 0; t < level && product_on_load; ++t) {
    const uint32_t shift = c->h.primes[t].shift;
    product_on_load = (shift >= 60 ? 4u : shift == 59 ? 8u : 16u) >= nd + 2;  // sum_terms of the kernel
  }
  if (product_on_load) product_on_load = do_precomp(c, digits, nd * T * N, a1, in_stride, nb, level, true, true, b1);
  if (!product_on_load) {
    launch_tensor(c->stream, c->d, d01, d01 ? d01 + level * N : nullptr, d2, a0, a1, b0, b1, c->q_lm, (u32)level,
                  (u32)nb, 2 * level * N, level * N, in_stride);
    do_precomp(c, digits, nd * T * N, d2, level * N, nb, level, true, from_d2);
  }
  const OwnLimbs own = product_on_load ? OwnLimbs{nullptr, 0, (u32)c->h.part_size, (u32)level, 1}
                                       : OwnLimbs{d2, (u64)(level * N), (u32)c->h.part_size, (u32)level, 0};
  PolySeq ds = seq_strided(d01 ? d01 : d2, level * N);  // (never read when the terms are formed on the way)
  if (shared) {
    Lift lift{ds, c->pmodq, (u32)level, nullptr, nullptr, nullptr, nullptr, 0};
    if (on_the_way) lift.a0 = a0, lift.a1 = a1, lift.b0 = b0, lift.b1 = b1, lift.in_stride = in_stride;
    do_switch_key_rescale(c, seq_pair(r0, r1, out_stride), digits, nd * T * N, swk, nb, level, lift,
                          from_d2 ? &own : nullptr, twice, constant);
    return;
  }
  do_switch_key(c, ds, digits, nd * T * N, one_key(swk), nb, level, &ds, 1, nullptr,
                from_d2 ? &own : nullptr);  // relinearised ct replaces d0, d1
  if (twice)
    for (size_t p = 0; p < 2 * nb; ++p)
      launch_ew(c->stream, c->d, EW_ADD, d01 + p * level * N, d01 + p * level * N, d01 + p * level * N, 0, c->q_lm,
                (u32)level, N);
  if (constant) {
    LimbScalars sc{};
    for (size_t t = 0; t < level; ++t) sc.v[t] = constant[t];
    launch_limb_scalars(c->stream, c->d, false, d01, d01, sc, poly_lm(c, level, false), (u32)level, N);
  }
  do_rescale(c, seq_pair(r0, r1, out_stride), ds, 2 * nb, level, true);
}

}  // namespace

static void run_poly_op(ace_ctx* c, int kind, const PolySeq& res, const PolySeq& src, size_t np, size_t level,
                        bool is_ntt) {
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  if (kind == 1) do_mod_down(c, res, src, np, level, is_ntt, nullptr, 0);
  else do_rescale(c, res, src, np, level, is_ntt);
}

void ace_ctx::flush_poly() {
  if (!ppoly.kind) return;
  const PendingPoly o = ppoly;
  ppoly.kind = 0;
  run_poly_op(this, o.kind, seq_strided(o.res, 0), seq_strided(const_cast<u64*>(o.src), 0), 1, o.level, o.is_ntt);
}

void ace_ctx::submit_poly(int kind, u64* res, const u64* src, size_t level, bool is_ntt) {
  const size_t N = h.N;
  const size_t res_words = (kind == 1 ? level : level - 1) * N, src_words = (kind == 1 ? level + h.K : level) * N;
  auto overlap = [](const u64* a, size_t na, const u64* b, size_t nb) { return a < b + nb && b < a + na; };
  if (ppoly.kind == kind && ppoly.level == level && ppoly.is_ntt == is_ntt &&
      !overlap(res, res_words, ppoly.res, res_words) && !overlap(res, res_words, ppoly.src, src_words) &&
      !overlap(src, src_words, ppoly.res, res_words)) {
    const PendingPoly o = ppoly;
    ppoly.kind = 0;
    run_poly_op(this, kind, seq_pair(o.res, res, 0), seq_pair(const_cast<u64*>(o.src), const_cast<u64*>(src), 0), 2,
                level, is_ntt);
    return;
  }
  flush_poly();
  if (!batching) {
    run_poly_op(this, kind, seq_strided(res, 0), seq_strided(const_cast<u64*>(src), 0), 1, level, is_ntt);
    return;
  }
  ppoly.kind = kind;
  ppoly.res = res;
  ppoly.src = src;
  ppoly.level = level;
  ppoly.is_ntt = is_ntt;
}


// ===========================================================================
// ACE_HIP_PROFILE=1: host time spent inside each entry point, printed when the process ends
namespace {
struct HostProf {
  bool on = false;
  std::map<std::string, std::pair<u64, double>> t;
  HostProf() {
    const char* e = std::getenv("ACE_HIP_PROFILE");
    on = e && std::atoi(e) != 0;
  }
  ~HostProf() {
    if (!on) return;
    std::vector<std::pair<double, std::string>> v;
    for (auto& kv : t) v.push_back({kv.second.second, kv.first});
    std::sort(v.rbegin(), v.rend());
    std::fprintf(stderr, "[ace_hip] host time by entry point\n");
    for (auto& e : v) std::fprintf(stderr, "  %-28s %9llu calls %9.1f ms\n", e.second.c_str(), (unsigned long long)t[e.second].first, e.first * 1e3);
  }
};
HostProf g_prof;

// ACE_HIP_CENSUS=<file>: how often each entry point was called with which size, written when the process ends as
// lines "<entry point> <a> <b> <calls>" (a: level or number of limbs, b: a second size such as the number of
// operands; 0 where there is none).  For cost models of a whole program on other machines (bench.py's estimate of
// the reference's CPU time): the counts, not this library's times, are what such a model needs.
struct Census {
  bool on = false;
  std::string path;
  std::mutex mu;
  std::map<std::tuple<std::string, size_t, size_t>, unsigned long long> n;
  Census() {
    const char* e = std::getenv("ACE_HIP_CENSUS");
    if (e && *e) on = true, path = e;
  }
  void add(const char* name, size_t a, size_t b) {
    std::lock_guard<std::mutex> lock(mu);
    ++n[std::make_tuple(std::string(name), a, b)];
  }
  void write(const std::string& to) {
    if (FILE* f = std::fopen(to.c_str(), "w")) {
      for (auto& kv : n)
        std::fprintf(f, "%s %zu %zu %llu\n", std::get<0>(kv.first).c_str(), std::get<1>(kv.first), std::get<2>(kv.first), kv.second);
      std::fclose(f);
    }
  }
  ~Census() {
    if (!on) return;
    if (FILE* f = std::fopen(path.c_str(), "w")) {
      for (auto& kv : n)
        std::fprintf(f, "%s %zu %zu %llu\n", std::get<0>(kv.first).c_str(), std::get<1>(kv.first), std::get<2>(kv.first), kv.second);
      std::fclose(f);
    }
  }
};
Census g_census;
#define CENSUS_AS(name, a, b) do { if (g_census.on) g_census.add(name, (size_t)(a), (size_t)(b)); } while (0)
#define CENSUS(a, b) CENSUS_AS(__func__, a, b)
struct ScopedProf {
  const char* name;
  timespec t0;
  explicit ScopedProf(const char* n) : name(n) {
    if (g_prof.on) clock_gettime(CLOCK_MONOTONIC, &t0);
  }
  ~ScopedProf() {
    if (!g_prof.on) return;
    timespec t1;
    clock_gettime(CLOCK_MONOTONIC, &t1);
    static std::mutex mu;  // contexts of a family run on several threads
    std::lock_guard<std::mutex> lock(mu);
    auto& e = g_prof.t[name];
    e.first += 1;
    e.second += (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
  }
};
}  // namespace

extern "C" {

#define ACE_TRY_BARE ScopedProf prof_scope_(__func__); try {                                                     \
  if (!c) return fail("null context");                                         \
  if (!c->device_ok) return fail("no HIP device: this context holds host tables only");
#define ACE_TRY_KEEP_RUN ACE_TRY_BARE c->flush_poly();
#define ACE_TRY ACE_TRY_BARE c->flush_pending();
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
  ace_ctx* c = make_ctx(degree, q, num_parts);
  if (c) {
    c->q0_bits = q0_bits;
    c->sf_bits = sf_bits;
  }
  return c;
}

ace_ctx* ace_ctx_create_with_primes(uint32_t degree, size_t num_q, const int64_t* q_primes, size_t num_parts) {
  if (!q_primes || num_q == 0 || num_parts == 0) {
    g_err = "ace_ctx_create_with_primes: invalid parameters";
    return nullptr;
  }
  return make_ctx(degree, std::vector<i64>(q_primes, q_primes + num_q), num_parts);
}

ace_ctx* ace_ctx_share(ace_ctx* from) {
  try {
    if (!from) throw std::runtime_error("ace_ctx_share: null context");
    if (!from->device_ok) throw std::runtime_error("ace_ctx_share: the context holds host tables only (no HIP device)");
    ace_ctx* root = from->parent ? from->parent : from;
    std::unique_ptr<ace_ctx> c(new ace_ctx(root));
    c->init_shared(*root);
    c->device_ok = true;
    return c.release();
  } catch (const std::exception& e) {
    g_err = e.what();
    return nullptr;
  }
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
// Buffers handed back by ace_free are kept, by size, for the next ace_alloc of
// that size: programs allocate and free the same few polynomial shapes in a
// loop, and hipMalloc / hipFree cost far more than the kernels between them.
// Reuse is safe without a wait because every use of a buffer is ordered on
// the context's one stream.
static int64_t* alloc_words(ace_ctx* c, size_t n_words, bool zero);
int64_t* ace_alloc(ace_ctx* c, size_t n_words) { return alloc_words(c, n_words, true); }
int64_t* ace_alloc_uninit(ace_ctx* c, size_t n_words) { return alloc_words(c, n_words, false); }
static int64_t* alloc_words(ace_ctx* c, size_t n_words, bool zero) {
  ScopedProf prof_scope_("ace_alloc");
  try {
    if (!c || !c->device_ok) throw std::runtime_error("no HIP device: this context holds host tables only");
    const size_t words = std::max<size_t>(n_words, 1);
    u64* p = nullptr;
    auto it = c->pool.find(words);
    if (it != c->pool.end()) {
      p = static_cast<u64*>(it->second);
      c->pool.erase(it);
      c->pooled_words -= words;
      c->family->pooled_words -= words;
    } else {
      hipError_t e = hipMalloc((void**)&p, words * sizeof(u64));
      if (e != hipSuccess && c->pooled_words) {  // give the cached buffers back and try once more
        (void)hipGetLastError();
        c->flush_pending();  // recorded calls may name buffers of the pool
        c->drop_pool();
        e = hipMalloc((void**)&p, words * sizeof(u64));
      }
      HIP_OK(e);
    }
    {
      std::lock_guard<std::mutex> lock(c->family->mu);
      c->live[p] = words;
    }
    if (zero) {
      const size_t N = c->h.N;
      if (c->batching && n_words % N == 0 && n_words / N <= 64) {  // as entries of one limb each, next to the calls that follow
        for (size_t t = 0; t < n_words / N; ++t) c->run_append(BatchOp{p + t * N, nullptr, nullptr, 0, (u32)BATCH_ZERO, 0}, N);
      } else {
        launch_fill_zero(c->stream, p, n_words);
      }
    }
    return reinterpret_cast<int64_t*>(p);
  } catch (const std::exception& e) {
    g_err = e.what();
    return nullptr;
  }
}
void ace_free(ace_ctx* c, int64_t* p) {
  ScopedProf prof_scope_("ace_free");
  if (!p || !c || !c->device_ok) return;
  size_t words = 0;
  {
    std::lock_guard<std::mutex> lock(c->family->mu);
    auto it = c->live.find(p);
    if (it == c->live.end()) return;  // not from ace_alloc of this family (a view, or freed twice)
    words = it->second;
  }
  c->forget_orders(p, words);
  const bool keep = c->family->pooled_words.load() + words <= c->family->pool_limit_words;
  try {
    // A pending Mod_down / Rescale may read the buffer: it goes out now.  Recorded calls that name the buffer may
    // stay recorded where the buffer stays mapped (in this lane's pool): whoever is handed it next is served on the
    // same stream, and entries that are recorded for it later join the chain of those that name it now (the
    // ranges are the same: the pool hands a buffer out for the size it was made for).  A zero fill of the buffer
    // that nothing has looked at is moot.
    c->flush_poly();
    if (keep) c->drop_untouched_fills(p, words);
    else c->flush_run();
  } catch (const std::exception& e) {
    (void)fail(e.what());
  }
  {
    std::lock_guard<std::mutex> lock(c->family->mu);
    c->live.erase(p);
  }
  if (keep) {
    c->pool.emplace(words, p);
    c->pooled_words += words;
    c->family->pooled_words += words;
    return;
  }
  (void)hipStreamSynchronize(c->stream);
  (void)hipFree(p);
}
// copies and fills longer than this go to the copy engine's / the fill kernel's own launch: a recorded entry moves
// one word per thread, which is right for a limb and slow for a whole batch
static constexpr size_t kRecordedWords = (size_t)1 << 22;
int ace_upload(ace_ctx* c, int64_t* dst, const int64_t* src, size_t n) {
  ACE_TRY
  c->forget_orders(dst, n);
  HIP_OK(hipMemcpyAsync(dst, src, n * sizeof(u64), hipMemcpyHostToDevice, c->stream));
  HIP_OK(hipStreamSynchronize(c->stream));
  ACE_CATCH_INT
}
int ace_download(ace_ctx* c, int64_t* dst, const int64_t* src, size_t n) {
  ACE_TRY
  HIP_OK(hipMemcpyAsync(dst, src, n * sizeof(u64), hipMemcpyDeviceToHost, c->stream));
  c->check_deferred();
  ACE_CATCH_INT
}
int ace_copy(ace_ctx* c, int64_t* dst, const int64_t* src, size_t n) {
  ACE_TRY_KEEP_RUN
  CENSUS(n, 0);
  if (!dst || !src) return fail("ace_copy: null argument");
  if (dst == src || n == 0) return 0;
  c->forget_orders(dst, n);
  if (c->batching && n <= kRecordedWords) {  // a copy is an elementwise entry like any other
    // whole limbs go in limb by limb, so that they join the limb-sized calls around them in one run
    const size_t N = c->h.N, pieces = (n % N == 0 && n / N <= 64) ? n / N : 1, each = n / pieces;
    for (size_t t = 0; t < pieces; ++t)
      c->run_append(BatchOp{U(dst) + t * each, U(src) + t * each, nullptr, 0, (u32)BATCH_COPY, 0}, each);
    return 0;
  }
  c->flush_run();
  HIP_OK(hipMemcpyAsync(dst, src, n * sizeof(u64), hipMemcpyDeviceToDevice, c->stream));
  ACE_CATCH_INT
}
int ace_zero(ace_ctx* c, int64_t* dst, size_t n) {
  ACE_TRY_KEEP_RUN
  CENSUS(n, 0);
  if (!dst) return fail("ace_zero: null argument");
  if (n == 0) return 0;
  c->forget_orders(dst, n);
  if (c->batching && n <= kRecordedWords) {
    const size_t N = c->h.N, pieces = (n % N == 0 && n / N <= 64) ? n / N : 1, each = n / pieces;
    for (size_t t = 0; t < pieces; ++t)
      c->run_append(BatchOp{U(dst) + t * each, nullptr, nullptr, 0, (u32)BATCH_ZERO, 0}, each);
    return 0;
  }
  c->flush_run();
  launch_fill_zero(c->stream, U(dst), n);
  ACE_CATCH_INT
}
int ace_sync(ace_ctx* c) {
  ACE_TRY
  c->check_deferred();
  ACE_CATCH_INT
}
int ace_sync_device(ace_ctx* c) {
  ACE_TRY_BARE
  HIP_OK(hipDeviceSynchronize());
  ACE_CATCH_INT
}
// ---- two lanes ------------------------------------------------------------------
int ace_fork(ace_ctx* c) {
  ACE_TRY
  if (c->fork_state) return fail("ace_fork: the context is forked already");
  if (!c->idle.stream) {
    HIP_OK(hipStreamCreateWithFlags(&c->idle.stream, hipStreamNonBlocking));
    HIP_OK(hipEventCreateWithFlags(&c->fork_ev, hipEventDisableTiming));
    HIP_OK(hipEventCreateWithFlags(&c->join_ev, hipEventDisableTiming));
  }
  HIP_OK(hipEventRecord(c->fork_ev, c->stream));
  c->swap_lanes();
  HIP_OK(hipStreamWaitEvent(c->stream, c->fork_ev, 0));
  c->fork_state = 1;
  ACE_CATCH_INT
}
int ace_fork_switch(ace_ctx* c) {
  ACE_TRY  // launches what is still recorded, on the second lane
  if (c->fork_state != 1) return fail("ace_fork_switch: not on the second lane");
  HIP_OK(hipEventRecord(c->join_ev, c->stream));
  c->swap_lanes();
  c->fork_state = 2;
  ACE_CATCH_INT
}
int ace_join(ace_ctx* c) {
  ACE_TRY
  if (c->fork_state == 1) {
    HIP_OK(hipEventRecord(c->join_ev, c->stream));
    c->swap_lanes();
    c->fork_state = 2;
  }
  if (c->fork_state != 2) return fail("ace_join: the context is not forked");
  HIP_OK(hipStreamWaitEvent(c->stream, c->join_ev, 0));
  c->fork_state = 0;
  ACE_CATCH_INT
}

int ace_fork_release(ace_ctx* c) {
  ACE_TRY
  if (c->fork_state) return fail("ace_fork_release: the context is forked");
  if (c->idle.stream) {
    HIP_OK(hipStreamSynchronize(c->idle.stream));
    for (auto& kv : c->idle.pool) (void)hipFree(kv.second);
    c->idle.pool.clear();
    c->family->pooled_words -= c->idle.pooled_words;
    c->idle.pooled_words = 0;
    if (c->idle.ws) (void)hipFree(c->idle.ws);
    c->idle.ws = nullptr;
    c->idle.ws_words = c->idle.ws_used = 0;
    HIP_OK(hipStreamDestroy(c->idle.stream));
    c->idle.stream = nullptr;
    HIP_OK(hipEventDestroy(c->fork_ev));
    HIP_OK(hipEventDestroy(c->join_ev));
    c->fork_ev = c->join_ev = nullptr;
    // (the second lane's image of recorded runs, if any, stays with the context's other allocations)
  }
  ACE_CATCH_INT
}

void ace_census_mark(const char* label) {
  if (!g_census.on || !label) return;
  std::lock_guard<std::mutex> lock(g_census.mu);
  g_census.write(g_census.path + "." + label);
  g_census.n.clear();
}

void ace_memory_stats(const ace_ctx* c, size_t out[4]) {
  out[0] = c->ws_words;
  out[1] = c->pooled_words;
  {
    std::lock_guard<std::mutex> lock(c->family->mu);
    out[2] = c->live.size();
  }
  out[3] = c->pool.size();
}
int ace_timer_start(ace_ctx* c) {
  ACE_TRY
  HIP_OK(hipEventRecord(c->ev0, c->stream));
  ACE_CATCH_INT
}
float ace_timer_stop_ms(ace_ctx* c) {
  try {
    if (!c || !c->device_ok) throw std::runtime_error("no HIP device");
    c->flush_pending();
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
  CENSUS_AS(inverse ? "ace_intt" : "ace_ntt", n_limbs * n_polys, 0);
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
  const u64 stride = (u64)stride_limbs * c->h.N;
  if (!launch_ntt(c->stream, c->d, seq_strided(U(dst), stride), seq_strided(U(src), stride), lm, nullptr,
                  (u32)n_limbs, (u32)n_polys, inverse, nullptr, passes))
    return fail("ace_ntt: ring degree above 2^17, or a polynomial that does not start on a 16-byte boundary");
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
  ACE_TRY_KEEP_RUN
  CENSUS_AS(op == EW_ADD || op == EW_SUB ? "hw_add" : op == EW_MUL ? "hw_mul" : op == EW_MULADD ? "hw_mac" : op == EW_ADD_S || op == EW_SUB_S ? "hw_add_scalar" : op == EW_MUL_S ? "hw_mul_scalar" : "hw_mac_scalar", n, 0);
  if (n == 0) return 0;
  if (!r || !a || (op < EW_ADD_S && !b)) return fail("ace_hw: null argument");
  if (pi >= c->h.L + c->h.K) return fail("ace_hw: prime index out of range");
  if ((op == EW_MUL_S || op == EW_MULADD_S) && (s < 0 || (u64)s >= c->h.primes[pi].q))
    return fail("ace_hw: scalar multiplier must be a residue in [0, q)");
  if (c->batching) {
    c->run_append(BatchOp{U(r), U(a), U(b), (u64)s, (u32)op, (u32)pi}, n);
    return 0;
  }
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
  ACE_TRY_KEEP_RUN
  CENSUS(n, 0);
  if (n == 0) return 0;
  if (!r || !a || !order) return fail("ace_hw_rotate: null argument");
  if (r == a) return fail("ace_hw_rotate: in-place gather is not supported");
  if (pi >= c->h.L + c->h.K) return fail("ace_hw_rotate: prime index out of range");
  if (c->batching) {
    c->run_append(BatchOp{U(r), U(a), reinterpret_cast<const u64*>(order), 0, (u32)BATCH_ROTATE, (u32)pi}, n);
    return 0;
  }
  LimbMap lm{};
  lm.prime[0] = (uint8_t)pi;
  launch_gather(c->stream, c->d, U(r), U(a), order, lm, 1, n);
  ACE_CATCH_INT
}

int ace_set_batching(ace_ctx* c, int on) {
  ACE_TRY
  c->batching = on != 0;
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
int ace_host_fft_tables(const ace_ctx* c, double* rou, uint32_t* rot) {
  if (!c || !rou || !rot) return fail("ace_host_fft_tables: null argument");
  std::vector<double> r;
  std::vector<u32> g;
  fft_tables(c->h.N, r, g);
  std::memcpy(rou, r.data(), r.size() * sizeof(double));
  std::memcpy(rot, g.data(), (c->h.N / 2 ? c->h.N / 2 : 1) * sizeof(u32));
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
  c->h2d(dev_order, ord.data(), ord.size() * sizeof(i64));
  HIP_OK(hipStreamSynchronize(c->stream));
  c->forget_orders(dev_order, c->h.N);
  if (is_ntt) c->note_order(dev_order, true);
  ACE_CATCH_INT
}

// ---- polynomial ops ---------------------------------------------------------------
static int poly_ew(ace_ctx* c, EwOp op, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p) {
  ACE_TRY_KEEP_RUN
  CENSUS_AS(op == EW_MUL ? "poly_mul" : "poly_add", level + (with_p ? c->h.K : 0), 0);
  if (!r || !a || !b) return fail("ace_poly: null argument");
  if (!level_ok(c, level)) return fail("ace_poly: level out of range");
  LimbMap lm = poly_lm(c, level, with_p != 0);
  const size_t n_limbs = level + (with_p ? c->h.K : 0), N = c->h.N;
  if (c->batching) {  // limb by limb into the recorded run: the sums and differences between two larger calls leave
                      // as one launch (a ciphertext sum is two of these calls, often with a constant added next)
    for (size_t t = 0; t < n_limbs; ++t)
      c->run_append(BatchOp{U(r) + t * N, U(a) + t * N, U(b) + t * N, 0, (u32)op, (u32)lm.prime[t]}, N);
    return 0;
  }
  launch_ew(c->stream, c->d, op, U(r), U(a), U(b), 0, lm, (u32)n_limbs, N);
  ACE_CATCH_INT
}
int ace_poly_add(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p) { return poly_ew(c, EW_ADD, r, a, b, level, with_p); }
int ace_poly_sub(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p) { return poly_ew(c, EW_SUB, r, a, b, level, with_p); }
int ace_poly_mul(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* b, size_t level, int with_p) { return poly_ew(c, EW_MUL, r, a, b, level, with_p); }

int ace_ext_plain_mac(ace_ctx* c, int64_t* r0, int64_t* r1, const int64_t* const* a0, const int64_t* const* a1,
                      const int64_t* const* plain, size_t count, size_t level, size_t plain_level, int accumulate) {
  ACE_TRY
  CENSUS(level, count);
  if (!r0 || !r1 || !a0 || !a1 || !plain) return fail("ace_ext_plain_mac: null argument");
  if (!level_ok(c, level) || !level_ok(c, plain_level) || plain_level < level)
    return fail("ace_ext_plain_mac: levels out of range (the plaintext may not sit below the ciphertext)");
  if (!count) return fail("ace_ext_plain_mac: no operands");
  for (size_t j = 0; j < count; ++j) {
    if (!a0[j] || !a1[j] || !plain[j]) return fail("ace_ext_plain_mac: null operand");
    if (a0[j] == r0 || a1[j] == r1 || a0[j] == r1 || a1[j] == r0) return fail("ace_ext_plain_mac: an operand aliases the result");
  }
  LimbMap lm = poly_lm(c, level, true);
  for (size_t done = 0; done < count; done += kMaxMacOps) {
    MacSet ops{};
    ops.n = (u32)std::min<size_t>(kMaxMacOps, count - done);
    for (u32 j = 0; j < ops.n; ++j) {
      ops.a0[j] = U(a0[done + j]);
      ops.a1[j] = U(a1[done + j]);
      ops.p[j]  = U(plain[done + j]);
    }
    launch_plain_mac(c->stream, c->d, U(r0), U(r1), ops, lm, (u32)(level + c->h.K), (u32)level, (u32)plain_level,
                     accumulate != 0 || done != 0, c->h.N);
  }
  ACE_CATCH_INT
}

int ace_ext_plain_mac_groups(ace_ctx* c, int64_t* const* r0, int64_t* const* r1, size_t n_groups,
                             const int64_t* const* a0, const int64_t* const* a1, size_t count,
                             const int64_t* const* plain, size_t level, size_t plain_level) {
  ACE_TRY
  if (g_census.on && plain) {  // the products actually formed
    size_t terms = 0;
    for (size_t k = 0; k < n_groups * count; ++k) terms += plain[k] != nullptr;
    CENSUS_AS("ace_ext_plain_mac", level, terms);
  }
  if (!r0 || !r1 || !a0 || !a1 || !plain) return fail("ace_ext_plain_mac_groups: null argument");
  if (!level_ok(c, level) || !level_ok(c, plain_level) || plain_level < level)
    return fail("ace_ext_plain_mac_groups: levels out of range (the plaintext may not sit below the ciphertext)");
  if (!count || !n_groups) return fail("ace_ext_plain_mac_groups: no operands");
  for (size_t g = 0; g < n_groups; ++g) {
    if (!r0[g] || !r1[g]) return fail("ace_ext_plain_mac_groups: null result");
    for (size_t h = 0; h < n_groups; ++h)
      if (r0[g] == r1[h] || (g != h && (r0[g] == r0[h] || r1[g] == r1[h])))
        return fail("ace_ext_plain_mac_groups: two results share a buffer");
    for (size_t j = 0; j < count; ++j) {
      if (!a0[j] || !a1[j]) return fail("ace_ext_plain_mac_groups: null operand");
      if (a0[j] == r0[g] || a0[j] == r1[g] || a1[j] == r0[g] || a1[j] == r1[g])
        return fail("ace_ext_plain_mac_groups: an operand aliases a result");
    }
  }
  LimbMap lm = poly_lm(c, level, true);
  for (size_t g0 = 0; g0 < n_groups; g0 += kMacGroups) {
    for (size_t done = 0; done < count; done += kMacGroupOps) {
      MacGroups ops{};
      ops.n_groups = (u32)std::min<size_t>(kMacGroups, n_groups - g0);
      ops.n_ops = (u32)std::min<size_t>(kMacGroupOps, count - done);
      for (u32 g = 0; g < ops.n_groups; ++g) {
        ops.r0[g] = U(r0[g0 + g]);
        ops.r1[g] = U(r1[g0 + g]);
        for (u32 j = 0; j < ops.n_ops; ++j) ops.p[g][j] = U(plain[(g0 + g) * count + done + j]);
      }
      for (u32 j = 0; j < ops.n_ops; ++j) {
        ops.a0[j] = U(a0[done + j]);
        ops.a1[j] = U(a1[done + j]);
      }
      launch_plain_mac_groups(c->stream, c->d, ops, lm, (u32)(level + c->h.K), (u32)level, (u32)plain_level, done != 0,
                              c->h.N);
    }
  }
  ACE_CATCH_INT
}

static int poly_scalars(ace_ctx* c, bool mul, int64_t* r, const int64_t* a, const int64_t* scalars, size_t level) {
  ACE_TRY_KEEP_RUN
  CENSUS_AS(mul ? "poly_mul_scalars" : "poly_add_scalars", level, 0);
  if (!r || !a || !scalars) return fail("ace_poly_scalars: null argument");
  if (!level_ok(c, level)) return fail("ace_poly_scalars: level out of range");
  LimbScalars s{};
  for (size_t t = 0; t < level; ++t) {
    if (scalars[t] < 0 || (u64)scalars[t] >= c->h.primes[t].q) return fail("ace_poly_scalars: scalar is not a residue");
    s.v[t] = (u64)scalars[t];
  }
  if (c->batching) {  // (recorded like the sums above)
    const size_t N = c->h.N;
    for (size_t t = 0; t < level; ++t)
      c->run_append(BatchOp{U(r) + t * N, U(a) + t * N, nullptr, s.v[t], (u32)(mul ? EW_MUL_S : EW_ADD_S), (u32)t}, N);
    return 0;
  }
  launch_limb_scalars(c->stream, c->d, mul, U(r), U(a), s, poly_lm(c, level, false), (u32)level, c->h.N);
  ACE_CATCH_INT
}
int ace_poly_add_scalars(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* scalars, size_t level) { return poly_scalars(c, false, r, a, scalars, level); }
int ace_poly_mul_scalars(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* scalars, size_t level) { return poly_scalars(c, true, r, a, scalars, level); }

int ace_sample_uniform(ace_ctx* c, int64_t* res, size_t level, int with_p, uint64_t seed, uint64_t stream) {
  ACE_TRY
  if (!res) return fail("ace_sample_uniform: null argument");
  if (!level_ok(c, level)) return fail("ace_sample_uniform: level out of range");
  launch_sample_uniform(c->stream, c->d, U(res), seed, stream, poly_lm(c, level, with_p != 0),
                        (u32)(level + (with_p ? c->h.K : 0)), c->h.N);
  ACE_CATCH_INT
}
int ace_expand_small(ace_ctx* c, int64_t* res, const int64_t* small_host, size_t level, int with_p) {
  ACE_TRY
  if (!res || !small_host) return fail("ace_expand_small: null argument");
  if (!level_ok(c, level)) return fail("ace_expand_small: level out of range");
  for (size_t i = 0; i < c->h.N; ++i)
    if (small_host[i] > (1 << 30) || small_host[i] < -(1 << 30)) return fail("ace_expand_small: coefficient is not small");
  c->ensure_ws(c->h.N);
  c->ws_used = 0;
  u64* v = c->take(c->h.N);
  c->h2d(v, small_host, c->h.N * sizeof(i64));
  launch_expand_small(c->stream, c->d, U(res), reinterpret_cast<const i64*>(v), poly_lm(c, level, with_p != 0),
                      (u32)(level + (with_p ? c->h.K : 0)), c->h.N);
  ACE_CATCH_INT
}

int ace_ciph_wsum(ace_ctx* c, int64_t* r0, int64_t* r1, const int64_t* const* a0, const int64_t* const* a1,
                  const int64_t* weights, size_t count, size_t level) {
  ACE_TRY
  CENSUS(level, count);
  if (!r0 || !r1 || !a0 || !a1 || !weights) return fail("ace_ciph_wsum: null argument");
  if (!level_ok(c, level)) return fail("ace_ciph_wsum: level out of range");
  if (!count || count > kMaxMacOps) return fail("ace_ciph_wsum: between 1 and 32 terms");
  MacSet ops{};
  ops.n = (u32)count;
  for (size_t j = 0; j < count; ++j) {
    if (!a0[j] || !a1[j]) return fail("ace_ciph_wsum: null operand");
    ops.a0[j] = U(a0[j]);
    ops.a1[j] = U(a1[j]);
    for (size_t t = 0; t < level; ++t)
      if (weights[j * level + t] < 0 || (u64)weights[j * level + t] >= c->h.primes[t].q)
        return fail("ace_ciph_wsum: weight is not a residue");
  }
  c->ensure_ws(count * level);
  c->ws_used = 0;
  u64* w = c->take(count * level);
  c->h2d(w, weights, count * level * sizeof(u64));
  launch_wsum(c->stream, c->d, U(r0), U(r1), ops, w, poly_lm(c, level, false), (u32)level, c->h.N);
  ACE_CATCH_INT
}

int ace_poly_automorphism(ace_ctx* c, int64_t* r, const int64_t* a, const int64_t* order, size_t level, int with_p) {
  ACE_TRY
  CENSUS(level + (with_p ? c->h.K : 0), 0);
  if (!r || !a || !order) return fail("ace_poly_automorphism: null argument");
  if (r == a) return fail("ace_poly_automorphism: in-place gather is not supported");
  if (!level_ok(c, level)) return fail("ace_poly_automorphism: level out of range");
  LimbMap lm = poly_lm(c, level, with_p != 0);
  launch_gather(c->stream, c->d, U(r), U(a), order, lm, (u32)(level + (with_p ? c->h.K : 0)), c->h.N);
  ACE_CATCH_INT
}

int ace_decomp_modup(ace_ctx* c, int64_t* res, const int64_t* src, size_t level, size_t part, int is_ntt) {
  ACE_TRY_BARE
  CENSUS(level, part);
  if (!res || !src) return fail("ace_decomp_modup: null argument");
  if (!level_ok(c, level)) return fail("ace_decomp_modup: level out of range");
  if (part >= c->h.num_decomp(level)) return fail("ace_decomp_modup: digit index out of range");
  c->flush_pending_overwriting(res, (level + c->h.K) * (size_t)c->h.N, src, level * (size_t)c->h.N);
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_decomp_modup(c, U(res), U(src) + c->h.part_size * part * (size_t)c->h.N, level, part, is_ntt != 0);
  ACE_CATCH_INT
}

int ace_mod_up(ace_ctx* c, int64_t* res, const int64_t* digit, size_t level, size_t part, int is_ntt) {
  ACE_TRY_BARE
  CENSUS(level, part);
  if (!res || !digit) return fail("ace_mod_up: null argument");
  if (!level_ok(c, level)) return fail("ace_mod_up: level out of range");
  if (part >= c->h.num_decomp(level)) return fail("ace_mod_up: digit index out of range");
  c->flush_pending_overwriting(res, (level + c->h.K) * (size_t)c->h.N, digit, c->h.part_size * (size_t)c->h.N);
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_decomp_modup(c, U(res), U(digit), level, part, is_ntt != 0);
  ACE_CATCH_INT
}

int ace_precomp(ace_ctx* c, int64_t* res, const int64_t* src, size_t level, int is_ntt) {
  ACE_TRY_BARE
  CENSUS(level, 1);
  if (!res || !src) return fail("ace_precomp: null argument");
  if (!level_ok(c, level)) return fail("ace_precomp: level out of range");
  c->flush_pending_overwriting(res, c->h.num_decomp(level) * (level + c->h.K) * (size_t)c->h.N, src,
                               level * (size_t)c->h.N);
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_precomp(c, U(res), 0, U(src), 0, 1, level, is_ntt != 0);
  ACE_CATCH_INT
}

int ace_mod_down(ace_ctx* c, int64_t* res, const int64_t* src, size_t level, int is_ntt) {
  ACE_TRY_BARE
  CENSUS(level, 1);
  if (!res || !src) return fail("ace_mod_down: null argument");
  if (!level_ok(c, level)) return fail("ace_mod_down: level out of range");
  c->flush_pending_overwriting(res, level * (size_t)c->h.N, src, (level + c->h.K) * (size_t)c->h.N, true);
  c->submit_poly(1, U(res), U(src), level, is_ntt != 0);
  ACE_CATCH_INT
}

// Precomp / Mod_down of `count` polynomials at constant strides in one set of launches
static int batch_args_ok(const char* who, const void* res, size_t res_stride, size_t res_words, const void* src,
                         size_t src_stride, size_t src_words, size_t count) {
  if (!res || !src) return fail(std::string(who) + ": null argument");
  if (!count) return fail(std::string(who) + ": count is zero");
  if (count > 1 && (res_stride < res_words || src_stride < src_words))
    return fail(std::string(who) + ": a stride is shorter than the polynomial it steps over");
  const uintptr_t r0 = (uintptr_t)res, r1 = r0 + ((count - 1) * res_stride + res_words) * sizeof(u64);
  const uintptr_t s0 = (uintptr_t)src, s1 = s0 + ((count - 1) * src_stride + src_words) * sizeof(u64);
  if (r0 < s1 && s0 < r1) return fail(std::string(who) + ": results and operands overlap");
  return 0;
}

int ace_precomp_batch(ace_ctx* c, int64_t* res, size_t res_stride, const int64_t* src, size_t src_stride, size_t count,
                      size_t level, int is_ntt) {
  ACE_TRY_BARE
  CENSUS_AS("ace_precomp", level, count);
  if (!level_ok(c, level)) return fail("ace_precomp_batch: level out of range");
  const size_t N = c->h.N, res_words = c->h.num_decomp(level) * (level + c->h.K) * N, src_words = level * N;
  if (int rc = batch_args_ok("ace_precomp_batch", res, res_stride, res_words, src, src_stride, src_words, count)) return rc;
  // only a result range without gaps is overwritten as a whole
  if (res_stride == res_words || count == 1)
    c->flush_pending_overwriting(res, ((count - 1) * res_stride + res_words), src, (count - 1) * src_stride + src_words);
  else
    c->flush_pending();
  c->ensure_ws(c->std_ws(level) * count);
  c->ws_used = 0;
  do_precomp(c, U(res), res_stride, U(src), src_stride, count, level, is_ntt != 0);
  ACE_CATCH_INT
}

int ace_mod_down_batch(ace_ctx* c, int64_t* res, size_t res_stride, const int64_t* src, size_t src_stride, size_t count,
                       size_t level, int is_ntt) {
  ACE_TRY_BARE
  CENSUS_AS("ace_mod_down", level, count);
  if (!level_ok(c, level)) return fail("ace_mod_down_batch: level out of range");
  const size_t N = c->h.N, res_words = level * N, src_words = (level + c->h.K) * N;
  if (int rc = batch_args_ok("ace_mod_down_batch", res, res_stride, res_words, src, src_stride, src_words, count)) return rc;
  if (res_stride == res_words || count == 1)
    c->flush_pending_overwriting(res, ((count - 1) * res_stride + res_words), src, (count - 1) * src_stride + src_words);
  else
    c->flush_pending();
  c->ensure_ws(c->std_ws(level) * count);
  c->ws_used = 0;
  do_mod_down(c, seq_strided(U(res), res_stride), seq_strided(U(src), src_stride), count, level, is_ntt != 0, nullptr, 0);
  ACE_CATCH_INT
}

int ace_mod_down_noalloc(ace_ctx* c, int64_t* res, const int64_t* src, size_t level, int is_ntt) {
  ACE_TRY_BARE
  if (!res || !src) return fail("ace_mod_down_noalloc: null argument");
  if (!level_ok(c, level)) return fail("ace_mod_down_noalloc: level out of range");
  if (c->fork_state)  // both lanes would use the one static array
    return fail("ace_mod_down_noalloc: not between ace_fork and ace_join (the static scratch serves one stream)");
  const size_t need = (level + c->h.K) * (size_t)c->h.N;
  if (need > kStaticScratchWords)
    return fail("ace_mod_down_noalloc: (level + num_p) * degree = " + std::to_string(need) + " words exceeds the static "
                "scratch of " + std::to_string(kStaticScratchWords) + " words (16 MiB); use ace_mod_down");
  // Recorded calls that are pending go first, as before every entry point.  A short run travels as kernel
  // arguments; a longer one is staged through buffers that may have to be allocated, and a pending Mod_down or
  // Rescale takes its scratch from the arena, which may have to grow: those are refused here.
  if (c->ppoly.kind || c->run.ops.size() > kSmallRun)
    return fail("ace_mod_down_noalloc: more recorded calls are pending than can be launched without allocating; "
                "call ace_sync() first");
  c->flush_run();
  // the sequencer takes its intermediates from the arena: point the arena at the static array for this call
  struct ArenaSwap {
    ace_ctx* c;
    u64* ws;
    size_t words, used;
    ArenaSwap(ace_ctx* c_, u64* p, size_t n) : c(c_), ws(c_->ws), words(c_->ws_words), used(c_->ws_used) {
      c->ws = p;
      c->ws_words = n;
      c->ws_used = 0;
    }
    ~ArenaSwap() {
      c->ws = ws;
      c->ws_words = words;
      c->ws_used = used;
    }
  } swap(c, c->static_scratch, kStaticScratchWords);
  do_mod_down(c, seq_strided(U(res), 0), seq_strided(const_cast<u64*>(U(src)), 0), 1, level, is_ntt != 0, nullptr, 0);
  ACE_CATCH_INT
}

int ace_rescale(ace_ctx* c, int64_t* res, const int64_t* src, size_t level, int is_ntt) {
  ACE_TRY_BARE
  CENSUS(level, 1);
  if (!res || !src) return fail("ace_rescale: null argument");
  if (level < 2 || level > c->h.L) return fail("Level of rescale opnd is too small");
  c->flush_pending_overwriting(res, (level - 1) * (size_t)c->h.N, src, level * (size_t)c->h.N, true);
  c->submit_poly(2, U(res), U(src), level, is_ntt != 0);
  ACE_CATCH_INT
}

int ace_mod_down_rescale(ace_ctx* c, int64_t* res, int64_t* poly, size_t level, int is_ntt) {
  ACE_TRY
  CENSUS(level, 0);
  if (!res || !poly) return fail("ace_mod_down_rescale: null argument");
  if (level < 2 || level > c->h.L) return fail("ace_mod_down_rescale: level out of range");
  if (res == poly) return fail("ace_mod_down_rescale: the result must not overwrite the operand");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  u64* y = c->take(level * (size_t)c->h.N);
  do_moddown_rescale_core(c, U(res), y, nullptr, U(poly), level, is_ntt != 0);
  PolySeq rs = seq_strided(U(res), 0);
  launch_ntt(c->stream, c->d, rs, rs, c->q_lm, nullptr, (u32)(level - 1), 1, false, nullptr);
  ACE_CATCH_INT
}

int ace_reduce_rescale_modup(ace_ctx* c, int64_t* res, int64_t* raised, int64_t* poly, size_t level, int is_ntt) {
  ACE_TRY
  CENSUS(level, 0);
  if (!res || !raised || !poly) return fail("ace_reduce_rescale_modup: null argument");
  if (level < 2 || level > c->h.L) return fail("ace_reduce_rescale_modup: level out of range");
  if (res == poly || raised == poly || raised == res) return fail("ace_reduce_rescale_modup: buffers must be distinct");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  const size_t N = c->h.N, nl = level - 1;
  u64* x = c->take(nl * N);
  u64* last = c->take(N);
  // the reference leaves the converted P part in res and the reduced last limb in its limb level-1;
  // the kernel reads that limb of y from every block, so the reduced value goes to scratch first
  do_moddown_rescale_core(c, x, U(res), last, U(poly), level, is_ntt != 0);
  HIP_OK(hipMemcpyAsync(U(res) + nl * N, last, N * sizeof(u64), hipMemcpyDeviceToDevice, c->stream));
  do_precomp(c, U(raised), 0, x, 0, 1, nl, false);
  ACE_CATCH_INT
}

int ace_transform_from_level0(ace_ctx* c, int64_t* res, const int64_t* src, size_t level) {
  ACE_TRY
  CENSUS(level, 0);
  if (!res || !src) return fail("ace_transform_from_level0: null argument");
  if (!level_ok(c, level)) return fail("ace_transform_from_level0: level out of range");
  if (res != src && res < src + c->h.N && src < res + level * (size_t)c->h.N)
    return fail("ace_transform_from_level0: buffers overlap");
  launch_from_level0(c->stream, c->d, U(res), U(src), (u32)level);
  ACE_CATCH_INT
}

int ace_embedding_inv(ace_ctx* c, double* host_out, const double* host_in, size_t len) {
  ACE_TRY
  if (!host_out || !host_in) return fail("ace_embedding_inv: null argument");
  if (len == 0 || len > c->h.N / 2 || (len & (len - 1))) return fail("ace_embedding_inv: length must be a power of two of at most N/2");
  c->ensure_ws(4 * len + 16);
  c->ws_used = 0;
  double2* r = reinterpret_cast<double2*>(c->take(2 * len));
  double2* o = reinterpret_cast<double2*>(c->take(2 * len));
  HIP_OK(hipMemcpyAsync(r, host_in, len * sizeof(double2), hipMemcpyHostToDevice, c->stream));
  launch_embedding_inv(c->stream, c->d, o, r, c->fft_rou, c->rot_group, (u32)len);
  HIP_OK(hipMemcpyAsync(host_out, o, len * sizeof(double2), hipMemcpyDeviceToHost, c->stream));
  HIP_OK(hipStreamSynchronize(c->stream));
  ACE_CATCH_INT
}

int ace_decode(ace_ctx* c, double* host_out, const int64_t* poly, size_t level, int is_ntt, uint32_t slots,
               double factor) {
  ACE_TRY
  CENSUS(level, 0);
  if (!host_out || !poly) return fail("ace_decode: null argument");
  const size_t N = c->h.N, L = c->h.L;
  if (!slots) slots = (uint32_t)(N / 2);
  if (level == 0 || level > L) return fail("ace_decode: level out of range");
  if (level > (size_t)kDecodeWords) return fail("ace_decode: more than 64 limbs");
  if (slots > N / 2 || (slots & (slots - 1))) return fail("slot size must be a power of two of at most N/2");
  if (!(factor > 0.0)) return fail("ace_decode: the scale must be positive");
  if (!c->decode_tab) {
    std::vector<u64> tab(L + L * L, 0);
    for (size_t i = 0; i < L; ++i) {
      const u64 q = c->h.primes[i].q;
      u64 prod = 1;
      for (size_t j = 0; j < i; ++j) {
        tab[L + i * L + j] = prod;
        prod = mul_mod(prod, c->h.primes[j].q % q, q);
      }
      tab[i] = i ? inv_mod_prime(prod, q) : 1;
    }
    c->decode_tab = c->upload_vec(tab);
  }
  u64*& big_q = c->decode_q[level];
  if (!big_q) {
    std::vector<u64> w(level, 0);
    w[0] = 1;
    for (size_t i = 0; i < level; ++i) {
      unsigned __int128 carry = 0;
      for (size_t k = 0; k < level; ++k) {
        unsigned __int128 t = (unsigned __int128)w[k] * c->h.primes[i].q + carry;
        w[k] = (u64)t;
        carry = t >> 64;
      }
    }
    big_q = c->upload_vec(w);
  }
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  double2* r = reinterpret_cast<double2*>(c->take(2 * (size_t)slots));
  const u64* coef = U(poly);
  if (is_ntt) {  // the operand stays as it is
    u64* tmp = c->take(level * N);
    if (!launch_ntt(c->stream, c->d, seq_strided(tmp, 0), seq_strided(const_cast<u64*>(U(poly)), 0), c->q_lm, nullptr,
                    (u32)level, 1, true, nullptr))
      return fail("ace_decode: ring degree above 2^17, or a polynomial that does not start on a 16-byte boundary");
    coef = tmp;
  }
  launch_decode(c->stream, c->d, r, coef, (u32)level, slots, factor, c->decode_tab, c->decode_tab + L, (u32)L, big_q,
                c->fft_rou, c->rot_group);
  HIP_OK(hipMemcpyAsync(host_out, r, slots * sizeof(double2), hipMemcpyDeviceToHost, c->stream));
  HIP_OK(hipStreamSynchronize(c->stream));
  ACE_CATCH_INT
}

// kind: 0 complex doubles (re, im interleaved), 1 real doubles, 2 real floats.  Real inputs travel as they are and
// are widened to complex numbers on the device (a float widens exactly, as the host cast would).
// explicit_scale > 0: Encode_impl_with_scale (encoder.c:337-403): one multiplication by that scale, rounded without
// the half that Encode_impl adds first, and no further powers of the scaling factor.
// n_vec > 1: that many vectors (vecs[v], each n_values long, real-valued kinds only) are encoded in one set of
// launches into res + v * res_stride.
static int encode_impl(ace_ctx* c, int64_t* res, const void* values, int kind, size_t n_values, uint32_t slots,
                       size_t level, uint32_t sf_degree, size_t p_cnt, double explicit_scale = 0.0,
                       const void* const* vecs = nullptr, size_t n_vec = 1, size_t res_stride = 0) {
  ACE_TRY
  CENSUS_AS("ace_encode", level, n_vec);
  if (n_vec == 0) return 0;
  if (!vecs) vecs = &values;
  if (!res) return fail("ace_encode: null argument");
  for (size_t v = 0; v < n_vec; ++v)
    if (!vecs[v] && n_values) return fail("ace_encode: null argument");
  if (n_vec > 1 && (kind == 0 || n_values == 0)) return fail("ace_encode: batches take real-valued vectors");
  if (n_vec > 65535) return fail("ace_encode: more than 65535 vectors per call");
  if (!c->sf_bits) return fail("ace_encode: the context was created from explicit primes and has no scaling factor");
  const size_t N = c->h.N, K = c->h.K;
  if (!slots) slots = (uint32_t)(N / 2);
  if (!level) level = c->h.L;
  if (level > c->h.L) return fail("level should not be larger than mul_depth + 1");
  if (n_values > slots) return fail("slot size is too small");
  if (slots > N / 2 || (slots & (slots - 1))) return fail("slot size must be a power of two of at most N/2");
  if (p_cnt != 0 && p_cnt != K) return fail("ace_encode: p_cnt must be 0 or the number of special primes");
  const bool by_scale = explicit_scale > 0.0;
  if (by_scale) {
    // (encoder.c:355-357 casts log2(scale) to uint32_t and derives the scale degree the same way; below 1 both
    // conversions are out of range and what the reference then does depends on the compiler: refused here)
    if (explicit_scale < 1.0 || std::log2(explicit_scale) >= (double)(c->q0_bits + (level - 1) * c->sf_bits))
      return fail("invalid scale for encode");
    sf_degree = 1;
  } else if (sf_degree < 1 || c->sf_bits * sf_degree >= c->q0_bits + (level - 1) * c->sf_bits) {
    return fail("invalid scaling factor for encode");
  }
  const double scaling_factor = by_scale ? explicit_scale : std::ldexp(1.0, (int)c->sf_bits);
  const double scale = by_scale ? explicit_scale : std::pow(scaling_factor, (double)sf_degree);
  // Check_msg_range (encoder.c:48-59): the largest scaled coefficient must stay below 2^(valid bits - 1)
  const int valid = (int)c->q0_bits + (int)(level - 1) * (int)c->sf_bits;
  const double range_bound = std::ldexp(1.0, valid - 1);
  LimbMap lm = poly_lm(c, level, p_cnt != 0);
  const u32 n_limbs = (u32)(level + p_cnt);
  const size_t value_bytes = kind == 0 ? sizeof(double2) : kind == 1 ? sizeof(double) : sizeof(float);
  const size_t poly_words = (size_t)n_limbs * N;
  if (n_vec > 1 && res_stride < poly_words) return fail("ace_encode: result stride smaller than a polynomial");
  auto stage_values = [&](hipStream_t st, double2* z, void* raw) {  // z = the values, zero-padded to `slots`
    if (kind == 0) {
      if (n_values < slots)
        launch_fill_zero(st, reinterpret_cast<u64*>(z + n_values), 2 * (size_t)(slots - n_values));
      c->h2d(z, vecs[0], n_values * value_bytes);
    } else {
      c->h2d_gather(raw, vecs, n_vec, n_values * value_bytes);
      launch_widen_real(st, z, raw, kind == 2, (u32)n_values, slots, (u32)n_vec);
    }
  };
  c->ensure_ws(std::max(c->std_ws(level), 3 * (size_t)slots * n_vec + 2 * level + 64));
  c->ws_used = 0;
  double2* z = reinterpret_cast<double2*>(c->take(2 * (size_t)slots * n_vec));
  stage_values(c->stream, z, kind == 0 ? nullptr : c->take((size_t)slots * n_vec));
  launch_encode(c->stream, c->d, U(res), z, c->fft_rou, c->rot_group, slots, scaling_factor, scale,
                by_scale ? 0.0 : 0.5, range_bound, lm, n_limbs, c->d_err, (u32)n_vec, res_stride);
  if (sf_degree > 1) {  // encoder.c:297-312: the Q limbs are multiplied by scaling_factor^(sf_degree-1)
    std::vector<u64> cst(2 * level);
    for (size_t t = 0; t < level; ++t) {
      u64 q = c->h.primes[t].q, base = (u64)scaling_factor % q, powp = base;
      for (uint32_t d = 2; d < sf_degree; ++d) powp = mul_mod(powp, base, q);
      cst[2 * t] = powp;
      cst[2 * t + 1] = shoup(powp, q);
    }
    u64* dc = c->take(2 * level);
    c->h2d(dc, cst.data(), cst.size() * sizeof(u64));
    for (size_t v = 0; v < n_vec; ++v)
      launch_mul_const(c->stream, c->d, U(res) + v * res_stride, U(res) + v * res_stride, dc, c->q_lm, (u32)level);
  }
  PolySeq rs = seq_strided(U(res), res_stride);
  launch_ntt(c->stream, c->d, rs, rs, lm, nullptr, n_limbs, (u32)n_vec, false, nullptr);
  ACE_CATCH_INT
}
int ace_encode(ace_ctx* c, int64_t* res, const double* values, size_t n_values, uint32_t slots, size_t level,
               uint32_t sf_degree, size_t p_cnt) {
  return encode_impl(c, res, values, 0, n_values, slots, level, sf_degree, p_cnt);
}
int ace_encode_real(ace_ctx* c, int64_t* res, const void* values, int is_f32, size_t n_values, uint32_t slots,
                    size_t level, uint32_t sf_degree, size_t p_cnt) {
  return encode_impl(c, res, values, is_f32 ? 2 : 1, n_values, slots, level, sf_degree, p_cnt);
}
int ace_encode_real_batch(ace_ctx* c, int64_t* res, size_t res_stride, const void* const* values, int is_f32,
                          size_t n_values, size_t n_vec, uint32_t slots, size_t level, uint32_t sf_degree,
                          size_t p_cnt) {
  if (!values) return fail("ace_encode_real_batch: null argument");
  return encode_impl(c, res, nullptr, is_f32 ? 2 : 1, n_values, slots, level, sf_degree, p_cnt, 0.0, values, n_vec,
                     res_stride);
}
int ace_encode_scaled(ace_ctx* c, int64_t* res, const double* values, size_t n_values, uint32_t slots, size_t level,
                      double scale, size_t p_cnt) {
  if (!(scale > 0.0)) return fail("invalid scale for encode");
  return encode_impl(c, res, values, 0, n_values, slots, level, 1, p_cnt, scale);
}

int ace_extend(ace_ctx* c, int64_t* res, const int64_t* src, size_t level) {
  ACE_TRY
  CENSUS(level, 0);
  if (!res || !src) return fail("ace_extend: null argument");
  if (!level_ok(c, level)) return fail("ace_extend: level out of range");
  launch_mul_const(c->stream, c->d, U(res), U(src), c->pmodq, c->q_lm, (u32)level);
  launch_fill_zero(c->stream, U(res) + level * (size_t)c->h.N, c->h.K * (size_t)c->h.N);
  ACE_CATCH_INT
}

int ace_dot_prod(ace_ctx* c, int64_t* res, const int64_t* digits, const int64_t* key, size_t key_stride,
                 size_t n_parts, size_t level) {
  ACE_TRY
  CENSUS(level, 0);
  if (!res || !digits || !key) return fail("ace_dot_prod: null argument");
  if (!level_ok(c, level)) return fail("ace_dot_prod: level out of range");
  if (n_parts == 0 || n_parts > c->h.parts) return fail("ace_dot_prod: number of digits out of range");
  size_t T = level + c->h.K;
  LimbMap lm = poly_lm(c, level, true), kp = key_pos(c, level);
  launch_dotprod(c->stream, c->d, U(res), nullptr, 0, U(digits), T * (size_t)c->h.N, 0, one_key(U(key)), 0,
                 key_stride, (u32)n_parts, lm, kp, (u32)T, 1);
  ACE_CATCH_INT
}

int ace_ext_rotate(ace_ctx* c, int64_t* out0, int64_t* out1, const int64_t* digits, const int64_t* key,
                   size_t key_half_words, size_t key_stride, size_t n_parts, const int64_t* addend0,
                   const int64_t* order, size_t level, int accumulate) {
  ACE_TRY
  CENSUS(level, 0);
  if (!out0 || !out1 || !digits || !key || !order) return fail("ace_ext_rotate: null argument");
  if (!level_ok(c, level)) return fail("ace_ext_rotate: level out of range");
  if (n_parts == 0 || n_parts > c->h.parts) return fail("ace_ext_rotate: number of digits out of range");
  const size_t T = level + c->h.K, words = T * (size_t)c->h.N;
  auto overlap = [&](const int64_t* a, const int64_t* b, size_t nb) { return a < b + nb && b < a + words; };
  if (overlap(out0, digits, n_parts * words) || overlap(out1, digits, n_parts * words) || overlap(out0, out1, words) ||
      (addend0 && (overlap(out0, addend0, words) || overlap(out1, addend0, words))))
    return fail("ace_ext_rotate: the results must not overlap the operands (the automorphism is applied on the way in)");
  LimbMap lm = poly_lm(c, level, true), kp = key_pos(c, level);
  launch_ext_rotate(c->stream, c->d, U(out0), U(out1), U(digits), words, U(key), key_half_words, key_stride,
                    (u32)n_parts, addend0 ? U(addend0) : nullptr, order, accumulate & 3, lm, kp, (u32)T);
  ACE_CATCH_INT
}

// ---- ciphertext level ------------------------------------------------------------
int ace_mul_ciph3(ace_ctx* c, int64_t* d0, int64_t* d1, int64_t* d2, const int64_t* a0, const int64_t* a1,
                  const int64_t* b0, const int64_t* b1, size_t level) {
  ACE_TRY_BARE
  CENSUS(level, 0);
  if (!d0 || !d1 || !d2 || !a0 || !a1 || !b0 || !b1) return fail("ace_mul_ciph3: null argument");
  if (!level_ok(c, level)) return fail("ace_mul_ciph3: level out of range");
  {
    const size_t w = level * (size_t)c->h.N;
    c->flush_pending_declared({ace_ctx::span(d0, w), ace_ctx::span(d1, w), ace_ctx::span(d2, w)},
                              {ace_ctx::span(a0, w), ace_ctx::span(a1, w), ace_ctx::span(b0, w), ace_ctx::span(b1, w)});
  }
  launch_tensor(c->stream, c->d, U(d0), U(d1), U(d2), U(a0), U(a1), U(b0), U(b1), c->q_lm, (u32)level, 1, 0, 0, 0);
  ACE_CATCH_INT
}

int ace_fast_switch_key(ace_ctx* c, int64_t* out0, int64_t* out1, const int64_t* digits, const int64_t* swk,
                        size_t level) {
  ACE_TRY
  CENSUS(level, 0);
  if (!out0 || !out1 || !digits || !swk) return fail("ace_fast_switch_key: null argument");
  if (!level_ok(c, level)) return fail("ace_fast_switch_key: level out of range");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_switch_key(c, seq_pair(U(out0), U(out1), 0), U(digits), 0, one_key(U(swk)), 1, level, nullptr, 0);
  ACE_CATCH_INT
}

int ace_relin(ace_ctx* c, int64_t* r0, int64_t* r1, const int64_t* d0, const int64_t* d1, const int64_t* d2,
              const int64_t* swk, size_t level) {
  ACE_TRY
  CENSUS(level, 0);
  if (!r0 || !r1 || !d0 || !d1 || !d2 || !swk) return fail("ace_relin: null argument");
  if (!level_ok(c, level)) return fail("ace_relin: level out of range");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  size_t nd = c->h.num_decomp(level), T = level + c->h.K;
  u64* digits = c->take(nd * T * c->h.N);
  do_precomp(c, digits, 0, U(d2), 0, 1, level, true);
  PolySeq add = seq_pair(U(d0), U(d1), 0);
  do_switch_key(c, seq_pair(U(r0), U(r1), 0), digits, 0, one_key(U(swk)), 1, level, &add, 1);
  ACE_CATCH_INT
}

int ace_rescale_ciph(ace_ctx* c, int64_t* r0, int64_t* r1, const int64_t* c0, const int64_t* c1, size_t level) {
  ACE_TRY
  CENSUS(level, 0);
  if (!r0 || !r1 || !c0 || !c1) return fail("ace_rescale_ciph: null argument");
  if (level < 2 || level > c->h.L) return fail("Level of rescale opnd is too small");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_rescale(c, seq_pair(U(r0), U(r1), 0), seq_pair(U(c0), U(c1), 0), 2, level, true);
  ACE_CATCH_INT
}

int ace_mul_relin_rescale(ace_ctx* c, int64_t* r0, int64_t* r1, const int64_t* a0, const int64_t* a1,
                          const int64_t* b0, const int64_t* b1, const int64_t* swk, size_t level) {
  ACE_TRY
  CENSUS(level, 1);
  if (!r0 || !r1 || !a0 || !a1 || !b0 || !b1 || !swk) return fail("ace_mul_relin_rescale: null argument");
  if (level < 2 || level > c->h.L) return fail("ace_mul_relin_rescale: level out of range");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_mul_relin_rescale(c, U(r0), U(r1), 0, U(a0), U(a1), U(b0), U(b1), 0, U(swk), 1, level);
  ACE_CATCH_INT
}

int ace_mul_relin_double_rescale(ace_ctx* c, int64_t* r0, int64_t* r1, const int64_t* a0, const int64_t* a1,
                                 const int64_t* b0, const int64_t* b1, const int64_t* swk, size_t level) {
  ACE_TRY
  CENSUS(level, 1);
  if (!r0 || !r1 || !a0 || !a1 || !b0 || !b1 || !swk) return fail("ace_mul_relin_double_rescale: null argument");
  if (level < 2 || level > c->h.L) return fail("ace_mul_relin_double_rescale: level out of range");
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_mul_relin_rescale(c, U(r0), U(r1), 0, U(a0), U(a1), U(b0), U(b1), 0, U(swk), 1, level, true);
  ACE_CATCH_INT
}

int ace_mul_relin_double_add_rescale(ace_ctx* c, int64_t* r0, int64_t* r1, const int64_t* a0, const int64_t* a1,
                                     const int64_t* b0, const int64_t* b1, const int64_t* swk, const int64_t* constant,
                                     size_t level) {
  ACE_TRY
  CENSUS(level, 1);
  if (!r0 || !r1 || !a0 || !a1 || !b0 || !b1 || !swk || !constant)
    return fail("ace_mul_relin_double_add_rescale: null argument");
  if (level < 2 || level > c->h.L) return fail("ace_mul_relin_double_add_rescale: level out of range");
  u64 words[kMaxPrimes];
  for (size_t t = 0; t < level; ++t) {
    if (constant[t] < 0 || (u64)constant[t] >= c->h.primes[t].q)
      return fail("ace_mul_relin_double_add_rescale: constant is not a residue");
    words[t] = (u64)constant[t];
  }
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  do_mul_relin_rescale(c, U(r0), U(r1), 0, U(a0), U(a1), U(b0), U(b1), 0, U(swk), 1, level, true, words);
  ACE_CATCH_INT
}

static bool ranges_overlap(const void* a, size_t a_words, const void* b, size_t b_words);
int ace_mod_down_pair_rescale(ace_ctx* c, int64_t* r0, int64_t* r1, const int64_t* e0, const int64_t* e1, size_t level) {
  ACE_TRY
  CENSUS(level, 2);
  if (!r0 || !r1 || !e0 || !e1) return fail("ace_mod_down_pair_rescale: null argument");
  if (level < 2 || level > c->h.L) return fail("ace_mod_down_pair_rescale: level out of range");
  {
    const size_t rw = (level - 1) * (size_t)c->h.N, ew = (level + c->h.K) * (size_t)c->h.N;
    if (ranges_overlap(r0, rw, r1, rw) || ranges_overlap(r0, rw, e0, ew) || ranges_overlap(r0, rw, e1, ew) ||
        ranges_overlap(r1, rw, e0, ew) || ranges_overlap(r1, rw, e1, ew))
      return fail("ace_mod_down_pair_rescale: the results must not overlap the operands or each other");
  }
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  const size_t N = c->h.N;
  if (c->d.logN > 12 && c->share_transform) {
    do_moddown_rescale_shared(c, seq_pair(U(r0), U(r1), 0), seq_pair(U(e0), U(e1), 0), 2, level, false);
  } else {
    u64* x = c->take(2 * level * N);
    do_mod_down(c, seq_strided(x, level * N), seq_pair(U(e0), U(e1), 0), 2, level, true, nullptr, 0);
    do_rescale(c, seq_pair(U(r0), U(r1), 0), seq_strided(x, level * N), 2, level, true);
  }
  ACE_CATCH_INT
}

int ace_mul_relin_rescale_batch(ace_ctx* c, int64_t* r0, int64_t* r1, size_t out_stride, const int64_t* a0,
                                const int64_t* a1, const int64_t* b0, const int64_t* b1, size_t in_stride,
                                const int64_t* swk, size_t level, size_t count) {
  ACE_TRY
  CENSUS_AS("ace_mul_relin_rescale", level, count);
  if (count == 0) return 0;
  if (!r0 || !r1 || !a0 || !a1 || !b0 || !b1 || !swk) return fail("ace_mul_relin_rescale_batch: null argument");
  if (level < 2 || level > c->h.L) return fail("ace_mul_relin_rescale_batch: level out of range");
  if (count > 1 && (in_stride < level * (size_t)c->h.N || out_stride < (level - 1) * (size_t)c->h.N))
    return fail("ace_mul_relin_rescale_batch: stride smaller than one polynomial");
  const size_t chunk = 16;  // operands per pass: bounds the scratch arena at 16x the single-operand size
  c->ensure_ws(std::min(count, chunk) * c->std_ws(level));
  for (size_t o = 0; o < count; o += chunk) {
    size_t nb = std::min(chunk, count - o);
    c->ws_used = 0;
    do_mul_relin_rescale(c, U(r0) + o * out_stride, U(r1) + o * out_stride, out_stride, U(a0) + o * in_stride,
                         U(a1) + o * in_stride, U(b0) + o * in_stride, U(b1) + o * in_stride, in_stride, U(swk), nb,
                         level);
  }
  ACE_CATCH_INT
}

static bool ranges_overlap(const void* a, size_t a_words, const void* b, size_t b_words) {
  const uintptr_t x = (uintptr_t)a, y = (uintptr_t)b;
  return x < y + b_words * sizeof(u64) && y < x + a_words * sizeof(u64);
}

// Fast_rotate for nr <= kMaxBatchPtrs rotations of one ciphertext sharing the digits:
// switch key, add c0 to the first polynomial, permute -- the last two inside the Mod_down tail
static void do_fast_rotate(ace_ctx* c, u64* r0, u64* r1, u64 r_stride, const u64* c0, const u64* digits,
                           const KeySet& keys, const OrderSet& orders, size_t nr, size_t level) {
  PolySeq add = seq_pair(c0, c0, 0);  // c0 is added to the first polynomial of every rotation
  do_switch_key(c, seq_pair(r0, r1, r_stride), digits, 0, keys, nr, level, &add, 2, &orders);
}

int ace_fast_rotate(ace_ctx* c, int64_t* r0, int64_t* r1, const int64_t* c0, const int64_t* digits,
                    const int64_t* swk, const int64_t* order, size_t level) {
  ACE_TRY
  CENSUS(level, 0);
  if (!r0 || !r1 || !c0 || !digits || !swk || !order) return fail("ace_fast_rotate: null argument");
  if (!level_ok(c, level)) return fail("ace_fast_rotate: level out of range");
  {
    const size_t pw = level * (size_t)c->h.N, dw = c->h.num_decomp(level) * (level + c->h.K) * (size_t)c->h.N;
    if (ranges_overlap(r0, pw, c0, pw) || ranges_overlap(r1, pw, c0, pw) || ranges_overlap(r0, pw, digits, dw) ||
        ranges_overlap(r1, pw, digits, dw) || ranges_overlap(r0, pw, r1, pw))
      return fail("ace_fast_rotate: the results must not overlap c0, the digits or each other (they are permuted on the way out)");
  }
  c->ensure_ws(c->std_ws(level));
  c->ws_used = 0;
  OrderSet os{};
  os.n = 1;
  os.p[0] = order;
  do_fast_rotate(c, U(r0), U(r1), 0, U(c0), U(digits), one_key(U(swk)), os, 1, level);
  ACE_CATCH_INT
}

int ace_rotate_batch(ace_ctx* c, int64_t* r0s, int64_t* r1s, const int64_t* c0, const int64_t* c1,
                     const int64_t* const* swks, const int64_t* const* orders, size_t count, size_t level) {
  ACE_TRY
  CENSUS(level, count);
  if (count == 0) return 0;
  if (!r0s || !r1s || !c0 || !c1 || !swks || !orders) return fail("ace_rotate_batch: null argument");
  if (!level_ok(c, level)) return fail("ace_rotate_batch: level out of range");
  {
    const size_t pw = level * (size_t)c->h.N, rw = count * pw;
    if (ranges_overlap(r0s, rw, c0, pw) || ranges_overlap(r1s, rw, c0, pw) || ranges_overlap(r0s, rw, r1s, rw))
      return fail("ace_rotate_batch: the results must not overlap c0 or each other (they are permuted on the way out)");
  }
  for (size_t i = 0; i < count; ++i)
    if (!swks[i] || !orders[i]) return fail("ace_rotate_batch: null key or order table");
  const size_t N = c->h.N, nd = c->h.num_decomp(level), T = level + c->h.K;
  const size_t chunk = kMaxBatchPtrs;
  c->ensure_ws((std::min(count, chunk) + 1) * c->std_ws(level));
  c->ws_used = 0;
  u64* digits = c->take(nd * T * N);
  do_precomp(c, digits, 0, U(c1), 0, 1, level, true);
  for (size_t i0 = 0; i0 < count; i0 += chunk) {
    size_t nr = std::min(chunk, count - i0);
    KeySet ks{};
    OrderSet os{};
    ks.n = os.n = (u32)nr;
    for (size_t i = 0; i < nr; ++i) { ks.p[i] = U(swks[i0 + i]); os.p[i] = orders[i0 + i]; }
    if (nr == 1) { ks.n = os.n = 1; }
    do_fast_rotate(c, U(r0s) + i0 * level * N, U(r1s) + i0 * level * N, level * N, U(c0), digits, ks, os, nr, level);
  }
  ACE_CATCH_INT
}

}  // extern "C"
