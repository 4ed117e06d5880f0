// Negacyclic NTT / inverse NTT kernels for gfx950.
//
// Algorithm (value-identical to Forward_transform / Inverse_transform,
// fhe-cmplr/rtlib/ant/util/src/ntt.c:167-330): radix-2 Cooley-Tukey, natural
// order in / bit-reversed out, twiddle of group i at the stage with m groups
// is rou[m+i]; the inverse is Gentleman-Sande with rou_inv[m+i] and 1/N.
//
// Mapping for N = 2^logN > 4096, R = N/4096 = 2^LOGR:
//   forward  pass 1 "strided": stages 0..LOGR-1.  One thread owns one column
//            (R coefficients 4096 apart) entirely in registers; loads and
//            stores are 2 KiB-contiguous per wavefront row.  No LDS.
//            pass 2 "chunk": stages LOGR..logN-1 on one contiguous 4096-word
//            chunk per workgroup: 512 threads x 8 registers, four rounds of
//            three stages with the chunk passing through LDS between rounds
//            (LDS index padded by e>>4, which keeps every round's accesses
//            free of bank conflicts), and once more so that the global
//            store is coalesced.  Two of the exchanges stay inside the 512
//            words a wave owns and need no work-group barrier.  Eight registers per thread leave room for
//            eight waves per SIMD, which is what hides the memory waits.
//   inverse  the same two kernels mirrored (chunk first, strided last).
// N <= 4096 uses one workgroup per limb with the limb in LDS.
//
// Two arithmetic back ends share the index logic:
//   ArithInt  64-bit integers, Harvey lazy butterflies (forward < 8q, inverse
//             < 4q) with Shoup twiddles whose quotient is estimated from three
//             partial products (up to 2 too small); any prime below 2^61.
//             About 27 VALU instructions per butterfly, which makes the chunk
//             pass instruction-bound.
//   ArithFp   for primes below 2^50.2: residues are carried as exact integers
//             in FP64 (|x| < 2^53).  A twiddle product is y*w - rint(y*(w/q))*q
//             evaluated exactly with one FMA for the low half of y*w and one
//             for the subtraction (6 full-rate FP64 ops).  The twiddles are
//             stored centred on zero (|w| <= q/2): the quotient estimate is off
//             by at most 1/2 + 3*2^-53*|y||w|/q, so a product of a value of
//             magnitude B q comes out below (0.5 + 0.215 B) q, and a forward
//             stage takes a bound of B q to at most (1.215 B + 0.5) q.  From
//             centred values (B = 1/2) six stages reach 6.77 q, from canonical
//             residues (B = 1) five reach 6.49 q, both below 2^53 / q >= 6.98:
//             the forward strided pass reduces (x - rint(x/q)*q) only what it
//             stores, the forward chunk pass only before its third round.
//             An inverse stage doubles the bound of its sums, so inverse code
//             reduces every three stages (0.5 q -> 4 q).  All intermediate
//             values are integers below 2^53, so no rounding ever happens and
//             the final canonical residue is exact.
// Between the two passes the buffer holds back-end specific words (lazily
// reduced integers, or raw FP64 bits); the second pass stores canonical
// residues.
#include <vector>

#include "ace_kernels.h"

#pragma clang fp contract(off)

namespace ace {

// Coefficients are read once and written once by every pass, so they go past the caches with the non-temporal hint
// (twiddles keep the default policy).  Measured on the 768-limb batch: loads and stores both hinted take 4 to 10 % off
// the strided passes and up to 9 % off the forward chunk pass, depending on the machine; either alone changes nothing,
// and hinted 16-byte loads of the inverse chunk pass (four per 64-byte line and lane) cost 20 %, so those stay cached.
// The tails fused into the forward chunk pass (Mod_down, Rescale) read their operands and write their results once as
// well: hinted, the key switch gains about 1 %; the gathered reads of the tail that carries an automorphism gain nothing
// and stay cached.  The selector is a template argument: as a function argument of the inlined helpers it was folded
// away at some call sites and not at others once there were more of them.
// The inverse chunk pass, whose loads stay cached, does better with its stores cached too (key switch +1.2 %, the
// batch transform unchanged).
// ACE_NTT_NT bits: 1 strided stores, 2 strided loads, 4 forward chunk stores, 8 forward chunk loads, 16 tail stores,
// 32 tail loads, 64 gathered tail loads, 512 inverse chunk stores.
#ifndef ACE_NTT_NT
#define ACE_NTT_NT 63
#endif
template <int BIT, class P>
__device__ __forceinline__ P ldg(const P* p) {
  if constexpr ((ACE_NTT_NT & BIT) != 0) return __builtin_nontemporal_load(p);
  else return *p;
}
template <int BIT, class P>
__device__ __forceinline__ void stg(P* p, P v) {
  if constexpr ((ACE_NTT_NT & BIT) != 0) __builtin_nontemporal_store(v, p);
  else *p = v;
}
constexpr int kChunk = 4096;
constexpr int kLogChunk = 12;

__device__ __forceinline__ int lds_pos(int e) { return e + (e >> 4); }

// Orders the LDS writes of a wave before its own later LDS reads, where no other wave touches those words (the
// wave <-> octet <-> narrow exchanges of a chunk pass stay inside the 512 words a wave owns): the hardware carries
// out one wave's LDS instructions in order, so only the compiler has to be kept from moving them.
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// A 16-byte load per lane that writes LDS directly (no registers held while it is on its way).
__device__ __forceinline__ void stage_request(const u64* src, u64* lds_block) {
  // lane L's 16 bytes go to lds_block + 16 L; m0 carries the block's LDS address
  const u32 at = (u32)__builtin_amdgcn_readfirstlane((int)(u32)(size_t)(__attribute__((address_space(3))) void*)lds_block);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" : : "v"(src), "s"(at) : "memory", "m0");
}

// ---------------------------------------------------------------------------
struct ArithInt {
  typedef u64 T;
  static constexpr bool kFp = false;
  u64 q, q2, q4;
  const u64 *w, *wp;  // twiddle, Shoup companion
  u64 sc, scp;        // inverse: final scale constant
  __device__ __forceinline__ void init(const DevCtx& c, u32 pi, bool inverse, const u64* scale, u32 sidx) {
    const DevPrime& P = c.primes[pi];
    q = P.q;
    q2 = q << 1;
    q4 = q << 2;
    w = (inverse ? c.irou : c.rou) + (u64)pi * c.N;
    wp = (inverse ? c.irou_p : c.rou_p) + (u64)pi * c.N;
    sc = P.ninv;
    scp = P.ninv_p;
    if (scale) { sc = scale[2 * sidx]; scp = scale[2 * sidx + 1]; }
  }
  struct TW { u64 w, wp; };
  typedef TW TWL;  // as loaded == as used
  __device__ __forceinline__ TW prep(const TWL& t) const { return t; }
  // NG consecutive twiddles starting at index ti0 (a multiple of NG): 16-byte loads
  template <int NG>
  __device__ __forceinline__ void load_tw(u32 ti0, TWL* tw) const {
    if (NG == 1) {
      tw[0].w = w[ti0];
      tw[0].wp = wp[ti0];
    } else {
      const ulonglong2* a = reinterpret_cast<const ulonglong2*>(w + ti0);
      const ulonglong2* b = reinterpret_cast<const ulonglong2*>(wp + ti0);
#pragma unroll
      for (int k = 0; k < NG / 2; ++k) {
        ulonglong2 x = a[k], y = b[k];
        tw[2 * k].w = x.x; tw[2 * k + 1].w = x.y;
        tw[2 * k].wp = y.x; tw[2 * k + 1].wp = y.y;
      }
    }
  }
  __device__ __forceinline__ T in_canon(u64 v) const { return v; }
  __device__ __forceinline__ T in_mid(u64 v) const { return v; }
  __device__ __forceinline__ u64 out_mid(T v) const { return v; }
  __device__ __forceinline__ void reduce(T&) const {}
  __device__ __forceinline__ void recentre_sum_of_four(T&) const {}
  // forward, Harvey butterflies with the cheaper quotient estimate (product in [0, 4q)): x,y < 8q -> < 8q
  __device__ __forceinline__ void ct(T& x, T& y, const TW& tw) const {
    u64 a = csub(x, q4);
    u64 t = shoup_lazier(y, tw.w, tw.wp, q);
    x = a + t;
    y = a - t + q4;
  }
  // inverse: x,y < 4q -> < 4q
  __device__ __forceinline__ void gs(T& x, T& y, const TW& tw) const {
    u64 s = csub(x + y, q4);
    u64 d = x - y + q4;
    x = s;
    y = shoup_lazier(d, tw.w, tw.wp, q);
  }
  __device__ __forceinline__ u64 out_canon(T v) const { return csub(csub(csub(v, q4), q2), q); }
  __device__ __forceinline__ u64 out_scaled(T v) const { return shoup_mul(v, sc, scp, q); }
};

struct ArithFp {
  typedef double T;
  static constexpr bool kFp = true;
  double q, qinv;
  const double* w;  // twiddles as exact FP64 integers
  double sc, sci;
  static constexpr double kMagic = 4503599627370496.0;  // 2^52
  __device__ __forceinline__ void init(const DevCtx& c, u32 pi, bool inverse, const u64* scale, u32 sidx) {
    const DevPrime& P = c.primes[pi];
    q = (double)P.q;
    qinv = 1.0 / q;
    w = (inverse ? c.iroud : c.roud) + (u64)pi * c.N;
    u64 s = scale ? scale[2 * sidx] : P.ninv;
    sc = (double)s;
    sci = sc / q;
  }
  struct TW { double w, wi; };
  typedef double TWL;  // only w is loaded
  // w/q is formed at use as w * (1/q): two roundings, relative error 2^-52,
  // which only widens the quotient estimate (|product| <= (1/2 + 0.43 |y|/q) q),
  // never the exactness
  __device__ __forceinline__ TW prep(const TWL& t) const { return TW{t, t * qinv}; }
  // NG consecutive twiddles from index ti0 (a multiple of NG), 16-byte loads
  template <int NG>
  __device__ __forceinline__ void load_tw(u32 ti0, TWL* tw) const {
    if (NG == 1) {
      tw[0] = w[ti0];
    } else {
      const double2* a = reinterpret_cast<const double2*>(w + ti0);
#pragma unroll
      for (int k = 0; k < NG / 2; ++k) {
        double2 x = a[k];
        tw[2 * k] = x.x; tw[2 * k + 1] = x.y;
      }
    }
  }
  __device__ __forceinline__ T in_canon(u64 v) const {  // v < 2^52
    return __longlong_as_double((long long)(v | 0x4330000000000000ull)) - kMagic;
  }
  __device__ __forceinline__ T in_mid(u64 v) const { return __longlong_as_double((long long)v); }
  __device__ __forceinline__ u64 out_mid(T v) const { return (u64)__double_as_longlong(v); }
  // x - rint(x/q)*q: |result| <= (1/2 + 2^-49) q, exact
  __device__ __forceinline__ void reduce(T& x) const { x = __builtin_fma(-__builtin_rint(x * qinv), q, x); }
  // The first round of an inverse chunk pass starts from canonical residues, all in [0, q).  Instead of centring
  // all eight values (24 operations), the two sums of four that meet in the third stage, each in [0, 4q), are
  // shifted by 2q: their sum stays within +-4q, every other value has passed through a twiddle product and is
  // small, and the round ends with the same bound (4q) as one that starts from centred values.
  __device__ __forceinline__ void recentre_sum_of_four(T& x) const { x -= q + q; }
  // y*w mod q as a signed integer of magnitude <= (1/2 + 0.43 |y|/q) q, exact
  __device__ __forceinline__ double mulmod(double y, double ww, double wwi) const {
    double c = __builtin_rint(y * wwi);
    double h = y * ww;
    double l = __builtin_fma(y, ww, -h);
    double d = __builtin_fma(-c, q, h);
    return d + l;
  }
  __device__ __forceinline__ void ct(T& x, T& y, const TW& tw) const {
    double t = mulmod(y, tw.w, tw.wi);
    y = x - t;
    x = x + t;
  }
  __device__ __forceinline__ void gs(T& x, T& y, const TW& tw) const {
    double d = x - y;
    x = x + y;
    y = mulmod(d, tw.w, tw.wi);
  }
  __device__ __forceinline__ u64 to_u64(double r) const {  // |r| <= q/2 (+)
    r = r < 0.0 ? r + q : r;
    return (u64)__double_as_longlong(r + kMagic) & 0x000FFFFFFFFFFFFFull;
  }
  __device__ __forceinline__ u64 out_canon(T v) const {
    reduce(v);
    return to_u64(v);
  }
  __device__ __forceinline__ u64 out_scaled(T v) const {
    reduce(v);
    double t = mulmod(v, sc, sci);
    reduce(t);
    return to_u64(t);
  }
};

// ---------------------------------------------------------------------------
// One radix-2 stage over a register file of R values.
// forward stage K (0 = widest span): groups = 2^K, pairs (i, i + R/2^(K+1))
template <class A, int R, int K>
__device__ __forceinline__ void ct_stage_pre(const A& ar, typename A::T* v, const typename A::TWL* tw) {
  constexpr int G = 1 << K, half = R >> (K + 1);
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const typename A::TW w = ar.prep(tw[g]);
#pragma unroll
    for (int j = 0; j < half; ++j) ar.ct(v[g * 2 * half + j], v[g * 2 * half + j + half], w);
  }
}
template <class A, int R, int K>
__device__ __forceinline__ void ct_stage(const A& ar, typename A::T* v, u32 ti0) {
  typename A::TWL tw[1 << K];
  ar.template load_tw<(1 << K)>(ti0, tw);
  ct_stage_pre<A, R, K>(ar, v, tw);
}
// inverse stage K (0 = narrowest span): span = 2^K, groups = R/2^(K+1)
template <class A, int R, int K>
__device__ __forceinline__ void gs_stage_pre(const A& ar, typename A::T* v, const typename A::TWL* tw) {
  constexpr int G = R >> (K + 1), span = 1 << K;
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const typename A::TW w = ar.prep(tw[g]);
#pragma unroll
    for (int j = 0; j < span; ++j) ar.gs(v[g * 2 * span + j], v[g * 2 * span + j + span], w);
  }
}
template <class A, int R, int K>
__device__ __forceinline__ void gs_stage(const A& ar, typename A::T* v, u32 ti0) {
  typename A::TWL tw[R >> (K + 1)];
  ar.template load_tw<(R >> (K + 1))>(ti0, tw);
  gs_stage_pre<A, R, K>(ar, v, tw);
}
template <class A, int R>
__device__ __forceinline__ void reduce_all(const A& ar, typename A::T* v) {
#pragma unroll
  for (int r = 0; r < R; ++r) ar.reduce(v[r]);
}

// all LOGR stages of the strided passes (twiddle indices are wave-uniform)
template <class A, int LOGR, int K = 0>
__device__ __forceinline__ void fwd_strided_stages(const A& ar, typename A::T* v) {
  if constexpr (K < LOGR) {
    // the FP64 back end may run five stages from canonical residues, six from centred ones (see the head of
    // this file): no reduction here for LOGR <= 5
    static_assert(LOGR <= 5, "reduce before the sixth stage");
    ct_stage<A, (1 << LOGR), K>(ar, v, 1u << K);
    fwd_strided_stages<A, LOGR, K + 1>(ar, v);
  }
}
template <class A, int LOGR, int K = 0>
__device__ __forceinline__ void inv_strided_stages(const A& ar, typename A::T* v) {
  if constexpr (K < LOGR) {
    if (K % 3 == 0) reduce_all<A, (1 << LOGR)>(ar, v);  // an inverse stage doubles the bound: three from centred values
    gs_stage<A, (1 << LOGR), K>(ar, v, (1u << LOGR) >> (K + 1));
    inv_strided_stages<A, LOGR, K + 1>(ar, v);
  }
}

// What a thread of a forward strided pass starts from: R words of its column, `step` words apart from `first` on.
// PRO = 0: read from src.  PRO = 1: formed from the last limb of a rescale (FwdFuse::pro).  PRO = 2: the same plus
// the source word, the last limb's word being the difference of two operands (a Mod_down and a Rescale that share
// this transform).
template <class A, int R, int PRO>
__device__ __forceinline__ void fwd_strided_input(const A& ar, const DevCtx& c, const PolySeq& srcs, const LimbMap& pos,
                                                  const FwdFuse& f, u32 limb, u32 pi, u32 col, u64 first, u64 step,
                                                  typename A::T* v) {
  if (PRO == 0) {
    const u64* __restrict__ src = srcs.at(blockIdx.z) + (u64)pos.prime[limb] * c.N + first;
#pragma unroll
    for (int r = 0; r < R; ++r) v[r] = ar.in_canon(ldg<2>(src + r * step + col));
  } else {
    const DevPrime P = c.primes[pi];
    const u32 lt = pos.prime[limb];
    const u64 ql = c.primes[f.last_prime].q, half = ql >> 1;
    const u64 K = f.sw[3 * lt], Kp = f.sw[3 * lt + 1], diff = f.sw[3 * lt + 2];
    // All words are requested before the first is used, and the cases below are uniform over the launch's
    // limb: a per-word branch would make every load wait for the one before it.
    u64 xs[R], ys[R];
    if (PRO == 1) {
      const u64* __restrict__ last = f.last + blockIdx.z * f.last_stride + first + col;
#pragma unroll
      for (int r = 0; r < R; ++r) xs[r] = last[r * step];
    } else {
      const u64* __restrict__ z = f.z + blockIdx.z * f.z_stride + first + col;
      const u64* __restrict__ yl = f.ylast + blockIdx.z * f.ylast_stride + first + col;
      const u64* __restrict__ src = srcs.at(blockIdx.z) + (u64)lt * c.N + first + col;
      u64 zs[R];
#pragma unroll
      for (int r = 0; r < R; ++r) { zs[r] = z[r * step]; xs[r] = yl[r * step]; ys[r] = ldg<2>(src + r * step); }
#pragma unroll
      for (int r = 0; r < R; ++r) xs[r] = sub_mod(zs[r], xs[r], ql);
      if (f.twice) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          xs[r] = add_mod(xs[r], xs[r], ql);
          ys[r] = add_mod(ys[r], ys[r], P.q);
        }
      }
    }
    if constexpr (A::kFp) {
      // Both primes small enough for FP64: the centred value of the last limb's word (|x| <= ql/2 <= q) times the
      // centred constant is one exact FP64 product, about a fifth of the integer path's instructions; its result
      // (below 0.93 q) is what the stages take.  With the source word added (PRO = 2) the sum is reduced once.
      if (ql < ((u64)1 << 52) && ql <= 2 * P.q) {
        const double qld = (double)ql, halfd = (double)half;
        double kc = ar.in_canon(K);
        if (K > (P.q >> 1)) kc -= ar.q;
        const double kci = kc * ar.qinv;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          double x = ar.in_canon(xs[r]);
          x = x > halfd ? x - qld : x;
          v[r] = ar.mulmod(x, kc, kci);
          if (PRO == 2) {
            v[r] += ar.in_canon(ys[r]);
            ar.reduce(v[r]);
          }
        }
        return;
      }
    }
    if (P.q > ql) {
#pragma unroll
      for (int r = 0; r < R; ++r) xs[r] += xs[r] > half ? P.q - ql : 0;
    } else if (ql < 2 * P.q) {
      // diff = 2 q - ql here, so a shifted word stays below 2 q
#pragma unroll
      for (int r = 0; r < R; ++r) xs[r] = csub(xs[r] + (xs[r] > half ? diff : 0), P.q);
    } else {
#pragma unroll
      for (int r = 0; r < R; ++r) xs[r] = barrett128(0, xs[r] + (xs[r] > half ? diff : 0), P);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      u64 w = shoup_mul(xs[r], K, Kp, P.q);
      if (PRO == 2) w = add_mod(w, ys[r], P.q);
      v[r] = ar.in_canon(w);
    }
  }
}

// forward, strided pass: stages 0..LOGR-1.  grid = (N/R/256, n_limbs, n_polys)
template <class A, int LOGR, int PRO>
__device__ __forceinline__ void fwd_strided_body(const DevCtx& c, const PolySeq& dsts, const PolySeq& srcs,
                                                 const LimbMap& pos, const FwdFuse& f, u32 limb, u32 pi) {
  constexpr int R = 1 << LOGR;
  const u32 col = blockIdx.x * 256 + threadIdx.x;
  const u64 rs = c.N >> LOGR;  // row stride
  // uniform row base + per-thread 32-bit column: rows are addressed off scalar registers
  u64* __restrict__ dst = dsts.at(blockIdx.z) + (u64)pos.prime[limb] * c.N;
  A ar;
  ar.init(c, pi, false, nullptr, 0);
  typename A::T v[R];
  fwd_strided_input<A, R, PRO>(ar, c, srcs, pos, f, limb, pi, col, 0, rs, v);
  fwd_strided_stages<A, LOGR>(ar, v);
  // this pass is bound by HBM and has instruction slots to spare: it hands centred values to the chunk pass,
  // which then runs its first two rounds (six stages) without reducing
  reduce_all<A, R>(ar, v);
#pragma unroll
  for (int r = 0; r < R; ++r) stg<1>(dst + r * rs + col, ar.out_mid(v[r]));
}
// One launch covers limbs of both arithmetic back ends: the choice is uniform over a work-group.
template <int LOGR, int PRO>
__global__ __launch_bounds__(256, 4) void ntt_fwd_strided(DevCtx c, PolySeq dsts, PolySeq srcs, LimbMap lm,
                                                       LimbMap pos, FwdFuse f) {
  const u32 limb = gridDim.y - 1 - blockIdx.y, pi = lm.prime[limb];  // last limbs first, as in the chunk passes
  if (c.fp_ok[pi]) fwd_strided_body<ArithFp, LOGR, PRO>(c, dsts, srcs, pos, f, limb, pi);
  else fwd_strided_body<ArithInt, LOGR, PRO>(c, dsts, srcs, pos, f, limb, pi);
}

// ---------------------------------------------------------------------------
// Base conversion and the forward strided pass of the converted limbs in one kernel (N = 2^16, at most eight source
// limbs): the conversion's result never goes to memory in coefficient form.  A work-group takes 64 columns of all
// sixteen rows of one operand (polynomial x digit).  Its four waves hold the source words of four rows each as the
// matrix product's operands (see baseconv_mx_kernel: a wave converts 64 coefficients of a row as two tiles of 32);
// the targets are taken four at a time: every wave converts its rows to the quad's targets into LDS
// ([target][row][column], 32 KiB), then wave w runs the four strided stages of target w of the quad, a column per
// lane, and stores what ntt_fwd_strided would have stored (centred values for the chunk pass).
// grid = (N/16/64, operands), 256 threads.
constexpr int kCfsCols = 64;
// The input word of FwdFuse::pro 2 from the dropped limb's word `last` (canonical mod q_last) and the converted word y
// (canonical mod q_t), one word at a time: the arithmetic of fwd_strided_input, whose cases are uniform over a limb.
template <class A>
struct SwitchIn {
  DevPrime P;
  u64 ql, half, K, Kp, diff;
  double qld, halfd, kc, kci;
  int mode;  // 0 FP64 product, 1 q > ql, 2 ql < 2 q, 3 Barrett
  __device__ __forceinline__ void init(const A& ar, const DevCtx& c, u32 pi, u32 last_prime, const u64* sw, u32 lt) {
    P = c.primes[pi];
    ql = c.primes[last_prime].q;
    half = ql >> 1;
    K = sw[3 * lt], Kp = sw[3 * lt + 1], diff = sw[3 * lt + 2];
    mode = P.q > ql ? 1 : ql < 2 * P.q ? 2 : 3;
    if constexpr (A::kFp) {
      if (ql < ((u64)1 << 52) && ql <= 2 * P.q) {
        mode = 0;
        qld = (double)ql, halfd = (double)half;
        kc = ar.in_canon(K);
        if (K > (P.q >> 1)) kc -= ar.q;
        kci = kc * ar.qinv;
      }
    }
  }
  __device__ __forceinline__ typename A::T one(const A& ar, u64 last, u64 y) const {
    if constexpr (A::kFp) {
      if (mode == 0) {
        double x = ar.in_canon(last);
        x = x > halfd ? x - qld : x;
        typename A::T v = ar.mulmod(x, kc, kci);
        v += ar.in_canon(y);
        ar.reduce(v);
        return v;
      }
    }
    u64 x = last;
    if (mode == 1) x += x > half ? P.q - ql : 0;
    else if (mode == 2) x = csub(x + (x > half ? diff : 0), P.q);
    else x = barrett128(0, x + (x > half ? diff : 0), P);
    return ar.in_canon(add_mod(shoup_mul(x, K, Kp, P.q), y, P.q));
  }
};
// the Rescale half of a transform that a Mod_down and a Rescale share (FwdFuse::pro 2), for the kernel below
struct ConvRescale {
  const u64* z;  // null: a plain conversion
  u64 z_stride;
  const u64* sw;
  u32 last_prime;
  u32 twice;  // FwdFuse::twice
};
template <class A, bool SWITCH>
__device__ __forceinline__ void conv_strided_column(const DevCtx& c, u32 pi, const u64* lds_target, u32 lane,
                                                    u64* __restrict__ dst, u64 rs, const ConvRescale& rz,
                                                    const u64* lds_last, u32 lt) {
  A ar;
  ar.init(c, pi, false, nullptr, 0);
  typename A::T v[16];
  if constexpr (SWITCH) {
    SwitchIn<A> in;
    in.init(ar, c, pi, rz.last_prime, rz.sw, lt);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      u64 y = lds_target[r * kCfsCols + lane];
      if (rz.twice) y = add_mod(y, y, in.P.q);
      v[r] = in.one(ar, lds_last[r * kCfsCols + lane], y);
    }
  } else {
#pragma unroll
    for (int r = 0; r < 16; ++r) v[r] = ar.in_canon(lds_target[r * kCfsCols + lane]);
  }
  fwd_strided_stages<A, 4>(ar, v);
  reduce_all<A, 16>(ar, v);
#pragma unroll
  for (int r = 0; r < 16; ++r) stg<1>(dst + r * rs + lane, ar.out_mid(v[r]));
}
// SWITCH: the conversion's last target is not transformed; it is the `ylast` of FwdFuse::pro 2, and every other
// target's transform starts from Switch_modulus(z - ylast) * sw + (converted word), as ntt_fwd_strided<., 2> forms it.
// The quad that holds the last target goes first, and z - ylast stays in LDS (8 KiB more) for the other quads.
template <int STEPS, bool SWITCH>
__global__ __launch_bounds__(256, SWITCH ? 3 : 4) void conv_fwd_strided_kernel(DevCtx c, u64* __restrict__ out_base,
                                                               const u64* __restrict__ t_base, ConvBatch b,
                                                               ConvRescale rz) {
  __shared__ __attribute__((aligned(16))) u64 lds[4 * 16 * kCfsCols];
  __shared__ u64 lds_last[SWITCH ? 16 * kCfsCols : 1];
  const u64 n = c.N, rs = n >> 4;
  const u32 lane = threadIdx.x & 63, half = lane >> 5;
  const u32 wv = (u32)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const u32 col0 = blockIdx.x * kCfsCols;
  const u32 jobi = blockIdx.y % b.n_jobs, op = blockIdx.y / b.n_jobs;
  const ConvJob& J = b.job[jobi];
  const u32 nd = J.nd, nc = J.nc;
  const u64* __restrict__ t = t_base + op * b.t_stride + J.t_off + col0 + 2 * (lane & 31);
  u64* __restrict__ out = out_base + op * b.out_stride + J.out_off + col0;
  conv_v4i x[4][2][STEPS];
  {
    typedef u64 u64x2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      u64x2 v[STEPS][2];
#pragma unroll
      for (int s = 0; s < STEPS; ++s)
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          const u32 k = 4 * s + 2 * half + w;
          v[s][w] = ldg<2>(reinterpret_cast<const u64x2*>(t + (u64)min(k, nd - 1) * n + (u64)(4 * wv + rr) * rs));
        }
#pragma unroll
      for (int s = 0; s < STEPS; ++s)
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          const bool live = 4 * s + 2 * half + w < nd;
          int lo, hi;
          conv_mx_signed(v[s][w].x, live, lo, hi);
          x[rr][0][s][2 * w] = lo;
          x[rr][0][s][2 * w + 1] = hi;
          conv_mx_signed(v[s][w].y, live, lo, hi);
          x[rr][1][s][2 * w] = lo;
          x[rr][1][s][2 * w + 1] = hi;
        }
    }
  }
  const uint4* __restrict__ mx = J.mx + lane;
  const ConvTarget* __restrict__ mt = J.mt;
  const u32 quads = (nc + 3) / 4;
  // the order of the quads: as they lie, or, SWITCH, the last one first
  auto quad_at = [&](u32 k) { return !SWITCH ? k : k == 0 ? quads - 1 : k - 1; };
  uint4 row[STEPS];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) row[s] = mx[((u64)quad_at(0) * kMxSteps + s) * 64];
  for (u32 k = 0; k < quads; ++k) {
    const u32 quad = quad_at(k);
    const ConvTarget tg[2] = {mt[quad * 4 + 2 * half], mt[quad * 4 + 2 * half + 1]};
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      conv_v16i acc[2];
#pragma unroll
      for (u32 tile = 0; tile < 2; ++tile) {
        acc[tile] = conv_v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
          const conv_v4i a = {(int)row[s].x, (int)row[s].y, (int)row[s].z, (int)row[s].w};
          acc[tile] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, x[rr][tile][s], acc[tile], 0, 0, 0);
        }
      }
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        typedef u64 u64x2 __attribute__((ext_vector_type(2)));
        const u64x2 pr = {conv_mx_residue(acc[0], w, tg[w].m, tg[w].minv), conv_mx_residue(acc[1], w, tg[w].m, tg[w].minv)};
        *reinterpret_cast<u64x2*>(lds + ((2 * half + w) * 16 + 4 * wv + rr) * kCfsCols + 2 * (lane & 31)) = pr;
      }
    }
    __syncthreads();
    {
      // the next quad's rows are asked for now and arrive while the columns are transformed (the tables end with a
      // spare quad, which the last round reads)
      const u32 quad_next = k + 1 < quads ? quad_at(k + 1) : quads;
#pragma unroll
      for (int s = 0; s < STEPS; ++s) row[s] = mx[((u64)quad_next * kMxSteps + s) * 64];
    }
    if (SWITCH && k == 0) {
      const u64 ql = c.primes[rz.last_prime].q;
      const u64* __restrict__ z = rz.z + op * rz.z_stride + col0;
      const u64* ylast = lds + ((nc - 1) & 3) * 16 * kCfsCols;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const u32 p = threadIdx.x + 256 * i;  // row p / 64, column p % 64
        u64 last = sub_mod(z[(u64)(p >> 6) * rs + (p & 63)], ylast[p], ql);
        if (rz.twice) last = add_mod(last, last, ql);
        lds_last[p] = last;
      }
      __syncthreads();
    }
    const u32 j = quad * 4 + wv;
    if (j < (SWITCH ? nc - 1 : nc)) {  // uniform over the wave
      const u32 pi = J.map.prime[j], lt = J.map.out_limb[j];
      u64* __restrict__ dst = out + (u64)lt * n;
      if (c.fp_ok[pi]) conv_strided_column<ArithFp, SWITCH>(c, pi, lds + wv * 16 * kCfsCols, lane, dst, rs, rz, lds_last, lt);
      else conv_strided_column<ArithInt, SWITCH>(c, pi, lds + wv * 16 * kCfsCols, lane, dst, rs, rz, lds_last, lt);
    }
    __syncthreads();
  }
}

bool launch_baseconv_fwd_strided(hipStream_t st, const DevCtx& c, u64* out, const u64* t, const ConvBatch& b, u32 n_ops,
                                 const FwdFuse* rescale) {
  static const bool on = [] {
    const char* e = getenv("ACE_CONV_STRIDED");
    return !e || e[0] != '0';
  }();
  if (!on || !b.matrix || !b.n_jobs || !n_ops || c.logN != 16) return false;
  u32 max_nd = 0;
  u64 limbs = 0;
  for (u32 k = 0; k < b.n_jobs; ++k) {
    if (!b.job[k].mx || !b.job[k].nc) return false;
    max_nd = b.job[k].nd > max_nd ? b.job[k].nd : max_nd;
    limbs += b.job[k].nc;
  }
  // launches too small for the machine are better served by the two kernels (the strided pass spread over four waves
  // a column); more than eight source limbs would not fit the registers
  if (max_nd > 8 || limbs * n_ops < 192) return false;
  if ((((uintptr_t)out | (uintptr_t)t) & 15) || ((b.out_stride | b.t_stride) & 1)) return false;
  dim3 g((u32)(c.N >> 4) / kCfsCols, b.n_jobs * n_ops);
  ConvRescale rz{};
  if (rescale) {
    // the prologue that a Mod_down and a Rescale share: one job whose last target is the dropped limb's `ylast`,
    // written where the conversion puts it but read from LDS here
    const ConvJob& J = b.job[0];
    if (rescale->pro != 2 || b.n_jobs != 1 || J.nc < 2 || J.map.out_limb[J.nc - 1] != J.nc - 1 ||
        rescale->ylast != out + J.out_off + (u64)(J.nc - 1) * c.N || rescale->ylast_stride != b.out_stride)
      return false;
    rz = ConvRescale{rescale->z, rescale->z_stride, rescale->sw, rescale->last_prime, rescale->twice};
    if (max_nd <= 4) hipLaunchKernelGGL((conv_fwd_strided_kernel<1, true>), g, dim3(256), 0, st, c, out, t, b, rz);
    else hipLaunchKernelGGL((conv_fwd_strided_kernel<2, true>), g, dim3(256), 0, st, c, out, t, b, rz);
    return true;
  }
  if (max_nd <= 4) hipLaunchKernelGGL((conv_fwd_strided_kernel<1, false>), g, dim3(256), 0, st, c, out, t, b, rz);
  else hipLaunchKernelGGL((conv_fwd_strided_kernel<2, false>), g, dim3(256), 0, st, c, out, t, b, rz);
  return true;
}

// Work-group -> (chunk, limb, polynomial slot) for the chunk passes.  The grid
// is one-dimensional.  Hardware hands consecutive work-groups to the 8 XCDs in
// turn and each XCD has its own 4 MiB L2.  The map below gives every XCD whole
// (limb, chunk) groups, so that the polynomials of a group find the group's
// 32 KiB of twiddles in that L2.  (Measured with FETCH_SIZE on a 32-polynomial
// batch at N=2^16, 24 primes: 12 MiB of twiddle fetches with all polynomials of
// a group back to back, 230 MiB with groups varying fastest over all XCDs, where
// 4.6 MB of streaming data passes through the L2 between two uses of the same
// twiddles.)
// Within an XCD the slots of a group (its polynomials, or runs of them) are not all run back to back: work-groups
// that run at the same time would then touch the same chunk of many polynomials, whose addresses differ by multiples
// of the polynomial stride and crowd the same memory channels (chunk passes of the 768-limb batch in runs: 0.149 ->
// 0.141 ms forward, 0.159 -> 0.148 ms inverse).  The groups of an XCD are visited `visit` slots at a time: all groups
// for the first `visit` slots, then all groups for the next ones.  One slot per visit for the run kernels (SLOT_MAJOR),
// whose work-groups keep their twiddles in registers over a run; ACE_NTT_VISIT (4) for the others where a group has
// at least twice as many slots, so that a group's twiddles are in the L2 for the few work-groups that share them at a
// time and come from the memory-side cache on later visits; all slots (the plain limb-major order) otherwise.
#ifndef ACE_NTT_VISIT
#define ACE_NTT_VISIT 4
#endif
template <bool SLOT_MAJOR>
__host__ __device__ __forceinline__ u32 chunk_visit(u32 slots_per_group) {
  if (SLOT_MAJOR) return 1;
  return slots_per_group >= 2 * ACE_NTT_VISIT ? ACE_NTT_VISIT : slots_per_group;
}
template <int LOGC = kLogChunk, bool SLOT_MAJOR = false>
__device__ __forceinline__ bool chunk_block(const DevCtx& c, u32 n_limbs, u32 slots_per_group, u32& chunk,
                                            u32& limb, u32& slot_in_group) {
  const u32 n_chunks = c.N >> LOGC, n_groups = n_limbs * n_chunks;
  const u32 id = blockIdx.x, xcd = id & 7, slot = id >> 3;
  const u32 visit = chunk_visit<SLOT_MAJOR>(slots_per_group), per_xcd = (n_groups + 7) / 8;
  const u32 grp = ((slot / visit) % per_xcd) * 8 + xcd;
  slot_in_group = (slot / (visit * per_xcd)) * visit + slot % visit;
  if (grp >= n_groups || slot_in_group >= slots_per_group) return false;
  chunk = grp % n_chunks;
  // last limbs first: where a launch mixes back ends, the special primes (integer back end, 2.5x the work) sit at
  // the end of the limb list and should not be the tail of the launch
  limb = n_limbs - 1 - grp / n_chunks;
  return true;
}
template <bool SLOT_MAJOR = false>
static inline unsigned chunk_grid(const DevCtx& c, u32 n_limbs, u32 slots_per_group, int logc = kLogChunk) {
  const u32 n_groups = n_limbs * (c.N >> logc), visit = chunk_visit<SLOT_MAJOR>(slots_per_group);
  return ((n_groups + 7) / 8) * 8 * ((slots_per_group + visit - 1) / visit) * visit;
}

// Polynomials handled by one work-group of a chunk pass.  They share the
// (limb, chunk) pair; the next polynomial's words are requested before the
// current one is transformed.
#ifndef ACE_NTT_PB
#define ACE_NTT_PB 1
#endif
constexpr int kPolysPerBlock = ACE_NTT_PB;
#ifndef ACE_NTT_SHIFT
#define ACE_NTT_SHIFT 1
#endif
constexpr int kChunkThreads = 512;  // 8 coefficients per thread
#ifndef ACE_NTT_WAVES
#define ACE_NTT_WAVES 8
#endif
constexpr int kChunkWaves = ACE_NTT_WAVES;  // waves per SIMD the chunk kernels are compiled for

// The four thread -> element maps of a chunk pass (r = 0..7).  Each covers the
// chunk once and keeps the eight elements of three consecutive stages' worth of
// butterflies in one thread:
//   wide    t + 512 r                      spans 2048, 1024, 512  (also the coalesced global order)
//   wave    (t/64)*512 + 64 r + t%64       spans 256, 128, 64     (twiddles are wave-uniform)
//   octet   h*64 + 8 r + t%8               spans 32, 16, 8        (h = t/8 with its two low bits swapped, which
//                                                                  puts the two h of a 16-lane group 8 banks apart)
//   narrow  8 t + r                        spans 4, 2, 1
struct ChunkMap {
  int wide, wave, octet, narrow;  // LDS positions of element r = 0; element r is at +off(r)
  u32 wv, h;
  __device__ __forceinline__ ChunkMap(int t) {
    wv = (u32)__builtin_amdgcn_readfirstlane(t >> 6);
    const u32 a = (u32)t >> 3;
    h = (a & ~3u) | ((a & 1u) << 1) | ((a >> 1) & 1u);
    wide = lds_pos(t);
    wave = lds_pos((int)(wv * 512) + (t & 63));
    octet = lds_pos((int)(h * 64) + (t & 7));
    narrow = lds_pos(t * 8);
  }
  // lds_pos(e0 + d) == lds_pos(e0) + d + (d >> 4) whenever (e0 & 15) + (d & 15) < 16, which holds for
  // each map's increments below
  static __device__ __forceinline__ constexpr int wide_off(int r) { return 512 * r + 32 * r; }
  static __device__ __forceinline__ constexpr int wave_off(int r) { return 64 * r + 4 * r; }
  static __device__ __forceinline__ constexpr int octet_off(int r) { return 8 * r + (r >> 1); }
  static __device__ __forceinline__ constexpr int narrow_off(int r) { return r; }
};

// What a forward chunk pass with an epilogue (FwdFuse::epi) does with the chunk it has transformed, in place of storing
// it: the words lie in LDS in canonical form (`ldsu`, wave order: a wave reads the words it wrote); p is the
// polynomial, lt its limb's place, pi the prime.  barrier_after_gather: the caller writes the LDS again without a
// work-group barrier of its own.
template <int EPI>
__device__ __forceinline__ void fwd_chunk_tail(const DevCtx& c, const FwdFuse& f, u64* ldsu, const ChunkMap& cm, int t,
                                               u32 wpos, u32 p, u32 lt, u32 pi, u32 chunk, bool barrier_after_gather) {
  const u64 q = c.primes[pi].q, w = f.cst[2 * lt], wp = f.cst[2 * lt + 1];
  const u64* addend =
      (EPI == 1 && (f.addend_mode == 1 || (f.addend_mode == 2 && !(p & 1)))) ? f.addend.at(p) + (u64)lt * c.N : nullptr;
  if (EPI == 1 && f.orders.n) {
    // The automorphism on the way out: this chunk of the transform is the source of one chunk of the result.
    // The tail is formed at the source positions, operands read in the wave order like the plain tail's, and put
    // back into LDS in place of the transform's words; the result chunk is then gathered from LDS, so that no
    // global access is scattered.
    const i64* __restrict__ order = f.orders.p[f.orders.n == 1 ? 0 : (p >> 1)];
    const u32 n_chunks = c.N >> kLogChunk;
    u32 dc = chunk;
    for (u32 cc = 0; cc < n_chunks; ++cc)
      if ((u32)((u64)order[(u64)cc * kChunk] >> kLogChunk) == chunk) dc = cc;
    order += (u64)dc * kChunk + t;
    const u64 so = (u64)lt * c.N + (u64)chunk * kChunk + wpos;  // where this thread's operands lie
    u64* __restrict__ out = f.out.at(p) + (u64)lt * c.N + (u64)dc * kChunk + t;  // never an operand (checked by the callers)
    const u64* __restrict__ src = f.src.at(p) + so;
    if (addend) addend += (u64)chunk * kChunk + wpos;
    u32 s8[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) s8[r] = (u32)order[512 * r] & (u32)(kChunk - 1);
#pragma unroll
    for (int r0 = 0; r0 < 8; r0 += 4) {
      u64 sv[4], av[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) sv[r] = ldg<32>(src + 64 * (r0 + r));
      if (addend) {
#pragma unroll
        for (int r = 0; r < 4; ++r) av[r] = ldg<32>(addend + 64 * (r0 + r));
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int at = cm.wave + ChunkMap::wave_off(r0 + r);
        u64 v = shoup_mul(sub_mod(sv[r], ldsu[at], q), w, wp, q);
        if (addend) v = add_mod(v, av[r], q);
        ldsu[at] = v;
      }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 8; ++r) stg<16>(out + 512 * r, ldsu[lds_pos((int)s8[r])]);
    if (barrier_after_gather) __syncthreads();  // the gathered LDS reads are not the words this thread writes next
  } else {
    const u64 o = (u64)lt * c.N + (u64)chunk * kChunk + wpos;
    u64* out = f.out.at(p) + o;  // may alias the addend (in-place relinearisation)
    const u64* __restrict__ src = f.src.at(p) + o;
    if (addend) addend += (u64)chunk * kChunk + wpos;
    // four words at a time: the operands of all eight would not fit beside the 64 registers of a thread
#pragma unroll
    for (int r0 = 0; r0 < 8; r0 += 4) {
      u64 sv[4], av[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) sv[r] = ldg<32>(src + 64 * (r0 + r));
      if (addend) {
#pragma unroll
        for (int r = 0; r < 4; ++r) av[r] = ldg<32>(addend + 64 * (r0 + r));
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const u64 y = ldsu[cm.wave + ChunkMap::wave_off(r0 + r)];
        u64 v;
        if (EPI == 1) {
          v = shoup_mul(sub_mod(sv[r], y, q), w, wp, q);
          if (addend) v = add_mod(v, av[r], q);
        } else {
          u64 scaled = shoup_mul(sv[r], w, wp, q);
          if (f.twice) scaled = add_mod(scaled, scaled, q);
          v = add_mod(scaled, y, q);
        }
        stg<16>(out + 64 * (r0 + r), v);
      }
    }
  }
}

// forward, chunk pass: stages logr..logN-1 on 4096 contiguous words, in place.
// grid = chunk_grid(n_limbs, ceil(n_polys / kPolysPerBlock)), 512 threads: four
// rounds of three stages with the chunk passing through LDS between them, and
// once more so that the global store is coalesced.  A thread writes back the
// positions it read, so one barrier per round suffices.
// EPI != 0: the result is not stored back but consumed by FwdFuse::epi.
template <class A, int EPI, int SKIP>
__device__ __forceinline__ void fwd_chunk_body(u64* lds_words, const DevCtx& c, const PolySeq& datas,
                                               const LimbMap& pos, u32 logr, u32 n_polys, const FwdFuse& f, u32 chunk,
                                               u32 limb, u32 pblk, u32 pi) {
  typedef typename A::T T;
  T* lds = reinterpret_cast<T*>(lds_words);
  const int t = threadIdx.x;
  const u32 poly0 = pblk * kPolysPerBlock;
  const u32 cnt = min((u32)kPolysPerBlock, n_polys - poly0);
  const u64 loff = (u64)pos.prime[limb] * c.N + (u64)chunk * kChunk;
  u64* base = datas.at(poly0) + loff;
  A ar;
  ar.init(c, pi, false, nullptr, 0);
  const ChunkMap cm(t);
  // twiddle index of local stage ls, local group g of this chunk: (m0 << ls) + (chunk << ls) + g
  const u32 tw0 = (1u << logr) + chunk;
  u64 raw[8], nxt[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) raw[r] = ldg<8>(base + t + 512 * r);
  for (u32 it = 0; it < cnt; ++it) {
    base = datas.at(poly0 + it) + loff;
    if (it + 1 < cnt) {
      const u64* nb = datas.at(poly0 + it + 1) + loff;
#pragma unroll
      for (int r = 0; r < 8; ++r) nxt[r] = nb[t + 512 * r];
    }
    T v[8];
    // local stages 0..2
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = ar.in_mid(raw[r]);  // centred by the strided pass
    if (!SKIP) ct_stage<A, 8, 0>(ar, v, tw0 << 0);  // else the strided pass has run this stage as its last
    ct_stage<A, 8, 1>(ar, v, tw0 << 1);
    ct_stage<A, 8, 2>(ar, v, tw0 << 2);
#pragma unroll
    for (int r = 0; r < 8; ++r) lds[cm.wide + ChunkMap::wide_off(r)] = v[r];
    __syncthreads();
    // local stages 3..5: local group = (wv << (ls-3)) + g
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = lds[cm.wave + ChunkMap::wave_off(r)];
    ct_stage<A, 8, 0>(ar, v, (tw0 << 3) + (cm.wv << 0));
    ct_stage<A, 8, 1>(ar, v, (tw0 << 4) + (cm.wv << 1));
    ct_stage<A, 8, 2>(ar, v, (tw0 << 5) + (cm.wv << 2));
#pragma unroll
    for (int r = 0; r < 8; ++r) lds[cm.wave + ChunkMap::wave_off(r)] = v[r];
    wave_sync();  // the words read next were written by this wave
    // local stages 6..8: local group = (h << (ls-6)) + g
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = lds[cm.octet + ChunkMap::octet_off(r)];
    reduce_all<A, 8>(ar, v);
    ct_stage<A, 8, 0>(ar, v, (tw0 << 6) + (cm.h << 0));
    ct_stage<A, 8, 1>(ar, v, (tw0 << 7) + (cm.h << 1));
    ct_stage<A, 8, 2>(ar, v, (tw0 << 8) + (cm.h << 2));
#pragma unroll
    for (int r = 0; r < 8; ++r) lds[cm.octet + ChunkMap::octet_off(r)] = v[r];
    wave_sync();  // the words read next were written by this wave
    // local stages 9..11: local group = (t << (ls-9)) + g
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = lds[cm.narrow + ChunkMap::narrow_off(r)];
    ct_stage<A, 8, 0>(ar, v, (tw0 << 9) + ((u32)t << 0));
    ct_stage<A, 8, 1>(ar, v, (tw0 << 10) + ((u32)t << 1));
    ct_stage<A, 8, 2>(ar, v, (tw0 << 11) + ((u32)t << 2));
    u64* ldsu = lds_words;
#pragma unroll
    for (int r = 0; r < 8; ++r) ldsu[cm.narrow + ChunkMap::narrow_off(r)] = ar.out_canon(v[r]);
    // The result leaves in the wave order (lane + 64 r inside the 512 words a wave owns): 512 contiguous bytes
    // per store instruction, and every word a wave stores was written by that wave, so no work-group barrier is
    // needed.  Only the automorphism gathers from the whole chunk (after a barrier of its own).
    wave_sync();
    const u32 wpos = cm.wv * 512 + ((u32)t & 63);  // first of this thread's words in the wave order
    if (EPI == 0) {
#pragma unroll
      for (int r = 0; r < 8; ++r) stg<4>(base + wpos + 64 * r, ldsu[cm.wave + ChunkMap::wave_off(r)]);
    } else {
      fwd_chunk_tail<EPI>(c, f, ldsu, cm, t, wpos, poly0 + it, pos.prime[limb], pi, chunk, kPolysPerBlock > 1);
    }
    // the next polynomial's first round writes words that other waves may still be reading
    if (kPolysPerBlock > 1) __syncthreads();
#pragma unroll
    for (int r = 0; r < 8; ++r) raw[r] = nxt[r];
  }
}
// (the Mod_down tail keeps three more pointers and constants alive: 80 registers, 6 waves per SIMD)
template <int EPI, int SKIP>
__global__ __launch_bounds__(kChunkThreads, kChunkWaves) void ntt_fwd_chunk(DevCtx c, PolySeq datas, LimbMap lm, LimbMap pos,
                                                                  u32 logr, u32 n_limbs, u32 n_polys, FwdFuse f) {
  __shared__ u64 lds[kChunk + kChunk / 16];
  u32 chunk, limb, pblk;
  if (!chunk_block(c, n_limbs, (n_polys + kPolysPerBlock - 1) / kPolysPerBlock, chunk, limb, pblk)) return;
  const u32 pi = lm.prime[limb];
  if (c.fp_ok[pi]) fwd_chunk_body<ArithFp, EPI, SKIP>(lds, c, datas, pos, logr, n_polys, f, chunk, limb, pblk, pi);
  else fwd_chunk_body<ArithInt, EPI, SKIP>(lds, c, datas, pos, logr, n_polys, f, chunk, limb, pblk, pi);
}

// The forward chunk pass for launches of many polynomials whose limbs are all on the FP64 back end, in runs of
// `run` polynomials per work-group with the next polynomial's words on their way into LDS meanwhile (see
// ntt_inv_half_run below for the scheme and its reasons).  A wave stages the 512 words its first round works on
// (lane + 512 r of the chunk's 64-word column group): staging load j brings the 16-byte pairs of r = 2j (lanes 0-31)
// and r = 2j + 1 (lanes 32-63), which land as [r][lane] in the wave's 4 KiB.  66 KiB of LDS per work-group: two
// work-groups, 16 waves, per CU.
__global__ __launch_bounds__(kChunkThreads, 4) void ntt_fwd_chunk_run(DevCtx c, PolySeq datas, LimbMap lm, LimbMap pos,
                                                                    u32 logr, u32 n_limbs, u32 n_polys, u32 run) {
  typedef ArithFp A;
  __shared__ double lds[kChunk + kChunk / 16];
  __shared__ __attribute__((aligned(16))) u64 stage[kChunk];
  u32 chunk, limb, pblk;
  if (!chunk_block<kLogChunk, true>(c, n_limbs, (n_polys + run - 1) / run, chunk, limb, pblk)) return;
  // last polynomials first: the strided pass before this one has written them last, and part of them is still in
  // the memory-side cache
  pblk = (n_polys + run - 1) / run - 1 - pblk;
  const u32 pi = lm.prime[limb];
  const int t = threadIdx.x;
  const u32 poly0 = pblk * run;
  const u32 cnt = min(run, n_polys - poly0);
  const u64 loff = (u64)pos.prime[limb] * c.N + (u64)chunk * kChunk;
  A ar;
  ar.init(c, pi, false, nullptr, 0);
  const ChunkMap cm(t);
  const u32 lane = (u32)t & 63;
  u64* mine = stage + cm.wv * 512;
  auto request = [&](u32 poly) {
    const u64* src = datas.at(poly) + loff + cm.wv * 64 + 2 * (lane & 31) + 512 * (lane >> 5);
#pragma unroll
    for (int j = 0; j < 4; ++j) stage_request(src + 1024 * j, mine + 128 * j);
  };
  // twiddle index of local stage ls, local group g of this chunk: (m0 << ls) + (chunk << ls) + g
  const u32 tw0 = (1u << logr) + chunk;
  A::TWL a0[1], a1[2], a2[4], b0[1], b1[2], b2[4], c0[1], c1[2], c2[4], d0[1], d1[2], d2[4];
  ar.load_tw<1>(tw0 << 0, a0);
  ar.load_tw<2>(tw0 << 1, a1);
  ar.load_tw<4>(tw0 << 2, a2);
  ar.load_tw<1>((tw0 << 3) + (cm.wv << 0), b0);
  ar.load_tw<2>((tw0 << 4) + (cm.wv << 1), b1);
  ar.load_tw<4>((tw0 << 5) + (cm.wv << 2), b2);
  ar.load_tw<1>((tw0 << 6) + (cm.h << 0), c0);
  ar.load_tw<2>((tw0 << 7) + (cm.h << 1), c1);
  ar.load_tw<4>((tw0 << 8) + (cm.h << 2), c2);
  ar.load_tw<1>((tw0 << 9) + ((u32)t << 0), d0);
  ar.load_tw<2>((tw0 << 10) + ((u32)t << 1), d1);
  ar.load_tw<4>((tw0 << 11) + ((u32)t << 2), d2);
  {  // the compiler waits for the per-lane ones here, so that its count of pending loads is zero afterwards
    auto use = [](double& x) { asm volatile("" : "+v"(x)); };
    use(c0[0]);
    for (auto& x : c1) use(x);
    for (auto& x : c2) use(x);
    use(d0[0]);
    for (auto& x : d1) use(x);
    for (auto& x : d2) use(x);
  }
  request(poly0);
  u64* ldsu = reinterpret_cast<u64*>(lds);
  for (u32 it = 0; it < cnt; ++it) {
    // this polynomial's words are in LDS: its four loads are older than the eight stores of the previous one
    if (it == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    double v[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = ar.in_mid(mine[64 * r + lane]);  // centred by the strided pass
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // in registers before the next ones overwrite them
    if (it + 1 < cnt) request(poly0 + it + 1);
    ct_stage_pre<A, 8, 0>(ar, v, a0);
    ct_stage_pre<A, 8, 1>(ar, v, a1);
    ct_stage_pre<A, 8, 2>(ar, v, a2);
    __syncthreads();  // the previous polynomial's results have left the words written next (other waves stored them)
#pragma unroll
    for (int r = 0; r < 8; ++r) lds[cm.wide + ChunkMap::wide_off(r)] = v[r];
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = lds[cm.wave + ChunkMap::wave_off(r)];
    ct_stage_pre<A, 8, 0>(ar, v, b0);
    ct_stage_pre<A, 8, 1>(ar, v, b1);
    ct_stage_pre<A, 8, 2>(ar, v, b2);
#pragma unroll
    for (int r = 0; r < 8; ++r) lds[cm.wave + ChunkMap::wave_off(r)] = v[r];
    wave_sync();  // the words read next were written by this wave
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = lds[cm.octet + ChunkMap::octet_off(r)];
    reduce_all<A, 8>(ar, v);
    ct_stage_pre<A, 8, 0>(ar, v, c0);
    ct_stage_pre<A, 8, 1>(ar, v, c1);
    ct_stage_pre<A, 8, 2>(ar, v, c2);
#pragma unroll
    for (int r = 0; r < 8; ++r) lds[cm.octet + ChunkMap::octet_off(r)] = v[r];
    wave_sync();  // the words read next were written by this wave
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = lds[cm.narrow + ChunkMap::narrow_off(r)];
    ct_stage_pre<A, 8, 0>(ar, v, d0);
    ct_stage_pre<A, 8, 1>(ar, v, d1);
    ct_stage_pre<A, 8, 2>(ar, v, d2);
#pragma unroll
    for (int r = 0; r < 8; ++r) ldsu[cm.narrow + ChunkMap::narrow_off(r)] = ar.out_canon(v[r]);
    wave_sync();  // the result leaves in the wave order: every word a wave stores was written by that wave
    u64* out = datas.at(poly0 + it) + loff + cm.wv * 512 + lane;
#pragma unroll
    for (int r = 0; r < 8; ++r) stg<4>(out + 64 * r, ldsu[cm.wave + ChunkMap::wave_off(r)]);
  }
}

// ---------------------------------------------------------------------------
// inverse, chunk pass: spans 1..2048 on 4096 contiguous words; src -> dst.
// Nothing is scaled here: 1/N (times an optional per-limb constant) is applied
// by the strided pass that always follows.  The first round works on the eight
// consecutive words a thread loads itself.  At span 2^u the stage has
// m = N >> (u+1) groups and element j belongs to group j >> (u+1).  The rounds
// are those of the forward pass in reverse order.
template <class A, int SKIP, int COPY>
__device__ __forceinline__ void inv_chunk_body(u64* lds_words, const DevCtx& c, const PolySeq& dsts,
                                               const PolySeq& srcs, const CopyThrough& copies, const LimbMap& pos,
                                               u32 n_polys, u32 chunk, u32 limb, u32 pblk, u32 pi) {
  typedef typename A::T T;
  T* lds = reinterpret_cast<T*>(lds_words);
  const int t = threadIdx.x;
  const u32 poly0 = pblk * kPolysPerBlock;
  const u32 cnt = min((u32)kPolysPerBlock, n_polys - poly0);
  const u64 off = (u64)pos.prime[limb] * c.N + (u64)chunk * kChunk;
  A ar;
  ar.init(c, pi, true, nullptr, 0);
  const ChunkMap cm(t);
  const u32 mh = c.N >> 1;  // groups at span 1
  // A thread reads the eight consecutive words its first round works on (64 bytes, 16-byte loads): no pass
  // through LDS before the first stage.  Where a copy of the words is wanted as well (the digits that Mod_up
  // passes through), they are read in the coalesced order instead, copied from registers 512 contiguous bytes per
  // store (16-byte stores 64 bytes apart are slow) and brought into the first round's order through LDS.
  constexpr bool copying = COPY != 0;
  u64 raw[8], nxt[8];
  auto load8 = [&](u64* into, u32 poly) {
    if (copying) {
      const u64* src = srcs.at(poly) + off + t;
#pragma unroll
      for (int r = 0; r < 8; ++r) into[r] = src[512 * r];
    } else {
      const ulonglong2* src2 = reinterpret_cast<const ulonglong2*>(srcs.at(poly) + off + 8 * t);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const ulonglong2 x = src2[k];
        into[2 * k] = x.x;
        into[2 * k + 1] = x.y;
      }
    }
  };
  load8(raw, poly0);
  for (u32 it = 0; it < cnt; ++it) {
    u64* dst = dsts.at(poly0 + it);
    if (it + 1 < cnt) load8(nxt, poly0 + it + 1);
    T v[8];
    if (copying) {
      u64* cp = copies.seq.at(poly0 + it) + (u64)(pos.prime[limb] / copies.part_size) * copies.digit_stride;
#pragma unroll
      for (int r = 0; r < 8; ++r) cp[off + t + 512 * r] = raw[r];
#pragma unroll
      for (int r = 0; r < 8; ++r) lds[cm.wide + ChunkMap::wide_off(r)] = ar.in_canon(raw[r]);
      __syncthreads();
#pragma unroll
      for (int r = 0; r < 8; ++r) v[r] = lds[cm.narrow + ChunkMap::narrow_off(r)];
    } else {
#pragma unroll
      for (int r = 0; r < 8; ++r) v[r] = ar.in_canon(raw[r]);
    }
    // spans 1, 2, 4
    gs_stage<A, 8, 0>(ar, v, (mh >> 0) + (chunk << 11) + ((u32)t << 2));
    gs_stage<A, 8, 1>(ar, v, (mh >> 1) + (chunk << 10) + ((u32)t << 1));
    ar.recentre_sum_of_four(v[0]);
    ar.recentre_sum_of_four(v[4]);
    gs_stage<A, 8, 2>(ar, v, (mh >> 2) + (chunk << 9) + ((u32)t << 0));
#pragma unroll
    for (int r = 0; r < 8; ++r) lds[cm.narrow + ChunkMap::narrow_off(r)] = v[r];
    wave_sync();  // the words read next were written by this wave
    // spans 8, 16, 32
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = lds[cm.octet + ChunkMap::octet_off(r)];
    reduce_all<A, 8>(ar, v);
    gs_stage<A, 8, 0>(ar, v, (mh >> 3) + (chunk << 8) + (cm.h << 2));
    gs_stage<A, 8, 1>(ar, v, (mh >> 4) + (chunk << 7) + (cm.h << 1));
    gs_stage<A, 8, 2>(ar, v, (mh >> 5) + (chunk << 6) + (cm.h << 0));
#pragma unroll
    for (int r = 0; r < 8; ++r) lds[cm.octet + ChunkMap::octet_off(r)] = v[r];
    wave_sync();  // the words read next were written by this wave
    // spans 64, 128, 256
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = lds[cm.wave + ChunkMap::wave_off(r)];
    reduce_all<A, 8>(ar, v);
    gs_stage<A, 8, 0>(ar, v, (mh >> 6) + (chunk << 5) + (cm.wv << 2));
    gs_stage<A, 8, 1>(ar, v, (mh >> 7) + (chunk << 4) + (cm.wv << 1));
    gs_stage<A, 8, 2>(ar, v, (mh >> 8) + (chunk << 3) + (cm.wv << 0));
#pragma unroll
    for (int r = 0; r < 8; ++r) lds[cm.wave + ChunkMap::wave_off(r)] = v[r];
    __syncthreads();
    // spans 512, 1024, 2048; twiddles are uniform over the work-group.  The words read here are the
    // ones this thread overwrites first in the next iteration.
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = lds[cm.wide + ChunkMap::wide_off(r)];
    reduce_all<A, 8>(ar, v);
    gs_stage<A, 8, 0>(ar, v, (mh >> 9) + (chunk << 2));
    gs_stage<A, 8, 1>(ar, v, (mh >> 10) + (chunk << 1));
    if (!SKIP) gs_stage<A, 8, 2>(ar, v, (mh >> 11) + (chunk << 0));  // else the strided pass runs it as its first
#pragma unroll
    for (int r = 0; r < 8; ++r) stg<512>(dst + off + t + 512 * r, ar.out_mid(v[r]));
    if (kPolysPerBlock > 1) __syncthreads();  // the next polynomial's first round writes words other waves still read
#pragma unroll
    for (int r = 0; r < 8; ++r) raw[r] = nxt[r];
  }
}
// (compiled for six waves per SIMD: at eight, 64 registers, the integer body spills; the launches this kernel serves
// are those of whole programs, far too small to fill eight)
template <int SKIP, int COPY>
__global__ __launch_bounds__(kChunkThreads, 6) void ntt_inv_chunk(DevCtx c, PolySeq dsts, PolySeq srcs, CopyThrough copies,
                                                                  LimbMap lm, LimbMap pos, u32 n_limbs, u32 n_polys) {
  __shared__ u64 lds[kChunk + kChunk / 16];
  u32 chunk, limb, pblk;
  if (!chunk_block(c, n_limbs, (n_polys + kPolysPerBlock - 1) / kPolysPerBlock, chunk, limb, pblk)) return;
  const u32 pi = lm.prime[limb];
  if (c.fp_ok[pi]) inv_chunk_body<ArithFp, SKIP, COPY>(lds, c, dsts, srcs, copies, pos, n_polys, chunk, limb, pblk, pi);
  else inv_chunk_body<ArithInt, SKIP, COPY>(lds, c, dsts, srcs, copies, pos, n_polys, chunk, limb, pblk, pi);
}

// The inverse chunk pass of a transform whose strided pass takes the span of 2048 (SKIP): its eleven stages never
// pair words of different halves of a 4096-word chunk, so a half is a work-group's whole job: 2048 words, 256
// threads, and the one work-group barrier is among four waves, one on each SIMD, instead of eight.  Rounds as in
// inv_chunk_body; the last has two stages (spans 512 and 1024) on the words t + 256 r of a thread, register r holding
// the word at t + 256 (r >> 2 & 1) + 512 (r & 1) + 1024 (r >> 1 & 1) so that the two stages pair neighbouring registers
// and registers two apart.
constexpr int kLogHalf = 11, kHalf = 1 << kLogHalf, kHalfThreads = 256;
// the twiddles of a thread for the eleven stages of a half; they depend on the limb, the half and the thread only
template <class A>
struct HalfTw {
  typename A::TWL a0[4], a1[2], a2[1], b0[4], b1[2], b2[1], c0[4], c1[2], c2[1], d0[2], d1[1];
  __device__ __forceinline__ void load(const A& ar, const ChunkMap& cm, u32 mh, u32 half, u32 t) {
    ar.template load_tw<4>((mh >> 0) + (half << 10) + (t << 2), a0);
    ar.template load_tw<2>((mh >> 1) + (half << 9) + (t << 1), a1);
    ar.template load_tw<1>((mh >> 2) + (half << 8) + (t << 0), a2);
    ar.template load_tw<4>((mh >> 3) + (half << 7) + (cm.h << 2), b0);
    ar.template load_tw<2>((mh >> 4) + (half << 6) + (cm.h << 1), b1);
    ar.template load_tw<1>((mh >> 5) + (half << 5) + (cm.h << 0), b2);
    ar.template load_tw<4>((mh >> 6) + (half << 4) + (cm.wv << 2), c0);
    ar.template load_tw<2>((mh >> 7) + (half << 3) + (cm.wv << 1), c1);
    ar.template load_tw<1>((mh >> 8) + (half << 2) + (cm.wv << 0), c2);
    ar.template load_tw<2>((mh >> 9) + (half << 1), d0);
    ar.template load_tw<1>((mh >> 10) + half, d1);
  }
  // makes the compiler wait for the loads above here, so that its count of pending loads is zero afterwards
  __device__ __forceinline__ void settle() {
    auto use = [](typename A::TWL& x) { asm volatile("" : "+v"(x)); };
    for (auto& x : a0) use(x);
    for (auto& x : a1) use(x);
    use(a2[0]);
    for (auto& x : b0) use(x);
    for (auto& x : b1) use(x);
    use(b2[0]);
  }
};
// the eleven stages of a half from the words a thread loaded (raw[r] = word 8 t + r of the half) to the words it
// stores (word(r) of its column t); twiddles loaded stage by stage, or handed in (pre)
__device__ __forceinline__ constexpr int half_word(int r) { return 256 * ((r >> 2) & 1) + 512 * (r & 1) + 1024 * ((r >> 1) & 1); }
// CENTRED: the eight values come as `vin`, each of magnitude at most q/2, instead of canonical words (`raw`); the
// sums of four then stay within 2q without the shift that canonical words need.
template <class A, bool PRE, bool CENTRED = false>
__device__ __forceinline__ void inv_half_rounds(typename A::T* lds, const A& ar, const ChunkMap& cm, u32 mh, u32 half,
                                                const u64* raw, u64* out, const HalfTw<A>* pre,
                                                const typename A::T* vin = nullptr) {
  typedef typename A::T T;
  const int t = threadIdx.x;
  T v[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) v[r] = CENTRED ? vin[r] : ar.in_canon(raw[r]);
  // spans 1, 2, 4
  if constexpr (PRE) {
    gs_stage_pre<A, 8, 0>(ar, v, pre->a0);
    gs_stage_pre<A, 8, 1>(ar, v, pre->a1);
  } else {
    gs_stage<A, 8, 0>(ar, v, (mh >> 0) + (half << 10) + ((u32)t << 2));
    gs_stage<A, 8, 1>(ar, v, (mh >> 1) + (half << 9) + ((u32)t << 1));
  }
  if constexpr (!CENTRED) {
    ar.recentre_sum_of_four(v[0]);
    ar.recentre_sum_of_four(v[4]);
  }
  if constexpr (PRE) gs_stage_pre<A, 8, 2>(ar, v, pre->a2);
  else gs_stage<A, 8, 2>(ar, v, (mh >> 2) + (half << 8) + ((u32)t << 0));
  // in a run: the previous polynomial's last round, on other waves, has read the words written next
  if constexpr (PRE) __syncthreads();
#pragma unroll
  for (int r = 0; r < 8; ++r) lds[cm.narrow + ChunkMap::narrow_off(r)] = v[r];
  wave_sync();  // the words read next were written by this wave
  // spans 8, 16, 32
#pragma unroll
  for (int r = 0; r < 8; ++r) v[r] = lds[cm.octet + ChunkMap::octet_off(r)];
  reduce_all<A, 8>(ar, v);
  if constexpr (PRE) {
    gs_stage_pre<A, 8, 0>(ar, v, pre->b0);
    gs_stage_pre<A, 8, 1>(ar, v, pre->b1);
    gs_stage_pre<A, 8, 2>(ar, v, pre->b2);
  } else {
    gs_stage<A, 8, 0>(ar, v, (mh >> 3) + (half << 7) + (cm.h << 2));
    gs_stage<A, 8, 1>(ar, v, (mh >> 4) + (half << 6) + (cm.h << 1));
    gs_stage<A, 8, 2>(ar, v, (mh >> 5) + (half << 5) + (cm.h << 0));
  }
#pragma unroll
  for (int r = 0; r < 8; ++r) lds[cm.octet + ChunkMap::octet_off(r)] = v[r];
  wave_sync();  // the words read next were written by this wave
  // spans 64, 128, 256
#pragma unroll
  for (int r = 0; r < 8; ++r) v[r] = lds[cm.wave + ChunkMap::wave_off(r)];
  reduce_all<A, 8>(ar, v);
  if constexpr (PRE) {
    gs_stage_pre<A, 8, 0>(ar, v, pre->c0);
    gs_stage_pre<A, 8, 1>(ar, v, pre->c1);
    gs_stage_pre<A, 8, 2>(ar, v, pre->c2);
  } else {
    gs_stage<A, 8, 0>(ar, v, (mh >> 6) + (half << 4) + (cm.wv << 2));
    gs_stage<A, 8, 1>(ar, v, (mh >> 7) + (half << 3) + (cm.wv << 1));
    gs_stage<A, 8, 2>(ar, v, (mh >> 8) + (half << 2) + (cm.wv << 0));
  }
#pragma unroll
  for (int r = 0; r < 8; ++r) lds[cm.wave + ChunkMap::wave_off(r)] = v[r];
  __syncthreads();
  // spans 512 and 1024; twiddles are uniform over the work-group
#pragma unroll
  for (int r = 0; r < 8; ++r) v[r] = lds[cm.wide + half_word(r) + half_word(r) / 16];
  reduce_all<A, 8>(ar, v);
  {
    typename A::TWL two[2], tw[4];
    if constexpr (PRE) {
      two[0] = pre->d0[0];
      two[1] = pre->d0[1];
    } else {
      ar.template load_tw<2>((mh >> 9) + (half << 1), two);
    }
    tw[0] = tw[2] = two[0];
    tw[1] = tw[3] = two[1];
    gs_stage_pre<A, 8, 0>(ar, v, tw);
    if constexpr (PRE) two[0] = pre->d1[0];
    else ar.template load_tw<1>((mh >> 10) + half, two);
    two[1] = two[0];
    gs_stage_pre<A, 8, 1>(ar, v, two);
  }
#pragma unroll
  for (int r = 0; r < 8; ++r) out[r] = ar.out_mid(v[r]);
}
template <class A>
__device__ __forceinline__ void inv_half_body(u64* lds_words, const DevCtx& c, const PolySeq& dsts,
                                              const PolySeq& srcs, const LimbMap& pos, u32 half, u32 limb, u32 poly,
                                              u32 pi) {
  const int t = threadIdx.x;
  const u64 off = (u64)pos.prime[limb] * c.N + (u64)half * kHalf;
  A ar;
  ar.init(c, pi, true, nullptr, 0);
  const ChunkMap cm(t);
  u64 raw[8];
  {
    const ulonglong2* src2 = reinterpret_cast<const ulonglong2*>(srcs.at(poly) + off + 8 * t);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const ulonglong2 x = src2[k];
      raw[2 * k] = x.x;
      raw[2 * k + 1] = x.y;
    }
  }
  u64 out[8];
  inv_half_rounds<A, false>(reinterpret_cast<typename A::T*>(lds_words), ar, cm, c.N >> 1, half, raw, out, nullptr);
  u64* dst = dsts.at(poly) + off + t;
#pragma unroll
  for (int r = 0; r < 8; ++r) stg<512>(dst + half_word(r), out[r]);
}
__global__ __launch_bounds__(kHalfThreads, kChunkWaves) void ntt_inv_half(DevCtx c, PolySeq dsts, PolySeq srcs, LimbMap lm,
                                                                       LimbMap pos, u32 n_limbs, u32 n_polys) {
  __shared__ u64 lds[kHalf + kHalf / 16];
  u32 half, limb, poly;
  if (!chunk_block<kLogHalf>(c, n_limbs, n_polys, half, limb, poly)) return;
  const u32 pi = lm.prime[limb];
  if (c.fp_ok[pi]) inv_half_body<ArithFp>(lds, c, dsts, srcs, pos, half, limb, poly, pi);
  else inv_half_body<ArithInt>(lds, c, dsts, srcs, pos, half, limb, poly, pi);
}

// The same pass for launches of many polynomials whose limbs are all on the FP64 back end: a work-group takes the same
// half of the same limb of `run` polynomials one after the other, and the words of the next one are on their way
// into LDS (16-byte loads that write LDS directly, no registers held) while the current one is transformed.  A wave's
// loads fill its own 4 KiB of the staging array with the 512 consecutive words its lanes work on, 1 KiB of consecutive
// words per instruction; a lane then reads its eight words (64 bytes, 64 bytes apart over the lanes: the LDS reads
// collide, which costs less than loads that fetch every line four times).  Only the wave itself reads what its loads
// wrote, so no barrier guards the staging array.
// Vector memory operations complete in the order of issue, so any load issued after the staging loads would wait for
// them: the thread's 24 twiddles are therefore loaded once, ahead of the loop (they are the same for every
// polynomial), and the one wait of an iteration lets the eight stores issued after the staging loads stay outstanding
// (`vmcnt(8)`: at most the eight youngest operations pending, hence the four loads done).  The staging loads are
// issued from inline assembly: issued through the compiler's builtin, every LDS access after them (the exchanges
// through the other array included) is made to wait for them.  The compiler does not count these loads; its own counts
// are then too low, which makes its waits longer than needed, never shorter, and inside the loop it has no load of its
// own to wait for.  33 KiB of LDS per work-group: four work-groups, 16 waves, per CU.
// What the scheme buys is not the overlap alone (the same loop without any arithmetic is only 5 % faster): 15 % fewer
// vector instructions (no twiddle loads or addresses in the loop), the non-temporal hint on loads that fetch every
// byte once, and the order of the work-groups (chunk_block, SLOT_MAJOR).
// PRODUCT: the polynomial transformed is the limb-wise product of srcs and srcs2 (both staged; 49 KiB of LDS, three
// work-groups per CU): the product of a word of each, exact in FP64 and brought to magnitude q/2, enters the first
// round in place of a canonical word -- an HMult's d2 = a1 b1 is then never written in NTT form.
template <bool PRODUCT>
__device__ __forceinline__ void inv_half_run_body(double* lds, u64* stage, u64* stage2, const DevCtx& c,
                                                  const PolySeq& dsts, const PolySeq& srcs, const PolySeq& srcs2,
                                                  const LimbMap& pos, u32 n_polys, u32 run,
                                                  u32 half, u32 limb, u32 pblk, u32 pi) {
  typedef ArithFp A;
  const int t = threadIdx.x;
  const u32 poly0 = pblk * run;
  const u32 cnt = min(run, n_polys - poly0);
  const u64 off = (u64)pos.prime[limb] * c.N + (u64)half * kHalf;
  A ar;
  ar.init(c, pi, true, nullptr, 0);
  const ChunkMap cm(t);
  u64* mine = stage + cm.wv * 512;  // this wave's four blocks of 128 words
  u64* mine2 = PRODUCT ? stage2 + cm.wv * 512 : nullptr;
  auto request = [&](u32 poly) {  // 1 KiB of consecutive words per instruction
    const u64* src = srcs.at(poly) + off + cm.wv * 512 + 2 * (t & 63);
#pragma unroll
    for (int j = 0; j < 4; ++j) stage_request(src + 128 * j, mine + 128 * j);
    if constexpr (PRODUCT) {
      const u64* src2 = srcs2.at(poly) + off + cm.wv * 512 + 2 * (t & 63);
#pragma unroll
      for (int j = 0; j < 4; ++j) stage_request(src2 + 128 * j, mine2 + 128 * j);
    }
  };
  HalfTw<A> tw;
  tw.load(ar, cm, c.N >> 1, half, (u32)t);
  tw.settle();
  request(poly0);
  for (u32 it = 0; it < cnt; ++it) {
    // this polynomial's words are in LDS: its four (eight) loads are older than the eight stores of the previous one,
    // and before the first polynomial nothing was issued after them
    if (it == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    u64 raw[8], raw2[PRODUCT ? 8 : 1];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const ulonglong2 x = *reinterpret_cast<const ulonglong2*>(mine + 8 * (t & 63) + 2 * j);
      raw[2 * j] = x.x;
      raw[2 * j + 1] = x.y;
      if constexpr (PRODUCT) {
        const ulonglong2 y = *reinterpret_cast<const ulonglong2*>(mine2 + 8 * (t & 63) + 2 * j);
        raw2[2 * j] = y.x;
        raw2[2 * j + 1] = y.y;
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // ... and in registers, before the next ones overwrite them
    if (it + 1 < cnt) request(poly0 + it + 1);
    u64 out[8];
    if constexpr (PRODUCT) {
      double v[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const double y = ar.in_canon(raw2[r]);
        v[r] = ar.mulmod(ar.in_canon(raw[r]), y, y * ar.qinv);  // both in [0, q): magnitude below 1.4 q
        ar.reduce(v[r]);
      }
      inv_half_rounds<A, true, true>(lds, ar, cm, c.N >> 1, half, raw, out, &tw, v);
    } else {
      inv_half_rounds<A, true>(lds, ar, cm, c.N >> 1, half, raw, out, &tw);
    }
    u64* dst = dsts.at(poly0 + it) + off + t;
#pragma unroll
    // cached, like the other inverse chunk passes: the strided pass that follows finds part of them in the caches
    // (the pass alone is 5 % faster with the hint, the transform 3 % slower)
    for (int r = 0; r < 8; ++r) stg<512>(dst + half_word(r), out[r]);
  }
}
template <bool PRODUCT>
__global__ __launch_bounds__(kHalfThreads, PRODUCT ? 3 : 4) void ntt_inv_half_run(DevCtx c, PolySeq dsts, PolySeq srcs,
                                                                                PolySeq srcs2, LimbMap lm, LimbMap pos,
                                                                                u32 n_limbs, u32 n_polys, u32 run) {
  __shared__ double lds[kHalf + kHalf / 16];
  __shared__ __attribute__((aligned(16))) u64 stage[kHalf];
  __shared__ __attribute__((aligned(16))) u64 stage2[PRODUCT ? kHalf : 2];
  u32 half, limb, pblk;
  if (!chunk_block<kLogHalf, true>(c, n_limbs, (n_polys + run - 1) / run, half, limb, pblk)) return;
  inv_half_run_body<PRODUCT>(lds, stage, stage2, c, dsts, srcs, srcs2, pos, n_polys, run, half, limb, pblk, lm.prime[limb]);
}

// inverse, strided pass: spans 4096..N/2, then scale every word by the limb's
// constant (default 1/N) and store canonical residues.  In place.
// scale: nullptr, or (constant, Shoup companion) pairs indexed by the limb's place in the launch.
template <class A, int LOGR>
__device__ __forceinline__ void inv_strided_body(const DevCtx& c, const PolySeq& datas, const LimbMap& pos,
                                                 const u64* __restrict__ scale, u32 limb, u32 pi) {
  constexpr int R = 1 << LOGR;
  const u32 col = blockIdx.x * 256 + threadIdx.x;
  const u64 rs = c.N >> LOGR;
  // last polynomials first: the chunk pass before this one has written them last, and part of them is still in the
  // memory-side cache (hence also the plain loads below: with the hint the pass alone is 9 % faster on the 768-limb
  // batch, 0.128 against 0.140 ms, and the transform 2 % slower)
  u64* __restrict__ data = datas.at(gridDim.z - 1 - blockIdx.z) + (u64)pos.prime[limb] * c.N;
  A ar;
  ar.init(c, pi, true, scale, limb);
  typename A::T v[R];
#pragma unroll
  for (int r = 0; r < R; ++r) v[r] = ar.in_mid(data[r * rs + col]);
  inv_strided_stages<A, LOGR>(ar, v);
#pragma unroll
  for (int r = 0; r < R; ++r) stg<1>(data + r * rs + col, ar.out_scaled(v[r]));
}
// ONLY: 0 = limbs of both back ends (the choice is uniform over a work-group), 1 = integer limbs only, 2 = FP64
// limbs only.  The two bodies in one function need 130 registers at LOGR = 4 where each alone needs 78 / 90, and
// most launches are of one kind (the special primes of a Mod_down, the digit of a Mod_up).  A launch covers the limbs
// limb0 .. limb0 + gridDim.y - 1 of the transform, so that a transform whose limbs change kind once or twice along
// the list is served by one launch of the fitting kind per stretch.
template <int LOGR, int ONLY>
__global__ __launch_bounds__(256) void ntt_inv_strided(DevCtx c, PolySeq datas, LimbMap lm, LimbMap pos,
                                                       const u64* __restrict__ scale, u32 limb0) {
  const u32 limb = limb0 + gridDim.y - 1 - blockIdx.y, pi = lm.prime[limb];
  if (ONLY == 2 || (ONLY == 0 && c.fp_ok[pi])) inv_strided_body<ArithFp, LOGR>(c, datas, pos, scale, limb, pi);
  else inv_strided_body<ArithInt, LOGR>(c, datas, pos, scale, limb, pi);
}

// ---------------------------------------------------------------------------
// The strided passes of N = 2^16 for launches too small to fill the machine.  A column's sixteen words are spread
// over the four waves of a work-group, four words each: two stages, one exchange through LDS, two more stages.
// Such a launch is four times the waves of the plain pass, each with a quarter of a column's 32 butterflies, where
// the plain pass would leave most SIMDs with a single wave that works through a whole column on its own.
// grid = (N/16/64, n_limbs, n_polys), 256 threads; results are those of the plain pass.
constexpr int kSplitCols = 64;
template <class A, int PRO>
__device__ __forceinline__ void fwd_strided_split_body(u64* lds_words, const DevCtx& c, const PolySeq& dsts,
                                                       const PolySeq& srcs, const LimbMap& pos, const FwdFuse& f,
                                                       u32 limb, u32 pi) {
  typedef typename A::T T;
  const u32 j = (u32)__builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const u32 col = blockIdx.x * kSplitCols + lane;
  const u64 rs = c.N >> 4;
  u64* __restrict__ dst = dsts.at(blockIdx.z) + (u64)pos.prime[limb] * c.N;
  A ar;
  ar.init(c, pi, false, nullptr, 0);
  T v[4];
  // rows j, j+4, j+8, j+12: the pairs of the stages of span 8 and 4
  fwd_strided_input<A, 4, PRO>(ar, c, srcs, pos, f, limb, pi, col, j * rs, 4 * rs, v);
  ct_stage<A, 4, 0>(ar, v, 1);
  ct_stage<A, 4, 1>(ar, v, 2);
  T* x = reinterpret_cast<T*>(lds_words);
#pragma unroll
  for (int k = 0; k < 4; ++k) x[(j + 4 * k) * kSplitCols + lane] = v[k];
  __syncthreads();
  // rows 4j .. 4j+3: group j of the stage of span 2, groups 2j and 2j+1 of the last one
#pragma unroll
  for (int k = 0; k < 4; ++k) v[k] = x[(4 * j + k) * kSplitCols + lane];
  ct_stage<A, 4, 0>(ar, v, 4 + j);
  ct_stage<A, 4, 1>(ar, v, 8 + 2 * j);
  reduce_all<A, 4>(ar, v);
#pragma unroll
  for (int k = 0; k < 4; ++k) stg<1>(dst + (4 * j + k) * rs + col, ar.out_mid(v[k]));
}
template <int PRO>
__global__ __launch_bounds__(256) void ntt_fwd_strided_split(DevCtx c, PolySeq dsts, PolySeq srcs, LimbMap lm,
                                                             LimbMap pos, FwdFuse f) {
  __shared__ u64 lds[16 * kSplitCols];
  const u32 limb = gridDim.y - 1 - blockIdx.y, pi = lm.prime[limb];
  if (c.fp_ok[pi]) fwd_strided_split_body<ArithFp, PRO>(lds, c, dsts, srcs, pos, f, limb, pi);
  else fwd_strided_split_body<ArithInt, PRO>(lds, c, dsts, srcs, pos, f, limb, pi);
}
template <class A>
__device__ __forceinline__ void inv_strided_split_body(u64* lds_words, const DevCtx& c, const PolySeq& datas,
                                                       const LimbMap& pos, const u64* __restrict__ scale, u32 limb,
                                                       u32 pi) {
  typedef typename A::T T;
  const u32 j = (u32)__builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const u32 col = blockIdx.x * kSplitCols + lane;
  const u64 rs = c.N >> 4;
  u64* __restrict__ data = datas.at(blockIdx.z) + (u64)pos.prime[limb] * c.N;
  A ar;
  ar.init(c, pi, true, scale, limb);
  T v[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) v[k] = ar.in_mid(ldg<2>(data + (4 * j + k) * rs + col));
  // the reductions stand where inv_strided_stages has them: before the first and the fourth stage
  reduce_all<A, 4>(ar, v);
  gs_stage<A, 4, 0>(ar, v, 8 + 2 * j);
  gs_stage<A, 4, 1>(ar, v, 4 + j);
  T* x = reinterpret_cast<T*>(lds_words);
#pragma unroll
  for (int k = 0; k < 4; ++k) x[(4 * j + k) * kSplitCols + lane] = v[k];
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 4; ++k) v[k] = x[(j + 4 * k) * kSplitCols + lane];
  gs_stage<A, 4, 0>(ar, v, 2);
  reduce_all<A, 4>(ar, v);
  gs_stage<A, 4, 1>(ar, v, 1);
#pragma unroll
  for (int k = 0; k < 4; ++k) stg<1>(data + (j + 4 * k) * rs + col, ar.out_scaled(v[k]));
}
__global__ __launch_bounds__(256) void ntt_inv_strided_split(DevCtx c, PolySeq datas, LimbMap lm, LimbMap pos,
                                                             const u64* __restrict__ scale) {
  __shared__ u64 lds[16 * kSplitCols];
  const u32 limb = gridDim.y - 1 - blockIdx.y, pi = lm.prime[limb];
  if (c.fp_ok[pi]) inv_strided_split_body<ArithFp>(lds, c, datas, pos, scale, limb, pi);
  else inv_strided_split_body<ArithInt>(lds, c, datas, pos, scale, limb, pi);
}

// ---------------------------------------------------------------------------
// N <= 4096: one workgroup per limb, the limb in LDS, one butterfly per
// thread per step (integer back end).  grid = (1, n_limbs, n_polys)
__global__ __launch_bounds__(256) void ntt_small(DevCtx c, PolySeq dsts, PolySeq srcs, LimbMap lm, LimbMap pos,
                                                 int inverse, const u64* __restrict__ scale) {
  __shared__ u64 a[kChunk];
  const u32 N = c.N, logN = c.logN, limb = blockIdx.y, pi = lm.prime[limb];
  const u64 off = (u64)pos.prime[limb] * N;
  u64* __restrict__ dst = dsts.at(blockIdx.z);
  const u64* __restrict__ src = srcs.at(blockIdx.z);
  ArithInt ar;
  ar.init(c, pi, inverse != 0, scale, limb);
  for (u32 i = threadIdx.x; i < N; i += 256) a[i] = src[off + i];
  __syncthreads();
  if (!inverse) {
    for (u32 s = 0; s < logN; ++s) {
      const u32 tspan = N >> (s + 1);
      for (u32 b = threadIdx.x; b < (N >> 1); b += 256) {
        u32 g = b / tspan, j = b - g * tspan, i0 = g * 2 * tspan + j;
        ArithInt::TW tw;
        ar.load_tw<1>((1u << s) + g, &tw);
        ar.ct(a[i0], a[i0 + tspan], tw);
      }
      __syncthreads();
    }
    for (u32 i = threadIdx.x; i < N; i += 256) dst[off + i] = ar.out_canon(a[i]);
  } else {
    for (u32 u = 0; u < logN; ++u) {
      const u32 span = 1u << u, m = N >> (u + 1);
      for (u32 b = threadIdx.x; b < (N >> 1); b += 256) {
        u32 g = b >> u, j = b & (span - 1), i0 = g * 2 * span + j;
        ArithInt::TW tw;
        ar.load_tw<1>(m + g, &tw);
        ar.gs(a[i0], a[i0 + span], tw);
      }
      __syncthreads();
    }
    for (u32 i = threadIdx.x; i < N; i += 256) dst[off + i] = ar.out_scaled(a[i]);
  }
}

// ---------------------------------------------------------------------------
// LOGR = logN - 12 stages lie outside a 4096-word chunk.  With a shift of 1 the strided pass, which is bound by HBM
// and has instruction slots to spare, also runs the chunk's widest stage (LOGR + 1 stages on N / 2^(LOGR+1) rows of
// a column), and the chunk pass skips it.  Measured on 768 limbs at N = 2^16: the chunk passes gain 2 %, the inverse
// strided pass stays where it was and the forward one, which then needs 122 registers, loses 6 %: the inverse
// transform shifts (SI), the forward one does not (SF).
// Launches of fewer limbs than this take the split strided passes (N = 2^16) if any of their limbs is on the integer
// back end: an FP64 column is a fifth of the instructions, and a launch of those gains nothing from the split.
static bool split_strided(const DevCtx& c, const LimbMap& lm, u32 n_limbs, u32 n_polys) {
  static const long below = [] {
    const char* e = getenv("ACE_NTT_SPLIT_BELOW");
    return e ? atol(e) : 96L;
  }();
  if ((long)n_limbs * (long)n_polys >= below) return false;
  for (u32 t = 0; t < n_limbs; ++t)
    if (!c.fp_ok[lm.prime[t]]) return true;
  return false;
}
// How many polynomials a work-group of a run kernel takes one after the other: eight, or four where eight would leave
// fewer than two rounds of work-groups for the `resident` that fit the machine at once; 0 = too few polynomials for runs.
constexpr u32 kCUs = 256;  // MI355X
static u32 run_length(u32 groups, u32 n_polys, u32 resident) {
  for (u32 run : {8u, 4u})
    if (n_polys >= 2 * run && (u64)groups * ((n_polys + run - 1) / run) >= 2ull * resident) return run;
  return 0;
}
static bool all_fp(const DevCtx& c, const LimbMap& lm, u32 n_limbs) {
  for (u32 t = 0; t < n_limbs; ++t)
    if (!c.fp_ok[lm.prime[t]]) return false;
  return true;
}
// Whether a work-group may ask for its next polynomial's words before it has stored the current one's: in place (a
// polynomial's words are read before any of them is written, and polynomials of a sequence do not overlap), or source
// and destination apart altogether.
static bool in_place_or_apart(const DevCtx& c, const PolySeq& dst, const PolySeq& src, const LimbMap& pos, u32 n_limbs,
                              u32 n_polys) {
  if (dst.b[0] == src.b[0] && dst.b[1] == src.b[1] && dst.pair_stride == src.pair_stride) return true;
  u64 top = 0;
  for (u32 t = 0; t < n_limbs; ++t) top = std::max<u64>(top, pos.prime[t]);
  const u64 words = (top + 1) * c.N;
  auto span = [&](const PolySeq& q, const u64*& lo, const u64*& hi) {
    lo = std::min(q.b[0], q.b[1]);
    hi = std::max(q.b[0], q.b[1]) + (u64)((n_polys - 1) >> 1) * q.pair_stride + words;
  };
  const u64 *dl, *dh, *sl, *sh;
  span(dst, dl, dh);
  span(src, sl, sh);
  return dh <= sl || sh <= dl;
}
template <int LOGR, int SF, int SI>
static bool run_large(hipStream_t st, const DevCtx& c, const PolySeq& dst, const PolySeq& src, const LimbMap& lm,
                      const LimbMap& pos, u32 n_limbs, u32 n_polys, bool inverse, const u64* scale, int passes,
                      const FwdFuse& f, const CopyThrough& copies, const PolySeq* times) {
  dim3 gc(chunk_grid(c, n_limbs, (n_polys + kPolysPerBlock - 1) / kPolysPerBlock));
  if (times && (!inverse || !(passes & 1))) return false;
  if (!inverse) {
    constexpr int LS = LOGR + SF, SHIFT = SF;
    dim3 gs((c.N >> LS) / 256, n_limbs, n_polys);
    if ((passes & 1) && LS == 4 && split_strided(c, lm, n_limbs, n_polys)) {
      dim3 gq((c.N >> 4) / kSplitCols, n_limbs, n_polys);
      if (f.pro == 0)
        hipLaunchKernelGGL((ntt_fwd_strided_split<0>), gq, dim3(256), 0, st, c, dst, src, lm, pos, f);
      else if (f.pro == 1)
        hipLaunchKernelGGL((ntt_fwd_strided_split<1>), gq, dim3(256), 0, st, c, dst, src, lm, pos, f);
      else
        hipLaunchKernelGGL((ntt_fwd_strided_split<2>), gq, dim3(256), 0, st, c, dst, src, lm, pos, f);
    } else if (passes & 1) {
      if (f.pro == 0)
        hipLaunchKernelGGL((ntt_fwd_strided<LS, 0>), gs, dim3(256), 0, st, c, dst, src, lm, pos, f);
      else if (f.pro == 1)
        hipLaunchKernelGGL((ntt_fwd_strided<LS, 1>), gs, dim3(256), 0, st, c, dst, src, lm, pos, f);
      else
        hipLaunchKernelGGL((ntt_fwd_strided<LS, 2>), gs, dim3(256), 0, st, c, dst, src, lm, pos, f);
    }
    if (passes & 2) {
      const u32 lr = LOGR;
      static const bool runs = [] {
        const char* e = getenv("ACE_NTT_FWD_RUN");
        return !e || e[0] != '0';
      }();
      // (the chunk pass works in place on dst, which the strided pass has filled; with an epilogue the run kernel is
      // slower than the plain one, whose eight waves per SIMD hide the tail's loads: 32 rotations 16 060 against
      // 17 200 per second)
      const u32 run = runs && f.epi == 0 && SHIFT == 0 && all_fp(c, lm, n_limbs)
                          ? run_length(n_limbs * (c.N >> kLogChunk), n_polys, 2 * kCUs) : 0;
      if (run)
        hipLaunchKernelGGL(ntt_fwd_chunk_run, dim3(chunk_grid<true>(c, n_limbs, (n_polys + run - 1) / run)),
                           dim3(kChunkThreads), 0, st, c, dst, lm, pos, lr, n_limbs, n_polys, run);
      else if (f.epi == 0)
        hipLaunchKernelGGL((ntt_fwd_chunk<0, SHIFT>), gc, dim3(kChunkThreads), 0, st, c, dst, lm, pos, lr, n_limbs,
                           n_polys, f);
      else if (f.epi == 1)
        hipLaunchKernelGGL((ntt_fwd_chunk<1, SHIFT>), gc, dim3(kChunkThreads), 0, st, c, dst, lm, pos, lr, n_limbs,
                           n_polys, f);
      else
        hipLaunchKernelGGL((ntt_fwd_chunk<2, SHIFT>), gc, dim3(kChunkThreads), 0, st, c, dst, lm, pos, lr, n_limbs,
                           n_polys, f);
    }
  } else {
    constexpr int LS = LOGR + SI, SHIFT = SI;
    dim3 gs((c.N >> LS) / 256, n_limbs, n_polys);
    if (passes & 1) {
      static const bool halves = [] {
        const char* e = getenv("ACE_NTT_INV_HALF");
        return !e || e[0] != '0';
      }();
      static const bool runs = [] {
        const char* e = getenv("ACE_NTT_INV_RUN");
        return !e || e[0] != '0';
      }();
      const u32 run = SHIFT == 1 && halves && runs && !copies.seq.b[0] && all_fp(c, lm, n_limbs) &&
                              in_place_or_apart(c, dst, src, pos, n_limbs, n_polys) &&
                              (!times || in_place_or_apart(c, dst, *times, pos, n_limbs, n_polys))
                          ? run_length(n_limbs * (c.N >> kLogHalf), n_polys, 4 * kCUs) : 0;
      if (times) {  // only the run kernel multiplies on the way in
        if (!run) return false;
        hipLaunchKernelGGL(ntt_inv_half_run<true>, dim3(chunk_grid<true>(c, n_limbs, (n_polys + run - 1) / run, kLogHalf)),
                           dim3(kHalfThreads), 0, st, c, dst, src, *times, lm, pos, n_limbs, n_polys, run);
      } else if (copies.seq.b[0])
        hipLaunchKernelGGL((ntt_inv_chunk<SHIFT, 1>), gc, dim3(kChunkThreads), 0, st, c, dst, src, copies, lm, pos,
                           n_limbs, n_polys);
      else if (run)
        hipLaunchKernelGGL(ntt_inv_half_run<false>, dim3(chunk_grid<true>(c, n_limbs, (n_polys + run - 1) / run, kLogHalf)),
                           dim3(kHalfThreads), 0, st, c, dst, src, src, lm, pos, n_limbs, n_polys, run);
      else if (SHIFT == 1 && halves)
        hipLaunchKernelGGL(ntt_inv_half, dim3(chunk_grid(c, n_limbs, n_polys, kLogHalf)), dim3(kHalfThreads), 0, st, c,
                           dst, src, lm, pos, n_limbs, n_polys);
      else
        hipLaunchKernelGGL((ntt_inv_chunk<SHIFT, 0>), gc, dim3(kChunkThreads), 0, st, c, dst, src, copies, lm, pos,
                           n_limbs, n_polys);
    }
    if ((passes & 2) && LS == 4 && split_strided(c, lm, n_limbs, n_polys)) {
      dim3 gq((c.N >> 4) / kSplitCols, n_limbs, n_polys);
      hipLaunchKernelGGL(ntt_inv_strided_split, gq, dim3(256), 0, st, c, dst, lm, pos, scale);
    } else if (passes & 2) {
      // stretches of limbs of one kind
      u32 starts[4], n_runs = 0;
      for (u32 t = 0; t < n_limbs; ++t)
        if (t == 0 || c.fp_ok[lm.prime[t]] != c.fp_ok[lm.prime[t - 1]]) {
          if (n_runs < 4) starts[n_runs] = t;
          ++n_runs;
        }
      if (n_runs <= 3) {
        for (u32 k = 0; k < n_runs; ++k) {
          const u32 a = starts[k], b = k + 1 < n_runs ? starts[k + 1] : n_limbs;
          dim3 gr(gs.x, b - a, n_polys);
          if (c.fp_ok[lm.prime[a]])
            hipLaunchKernelGGL((ntt_inv_strided<LS, 2>), gr, dim3(256), 0, st, c, dst, lm, pos, scale, a);
          else
            hipLaunchKernelGGL((ntt_inv_strided<LS, 1>), gr, dim3(256), 0, st, c, dst, lm, pos, scale, a);
        }
      } else {
        hipLaunchKernelGGL((ntt_inv_strided<LS, 0>), gs, dim3(256), 0, st, c, dst, lm, pos, scale, 0u);
      }
    }
  }
  return true;
}

bool launch_ntt(hipStream_t st, const DevCtx& c, const PolySeq& dst, const PolySeq& src, const LimbMap& lm,
                const LimbMap* pos_in, u32 n_limbs, u32 n_polys, bool inverse, const u64* scale, int passes,
                const FwdFuse* fuse, const CopyThrough* copy_src_to, const PolySeq* times) {
  if (n_limbs == 0 || n_polys == 0) return true;
  if (times && (!inverse || c.logN <= kLogChunk || copy_src_to || !(passes & 1))) return false;
  CopyThrough copies{};
  if (copy_src_to) {  // only the inverse chunk pass can drop a copy of what it reads
    if (!inverse || c.logN <= kLogChunk || !(passes & 1)) return false;
    if (!copy_src_to->part_size) return false;
    copies = *copy_src_to;
  }
  FwdFuse f{};
  if (fuse) {
    // only forward transforms of N > 4096: whole ones, or the chunk pass alone with its epilogue, for a caller whose own
    // kernel has run the strided pass and the prologue (launch_baseconv_fwd_strided)
    if (inverse || c.logN <= kLogChunk || !(passes == 3 || passes == 2)) return false;
    f = *fuse;
  }
  LimbMap pos{};
  if (pos_in) pos = *pos_in;
  else
    for (u32 t = 0; t < n_limbs; ++t) pos.prime[t] = (uint8_t)t;
  if (c.logN > kLogChunk) {
    // the chunk passes move 16 bytes per access: every polynomial must start on a 16-byte boundary (limbs are
    // multiples of 4096 words apart, so this is a condition on the base pointers and strides only)
    auto aligned = [](const PolySeq& q) {
      return (((uintptr_t)q.b[0] | (uintptr_t)q.b[1]) & 15) == 0 && (q.pair_stride & 1) == 0;
    };
    if (!aligned(dst) || !aligned(src) || (times && !aligned(*times))) return false;
    if (f.epi && (!aligned(f.out) || !aligned(f.src) || (f.addend_mode && !aligned(f.addend)))) return false;
    if (copies.seq.b[0] && (!aligned(copies.seq) || (copies.digit_stride & 1))) return false;
  }
  if (c.logN <= kLogChunk) {
    hipLaunchKernelGGL(ntt_small, dim3(1, n_limbs, n_polys), dim3(256), 0, st, c, dst, src, lm, pos, inverse ? 1 : 0,
                       scale);
    return true;
  }
  // the shifted inverse (see run_large) halves the threads of the strided pass: only for launches that fill the
  // machine anyway.  The rule depends on the shape of the launch alone, so the two passes of a transform agree
  // also when a caller runs them apart.
  const bool big = (u64)n_limbs * n_polys >= 192;
  switch (c.logN - kLogChunk) {
#define ACE_NTT_CASE(LR, SH)                                                                       \
  case LR:                                                                                         \
    if (SH && big)                                                                                   \
      return run_large<LR, 0, SH>(st, c, dst, src, lm, pos, n_limbs, n_polys, inverse, scale, passes, f, copies, times); \
    if (times) return false;                                                                         \
    return run_large<LR, 0, 0>(st, c, dst, src, lm, pos, n_limbs, n_polys, inverse, scale, passes, f, copies, times);
    ACE_NTT_CASE(1, ACE_NTT_SHIFT)
    ACE_NTT_CASE(2, ACE_NTT_SHIFT)
    ACE_NTT_CASE(3, ACE_NTT_SHIFT)
    ACE_NTT_CASE(4, ACE_NTT_SHIFT)
    ACE_NTT_CASE(5, 0)  // 64 rows of a column would not fit the registers of a thread
#undef ACE_NTT_CASE
    default:
      return false;  // ring degree above 2^17 not supported
  }
}

}  // namespace ace
