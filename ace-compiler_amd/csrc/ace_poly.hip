// Streaming RNS-polynomial kernels for gfx950: per-limb modular vector ops,
// automorphism gather, ciphertext tensor product, fast base conversion,
// switch-key inner product, Mod_down and Rescale tails.
//
// All are HBM-streaming except the base conversion, which is VALU-bound
// (nd 128-bit multiply-accumulates plus one Barrett-128 per output word).
// Grids are (ceil(n / (256*kUnroll)), n_limbs): blockIdx.y picks the limb and
// with it the modulus, so modulus constants are wave-uniform (scalar loads).
#include "ace_kernels.h"

namespace ace {

// Streams that a kernel reads or writes once go past the caches with the non-temporal hint where that was measured
// to pay (loads and stores of a kernel together: either alone changes nothing).  ACE_POLY_NT bits, with what each
// gave on one machine: 2 the inner product that shares a key, digits and results (key switch +2 %; its key, read
// once per four operands, is better left cached: bit 16); 4 the inner product that shares the digits, keys and
// results (rotations +3 %; its digits stay cached: bit 32); 64 the extended-basis rotation, 128 the grouped plaintext
// sums, 256 the plain inner product (a bootstrap 21.45 -> 21.2 ms together).  Not set: 1 the tensor product (no
// change), 8 the base conversion (1 % slower).
#ifndef ACE_POLY_NT
#define ACE_POLY_NT (2 | 4 | 64 | 128 | 256)
#endif
template <int BIT, class P>
__device__ __forceinline__ P ldn(const P* p) {
  if constexpr ((ACE_POLY_NT & BIT) != 0) return __builtin_nontemporal_load(p);
  else return *p;
}
template <int BIT, class P>
__device__ __forceinline__ void stn(P* p, P v) {
  if constexpr ((ACE_POLY_NT & BIT) != 0) __builtin_nontemporal_store(v, p);
  else *p = v;
}

constexpr int kThreads = 256;
// Coefficients per thread of the elementwise kernels.  One: the launches of whole programs are a few thousand
// work-groups at most, and more, smaller ones fill the machine better than fewer with four coefficients each (a
// bootstrap 2 % faster, the hoisted rotation in the extended basis included; the large batched launches unchanged).
constexpr int kUnroll = 1;

static inline dim3 ew_grid(u64 n, u32 n_limbs, u32 z = 1) {
  u64 per_block = (u64)kThreads * kUnroll;
  return dim3((unsigned)((n + per_block - 1) / per_block), n_limbs, z);
}

#define ACE_EW_LOOP(i, n)                                                      \
  for (u64 i = (u64)blockIdx.x * (kThreads * kUnroll) + threadIdx.x, _k = 0;   \
       _k < kUnroll && i < (n); ++_k, i += kThreads)

// ---- Hw_modadd ... Hw_modmuladd_scalar (hal/src/hal.c:15-121) -------------
template <int OP>
__global__ __launch_bounds__(kThreads) void ew_kernel(DevCtx c, u64* __restrict__ r, const u64* __restrict__ a,
                                                      const u64* __restrict__ b, u64 scalar, LimbMap lm, u64 n) {
  const u32 limb = blockIdx.y;
  const DevPrime P = c.primes[lm.prime[limb]];
  const u64 base = (u64)limb * n;
#pragma unroll
  ACE_EW_LOOP(i, n) {
    u64 x = a[base + i];
    u64 y = (OP >= EW_ADD_S) ? scalar : b[base + i];
    u64 v;
    if (OP == EW_ADD || OP == EW_ADD_S) v = add_mod(x, y, P.q);
    else if (OP == EW_SUB || OP == EW_SUB_S) v = sub_mod(x, y, P.q);
    else if (OP == EW_MUL || OP == EW_MUL_S) v = mulmod(x, y, P);
    else v = add_mod(r[base + i], mulmod(x, y, P), P.q);
    r[base + i] = v;
  }
}

void launch_ew(hipStream_t st, const DevCtx& c, EwOp op, u64* r, const u64* a, const u64* b, u64 scalar,
               const LimbMap& lm, u32 n_limbs, u64 n) {
  if (!n || !n_limbs) return;
  dim3 g = ew_grid(n, n_limbs);
#define ACE_EW_CASE(OP) \
  case OP: hipLaunchKernelGGL(ew_kernel<OP>, g, dim3(kThreads), 0, st, c, r, a, b, scalar, lm, n); break;
  switch (op) {
    ACE_EW_CASE(EW_ADD) ACE_EW_CASE(EW_SUB) ACE_EW_CASE(EW_MUL) ACE_EW_CASE(EW_MULADD)
    ACE_EW_CASE(EW_ADD_S) ACE_EW_CASE(EW_SUB_S) ACE_EW_CASE(EW_MUL_S) ACE_EW_CASE(EW_MULADD_S)
  }
#undef ACE_EW_CASE
}

// ---- sum over operands of (a0_j, a1_j) * plain_j: the inner sum of a baby-step group --------------
// (the Mul_plaintext + Add_ciphertext loop of Rotate_iteration, ckks/src/bootstrap.c:1291-1311).
// The operands are extended polynomials (level Q limbs, then the P limbs); a plaintext may be kept at a
// higher level, so its P limbs start plain_level limbs in (Derive_plain, include/ckks/plaintext.h:107-114).
__global__ __launch_bounds__(kThreads) void plain_mac_kernel(DevCtx c, u64* __restrict__ r0, u64* __restrict__ r1,
                                                             MacSet ops, LimbMap lm, u32 level, u32 plain_level,
                                                             int accumulate, u64 n) {
  const u32 limb = blockIdx.y;
  const DevPrime P = c.primes[lm.prime[limb]];
  const u64 base = (u64)limb * n;
  const u64 pbase = (u64)(limb < level ? limb : plain_level + (limb - level)) * n;
#pragma unroll
  ACE_EW_LOOP(i, n) {
    // summed in 128 bits, reduced once: at most kMaxMacOps = 32 products of residues below 2^61 and the running sum
    u64 l0 = accumulate ? r0[base + i] : 0, l1 = accumulate ? r1[base + i] : 0, h0 = 0, h1 = 0;
    for (u32 j = 0; j < ops.n; ++j) {
      u64 w = ops.p[j][pbase + i];
      mac128(h0, l0, ops.a0[j][base + i], w);
      mac128(h1, l1, ops.a1[j][base + i], w);
    }
    r0[base + i] = barrett128(h0, l0, P);
    r1[base + i] = barrett128(h1, l1, P);
  }
}
void launch_plain_mac(hipStream_t st, const DevCtx& c, u64* r0, u64* r1, const MacSet& ops, const LimbMap& lm,
                      u32 n_limbs, u32 level, u32 plain_level, bool accumulate, u64 n) {
  if (!n || !n_limbs || !ops.n) return;
  hipLaunchKernelGGL(plain_mac_kernel, ew_grid(n, n_limbs), dim3(kThreads), 0, st, c, r0, r1, ops, lm, level,
                     plain_level, accumulate ? 1 : 0, n);
}

__global__ __launch_bounds__(kThreads) void plain_mac_groups_kernel(DevCtx c, MacGroups ops, LimbMap lm, u32 level,
                                                                    u32 plain_level, int accumulate, u64 n) {
  const u32 limb = blockIdx.y;
  const DevPrime P = c.primes[lm.prime[limb]];
  const u64 base = (u64)limb * n;
  const u64 pbase = (u64)(limb < level ? limb : plain_level + (limb - level)) * n;
#pragma unroll
  ACE_EW_LOOP(i, n) {
    // The products of a group are summed in 128 bits and reduced once (at most kMaxMacOps = 32 products of residues
    // below 2^61, plus the running sum: below 2^128); the canonical residue is the one a reduction per product gives.
    u64 l0[kMacGroups], h0[kMacGroups], l1[kMacGroups], h1[kMacGroups];
#pragma unroll
    for (int g = 0; g < kMacGroups; ++g) {
      const bool on = g < (int)ops.n_groups && accumulate;
      l0[g] = on ? ops.r0[g][base + i] : 0;
      l1[g] = on ? ops.r1[g][base + i] : 0;
      h0[g] = h1[g] = 0;
    }
    for (u32 j = 0; j < ops.n_ops; ++j) {
      const u64 x0 = ldn<128>(ops.a0[j] + base + i), x1 = ldn<128>(ops.a1[j] + base + i);
#pragma unroll
      for (int g = 0; g < kMacGroups; ++g) {
        if (g < (int)ops.n_groups && ops.p[g][j]) {
          const u64 w = ldn<128>(ops.p[g][j] + pbase + i);
          mac128(h0[g], l0[g], x0, w);
          mac128(h1[g], l1[g], x1, w);
        }
      }
    }
#pragma unroll
    for (int g = 0; g < kMacGroups; ++g) {
      if (g < (int)ops.n_groups) {
        stn<128>(ops.r0[g] + base + i, barrett128(h0[g], l0[g], P));
        stn<128>(ops.r1[g] + base + i, barrett128(h1[g], l1[g], P));
      }
    }
  }
}
void launch_plain_mac_groups(hipStream_t st, const DevCtx& c, const MacGroups& ops, const LimbMap& lm, u32 n_limbs,
                             u32 level, u32 plain_level, bool accumulate, u64 n) {
  if (!n || !n_limbs || !ops.n_ops || !ops.n_groups) return;
  hipLaunchKernelGGL(plain_mac_groups_kernel, ew_grid(n, n_limbs), dim3(kThreads), 0, st, c, ops, lm, level,
                     plain_level, accumulate ? 1 : 0, n);
}

// ---- a recorded run of Hw_* calls (hal/src/hal.c:15-138) in one launch --------------------------------
// The host splits a run into chains that share no written range; a chain's entries are carried out in order by
// the thread of element i, so an entry may read what an earlier one of its chain wrote (identical ranges only;
// a rotate never reads or overwrites anything the run touches).
// A thread carries V consecutive elements (V = 2 when every range of the run is 16-byte aligned: 16-byte loads
// and stores, half the waves).
template <int V>
struct Words {
  u64 v[V];
};
template <int V>
__device__ __forceinline__ Words<V> load_words(const u64* p) {
  Words<V> w;
  if constexpr (V == 2) {
    const ulonglong2 t = *reinterpret_cast<const ulonglong2*>(p);
    w.v[0] = t.x;
    w.v[1] = t.y;
  } else {
    w.v[0] = p[0];
  }
  return w;
}
template <int V>
__device__ __forceinline__ void store_words(u64* p, const Words<V>& w) {
  if constexpr (V == 2) *reinterpret_cast<ulonglong2*>(p) = make_ulonglong2(w.v[0], w.v[1]);
  else p[0] = w.v[0];
}

template <int V>
__device__ __forceinline__ void run_chain(const DevCtx& c, const BatchOpDev* ops, u32 first, u32 last, u64 i) {
  // what the previous entry produced stays in registers: an operand that names that range is not loaded again
  const u64* prev_r = nullptr;
  Words<V> prev{};
  for (u32 k = first; k < last; ++k) {
    const BatchOpDev o = ops[k];
    const u64* ob = reinterpret_cast<const u64*>(o.b);
    const u32 op = o.op & ~kBatchDeadStore;
    const DevPrime P = c.primes[o.prime];
    Words<V> v;
    if (op == BATCH_ROTATE) {
      const Words<V> src = load_words<V>(ob + i);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const i64 j = (i64)src.v[e];
        v.v[e] = j >= 0 ? o.a[j] : P.q - o.a[-j];
      }
    } else if (op == BATCH_COPY) {
      v = o.a == prev_r ? prev : load_words<V>(o.a + i);
    } else if (op == BATCH_ZERO) {
#pragma unroll
      for (int e = 0; e < V; ++e) v.v[e] = 0;
    } else {
      const Words<V> x = o.a == prev_r ? prev : load_words<V>(o.a + i);
      Words<V> y;
      if (op >= EW_ADD_S) {
#pragma unroll
        for (int e = 0; e < V; ++e) y.v[e] = o.b;
      } else {
        y = ob == prev_r ? prev : load_words<V>(ob + i);
      }
      if (op == EW_ADD || op == EW_ADD_S) {
#pragma unroll
        for (int e = 0; e < V; ++e) v.v[e] = add_mod(x.v[e], y.v[e], P.q);
      } else if (op == EW_SUB || op == EW_SUB_S) {
#pragma unroll
        for (int e = 0; e < V; ++e) v.v[e] = sub_mod(x.v[e], y.v[e], P.q);
      } else if (op == EW_MUL || op == EW_MUL_S) {
#pragma unroll
        for (int e = 0; e < V; ++e) v.v[e] = mulmod(x.v[e], y.v[e], P);
      } else {
        const Words<V> acc = o.r == prev_r ? prev : load_words<V>(o.r + i);
#pragma unroll
        for (int e = 0; e < V; ++e) v.v[e] = add_mod(acc.v[e], mulmod(x.v[e], y.v[e], P), P.q);
      }
    }
    if (!(o.op & kBatchDeadStore)) store_words<V>(o.r + i, v);
    // a rotate's result is never read inside its run
    prev_r = op == BATCH_ROTATE ? nullptr : o.r;
    prev = v;
  }
}
template <int V>
__global__ __launch_bounds__(kThreads) void ew_batch_kernel(DevCtx c, const BatchOpDev* ops, const u32* chain_start, u64 n) {
  const u64 i = ((u64)blockIdx.x * kThreads + threadIdx.x) * V;
  if (i >= n) return;
  run_chain<V>(c, ops, chain_start[blockIdx.y], chain_start[blockIdx.y + 1], i);
}
template <int V>
__global__ __launch_bounds__(kThreads) void ew_batch_small_kernel(DevCtx c, SmallRun run, u64 n) {
  const u64 i = ((u64)blockIdx.x * kThreads + threadIdx.x) * V;
  if (i >= n) return;
  run_chain<V>(c, run.ops, run.chain_start[blockIdx.y], run.chain_start[blockIdx.y + 1], i);
}
// pairs: every range of the run starts on a 16-byte boundary and n is even
void launch_ew_batch_small(hipStream_t st, const DevCtx& c, const SmallRun& run, u32 n_chains, u64 n, bool pairs) {
  if (!n || !n_chains) return;
  const u64 per_block = (u64)kThreads * (pairs ? 2 : 1);
  dim3 g((unsigned)((n + per_block - 1) / per_block), n_chains, 1);
  if (pairs) hipLaunchKernelGGL(ew_batch_small_kernel<2>, g, dim3(kThreads), 0, st, c, run, n);
  else hipLaunchKernelGGL(ew_batch_small_kernel<1>, g, dim3(kThreads), 0, st, c, run, n);
}
void launch_ew_batch(hipStream_t st, const DevCtx& c, const BatchOpDev* dev_ops, const u32* dev_chain_start, u32 n_chains,
                     u64 n, bool pairs) {
  if (!n || !n_chains) return;
  const u64 per_block = (u64)kThreads * (pairs ? 2 : 1);
  dim3 g((unsigned)((n + per_block - 1) / per_block), n_chains, 1);
  if (pairs) hipLaunchKernelGGL(ew_batch_kernel<2>, g, dim3(kThreads), 0, st, c, dev_ops, dev_chain_start, n);
  else hipLaunchKernelGGL(ew_batch_kernel<1>, g, dim3(kThreads), 0, st, c, dev_ops, dev_chain_start, n);
}

// ---- key-generation helpers: uniform residues and small signed polynomials spread over limbs ------------
__device__ __forceinline__ u64 mix64(u64 z) {  // the finaliser of splitmix64
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
// limb t, word i = floor(x q_t / 2^128) for a 128-bit x hashed from (seed, stream, t, i): uniform on [0, q_t) up to
// a bias below 2^-64
__global__ __launch_bounds__(kThreads) void sample_uniform_kernel(DevCtx c, u64* __restrict__ r, u64 seed, u64 stream,
                                                                  LimbMap lm, u64 n) {
  const u32 limb = blockIdx.y;
  const u64 q = c.primes[lm.prime[limb]].q;
#pragma unroll
  ACE_EW_LOOP(i, n) {
    const u64 key = mix64(seed + 0x9E3779B97F4A7C15ull * (stream + 1)) ^ ((u64)limb << 40) ^ i;
    const u64 hi = mix64(key + 0x9E3779B97F4A7C15ull), lo = mix64(key + 2 * 0x9E3779B97F4A7C15ull + 1);
    const u64 carry = __umul64hi(lo, q);
    const u64 low = hi * q, sum = low + carry;
    r[(u64)limb * n + i] = __umul64hi(hi, q) + (sum < low ? 1 : 0);
  }
}
void launch_sample_uniform(hipStream_t st, const DevCtx& c, u64* r, u64 seed, u64 stream, const LimbMap& lm,
                           u32 n_limbs, u64 n) {
  if (!n || !n_limbs) return;
  hipLaunchKernelGGL(sample_uniform_kernel, ew_grid(n, n_limbs), dim3(kThreads), 0, st, c, r, seed, stream, lm, n);
}
// limb t, word i = v[i] mod q_t for small signed v (|v| < q_t)
__global__ __launch_bounds__(kThreads) void expand_small_kernel(DevCtx c, u64* __restrict__ r, const i64* __restrict__ v,
                                                                LimbMap lm, u64 n) {
  const u32 limb = blockIdx.y;
  const u64 q = c.primes[lm.prime[limb]].q;
#pragma unroll
  ACE_EW_LOOP(i, n) {
    const i64 x = v[i];
    r[(u64)limb * n + i] = x < 0 ? q - (u64)(-x) : (u64)x;
  }
}
void launch_expand_small(hipStream_t st, const DevCtx& c, u64* r, const i64* v, const LimbMap& lm, u32 n_limbs, u64 n) {
  if (!n || !n_limbs) return;
  hipLaunchKernelGGL(expand_small_kernel, ew_grid(n, n_limbs), dim3(kThreads), 0, st, c, r, v, lm, n);
}

// ---- per-limb scalars: Scalars_integer_add_poly / Scalars_integer_multiply_poly (poly/src/rns_poly.c) ----
template <int MUL>
__global__ __launch_bounds__(kThreads) void limb_scalar_kernel(DevCtx c, u64* __restrict__ r, const u64* __restrict__ a,
                                                               LimbScalars s, LimbMap lm, u64 n) {
  const u32 limb = blockIdx.y;
  const DevPrime P = c.primes[lm.prime[limb]];
  const u64 base = (u64)limb * n, v = s.v[limb];
#pragma unroll
  ACE_EW_LOOP(i, n) r[base + i] = MUL ? mulmod(a[base + i], v, P) : add_mod(a[base + i], v, P.q);
}
void launch_limb_scalars(hipStream_t st, const DevCtx& c, bool mul, u64* r, const u64* a, const LimbScalars& s,
                         const LimbMap& lm, u32 n_limbs, u64 n) {
  if (!n || !n_limbs) return;
  if (mul)
    hipLaunchKernelGGL(limb_scalar_kernel<1>, ew_grid(n, n_limbs), dim3(kThreads), 0, st, c, r, a, s, lm, n);
  else
    hipLaunchKernelGGL(limb_scalar_kernel<0>, ew_grid(n, n_limbs), dim3(kThreads), 0, st, c, r, a, s, lm, n);
}

// ---- weighted sum of ciphertexts: (r0, r1) = sum_j w[j][limb] * (a0_j, a1_j) -------------------------------
// (Mul_const + Add_ciphertext over the terms of Eval_linear_wsum, ckks/src/chebyshev_impl.c:276-318)
__global__ __launch_bounds__(kThreads) void wsum_kernel(DevCtx c, u64* __restrict__ r0, u64* __restrict__ r1,
                                                        MacSet ops, const u64* __restrict__ w, LimbMap lm,
                                                        u32 n_limbs, u64 n) {
  const u32 limb = blockIdx.y;
  const DevPrime P = c.primes[lm.prime[limb]];
  const u64 base = (u64)limb * n;
#pragma unroll
  ACE_EW_LOOP(i, n) {
    // summed in 128 bits, reduced once: at most kMaxMacOps = 32 products of residues below 2^61 (the weights are
    // checked to be residues by the caller)
    u64 l0 = 0, l1 = 0, h0 = 0, h1 = 0;
    for (u32 j = 0; j < ops.n; ++j) {
      u64 v = w[j * n_limbs + limb];
      mac128(h0, l0, ops.a0[j][base + i], v);
      mac128(h1, l1, ops.a1[j][base + i], v);
    }
    r0[base + i] = barrett128(h0, l0, P);
    r1[base + i] = barrett128(h1, l1, P);
  }
}
void launch_wsum(hipStream_t st, const DevCtx& c, u64* r0, u64* r1, const MacSet& ops, const u64* w,
                 const LimbMap& lm, u32 n_limbs, u64 n) {
  if (!n || !n_limbs || !ops.n) return;
  hipLaunchKernelGGL(wsum_kernel, ew_grid(n, n_limbs), dim3(kThreads), 0, st, c, r0, r1, ops, w, lm, n_limbs, n);
}

// ---- Hw_rotate / Automorphism_transform (hal.c:123-138, rns_poly.c:1056-1099)
// blockIdx.z = rotation: its own index table, input pair and output pair.
__global__ __launch_bounds__(kThreads) void gather_kernel(DevCtx c, u64* __restrict__ r0, u64* __restrict__ r1,
                                                          u64 r_stride, const u64* __restrict__ a0,
                                                          const u64* __restrict__ a1, u64 a_stride, OrderSet orders,
                                                          LimbMap lm, u64 n) {
  const u32 limb = blockIdx.y, z = blockIdx.z;
  const u64 q = c.primes[lm.prime[limb]].q;
  const u64 base = (u64)limb * n;
  const i64* __restrict__ order = orders.p[orders.n == 1 ? 0 : z];
  r0 += z * r_stride;
  a0 += z * a_stride;
  if (r1) { r1 += z * r_stride; a1 += z * a_stride; }
#pragma unroll
  ACE_EW_LOOP(i, n) {
    i64 k = order[i];
    if (k >= 0) {
      r0[base + i] = a0[base + k];
      if (r1) r1[base + i] = a1[base + k];
    } else {
      r0[base + i] = q - a0[base - k];
      if (r1) r1[base + i] = q - a1[base - k];
    }
  }
}

void launch_gather(hipStream_t st, const DevCtx& c, u64* r, const u64* a, const i64* order, const LimbMap& lm,
                   u32 n_limbs, u64 n) {
  if (!n || !n_limbs) return;
  OrderSet os{};
  os.n = 1;
  os.p[0] = order;
  hipLaunchKernelGGL(gather_kernel, ew_grid(n, n_limbs), dim3(kThreads), 0, st, c, r, (u64*)nullptr, (u64)0, a,
                     (const u64*)nullptr, (u64)0, os, lm, n);
}
void launch_gather2(hipStream_t st, const DevCtx& c, u64* r0, u64* r1, u64 r_stride, const u64* a0, const u64* a1,
                    u64 a_stride, const OrderSet& orders, const LimbMap& lm, u32 n_limbs, u32 n_rot) {
  if (!n_limbs || !n_rot) return;
  hipLaunchKernelGGL(gather_kernel, ew_grid(c.N, n_limbs, n_rot), dim3(kThreads), 0, st, c, r0, r1, r_stride, a0, a1,
                     a_stride, orders, lm, (u64)c.N);
}

// ---- Mul_ciphertext3 (evaluator.c:142-175) in one pass -------------------
__global__ __launch_bounds__(kThreads) void tensor_kernel(DevCtx c, u64* __restrict__ d0, u64* __restrict__ d1,
                                                          u64* __restrict__ d2, const u64* __restrict__ a0,
                                                          const u64* __restrict__ a1, const u64* __restrict__ b0,
                                                          const u64* __restrict__ b1, LimbMap lm, u64 d01_stride,
                                                          u64 d2_stride, u64 in_stride) {
  const u32 limb = blockIdx.y;
  const DevPrime P = c.primes[lm.prime[limb]];
  const u64 n = c.N, base = (u64)limb * n;
  d0 += blockIdx.z * d01_stride; d1 += blockIdx.z * d01_stride; d2 += blockIdx.z * d2_stride;
  a0 += blockIdx.z * in_stride; a1 += blockIdx.z * in_stride;
  b0 += blockIdx.z * in_stride; b1 += blockIdx.z * in_stride;
#pragma unroll
  ACE_EW_LOOP(i, n) {
    u64 x0 = ldn<1>(a0 + base + i), x1 = ldn<1>(a1 + base + i), y0 = ldn<1>(b0 + base + i), y1 = ldn<1>(b1 + base + i);
    stn<1>(d0 + base + i, mulmod(x0, y0, P));
    stn<1>(d1 + base + i, add_mod(mulmod(x0, y1, P), mulmod(x1, y0, P), P.q));
    stn<1>(d2 + base + i, mulmod(x1, y1, P));
  }
}

// the last term alone, for callers that form the other two where they are consumed (Lift)
__global__ __launch_bounds__(kThreads) void tensor_d2_kernel(DevCtx c, u64* __restrict__ d2, const u64* __restrict__ a1,
                                                             const u64* __restrict__ b1, LimbMap lm, u64 d2_stride,
                                                             u64 in_stride) {
  const u32 limb = blockIdx.y;
  const DevPrime P = c.primes[lm.prime[limb]];
  const u64 n = c.N, base = (u64)limb * n;
  d2 += blockIdx.z * d2_stride;
  a1 += blockIdx.z * in_stride;
  b1 += blockIdx.z * in_stride;
#pragma unroll
  ACE_EW_LOOP(i, n) stn<1>(d2 + base + i, mulmod(ldn<1>(a1 + base + i), ldn<1>(b1 + base + i), P));
}

void launch_tensor(hipStream_t st, const DevCtx& c, u64* d0, u64* d1, u64* d2, const u64* a0, const u64* a1,
                   const u64* b0, const u64* b1, const LimbMap& lm, u32 n_limbs, u32 n_ops, u64 d01_stride,
                   u64 d2_stride, u64 in_stride) {
  if (!n_limbs || !n_ops) return;
  if (!d0) {
    hipLaunchKernelGGL(tensor_d2_kernel, ew_grid(c.N, n_limbs, n_ops), dim3(kThreads), 0, st, c, d2, a1, b1, lm,
                       d2_stride, in_stride);
    return;
  }
  hipLaunchKernelGGL(tensor_kernel, ew_grid(c.N, n_limbs, n_ops), dim3(kThreads), 0, st, c, d0, d1, d2, a0, a1, b0,
                     b1, lm, d01_stride, d2_stride, in_stride);
}

// ---- fast base conversion (rns_poly.c:218-242, rns_poly_impl.c:324-336) ----
// One thread per coefficient and kConvTargets targets.  blockIdx.z enumerates (operand, job): a job is one
// digit's conversion, all jobs of a launch share the operand strides.
//
// Targets below kFpConvTargetLimit are converted in exact FP64 arithmetic: a source word (< 2^63) is cut into
// three 21-bit pieces; the table holds, for piece i of source k, the two halves (above and below bit 26) of
// hat * 2^(21 i) mod m.  3 * 16 products below 2^47 add up exactly in each of the two sums (below 2^52.6 < 2^53,
// one FMA each), and high * 2^26 + low is reduced once per target.  A group whose targets are all of that kind
// makes one pass over the sources with the table read through wave-uniform loads, a row of it holding the group's
// entries side by side.  Larger targets (the 60-bit special primes) take nd 128-bit multiply-adds and one
// Barrett reduction each, from source words kept in registers.
constexpr int kConvTargets = 4;

__device__ __forceinline__ void conv_pieces(u64 x, double piece[3]) {
  piece[0] = (double)((u32)x & 0x1FFFFFu);
  piece[1] = (double)((u32)(x >> 21) & 0x1FFFFFu);
  piece[2] = (double)(u32)(x >> 42);
}

__device__ __forceinline__ u64 conv_fp_finish(double hi, double lo, double q, double qinv) {
#pragma clang fp contract(off)
  hi = __builtin_fma(-__builtin_rint(hi * qinv), q, hi);  // |hi| <= m/2
  lo = __builtin_fma(-__builtin_rint(lo * qinv), q, lo);
  // hi * 2^26 mod m: the product is exact (a power of two), the quotient is off by less than 1/2 + |hi| 2^-52
  const double c = __builtin_rint(hi * (67108864.0 * qinv));
  double acc = __builtin_fma(-c, q, hi * 67108864.0) + lo;  // |acc| < 1.4 m < 2^53
  acc = __builtin_fma(-__builtin_rint(acc * qinv), q, acc);
  acc = acc < 0.0 ? acc + q : acc;
  return (u64)__double_as_longlong(acc + 4503599627370496.0) & 0x000FFFFFFFFFFFFFull;
}

// MAXS: compile-time bound on the number of source limbs (register array of the integer path); 0 = any number,
// looped, integer arithmetic only.  FP: every job of the launch has FP64 tables.
template <int MAXS, int FP>
__global__ __launch_bounds__(kThreads) void baseconv_kernel(DevCtx c, u64* __restrict__ out_base,
                                                            const u64* __restrict__ t_base, ConvBatch b) {
  const u64 n = c.N;
  const u64 i = (u64)blockIdx.x * kThreads + threadIdx.x;
  if (i >= n) return;
  const u32 jobi = blockIdx.z % b.n_jobs, op = blockIdx.z / b.n_jobs;
  const ConvJob& J = b.job[jobi];
  const u32 nd = J.nd, nc = J.nc, hat_stride = J.hat_stride;
  const u64* __restrict__ hat = J.hat;
  const u64* __restrict__ t = t_base + op * b.t_stride + J.t_off;
  u64* __restrict__ out = out_base + op * b.out_stride + J.out_off;
  const u32 j0 = blockIdx.y * kConvTargets;
  if (j0 >= nc) return;
  if constexpr (MAXS > 0) {
    if constexpr (FP != 0) {
      bool all_fp = true;  // wave-uniform
#pragma unroll
      for (int jj = 0; jj < kConvTargets; ++jj) all_fp &= j0 + jj >= nc || J.fp_target[j0 + jj] != 0;
      if (all_fp) {
        // rows are read up to three entries past a ragged last group: the table is allocated with that margin
        double hi[kConvTargets], lo[kConvTargets];
#pragma unroll
        for (int jj = 0; jj < kConvTargets; ++jj) hi[jj] = lo[jj] = 0.0;
        const double2* __restrict__ row = reinterpret_cast<const double2*>(J.fw) + j0;
        const u32 stride = J.fw_stride;
#pragma unroll 4
        for (u32 k = 0; k < nd; ++k) {
          double piece[3];
          conv_pieces(t[(u64)k * n + i], piece);
#pragma unroll
          for (int pc = 0; pc < 3; ++pc) {
#pragma unroll
            for (int jj = 0; jj < kConvTargets; ++jj) {
              const double2 ww = row[(u64)(3 * k + pc) * stride + jj];
              hi[jj] = __builtin_fma(piece[pc], ww.x, hi[jj]);
              lo[jj] = __builtin_fma(piece[pc], ww.y, lo[jj]);
            }
          }
        }
#pragma unroll
        for (int jj = 0; jj < kConvTargets; ++jj) {
          const u32 j = j0 + jj;
          if (j < nc) out[(u64)J.map.out_limb[j] * n + i] = conv_fp_finish(hi[jj], lo[jj], J.fq[2 * j], J.fq[2 * j + 1]);
        }
        return;
      }
    }
    u64 x[MAXS];
#pragma unroll
    for (int k = 0; k < MAXS; ++k) x[k] = (u32)k < nd ? t[(u64)k * n + i] : 0;
#pragma unroll
    for (int jj = 0; jj < kConvTargets; ++jj) {
      u32 j = j0 + jj;
      if (j >= nc) break;
      if (FP != 0 && J.fp_target[j]) {  // wave-uniform: an FP64 target in a group that has others too
        double hi = 0.0, lo = 0.0;
        const double2* __restrict__ col = reinterpret_cast<const double2*>(J.fw) + j;
#pragma unroll
        for (int k = 0; k < MAXS; ++k) {
          if ((u32)k < nd) {
            double piece[3];
            conv_pieces(x[k], piece);
#pragma unroll
            for (int pc = 0; pc < 3; ++pc) {
              const double2 ww = col[(u64)(3 * k + pc) * J.fw_stride];
              hi = __builtin_fma(piece[pc], ww.x, hi);
              lo = __builtin_fma(piece[pc], ww.y, lo);
            }
          }
        }
        out[(u64)J.map.out_limb[j] * n + i] = conv_fp_finish(hi, lo, J.fq[2 * j], J.fq[2 * j + 1]);
        continue;
      }
      u64 hi = 0, lo = 0;
#pragma unroll
      for (int k = 0; k < MAXS; ++k)
        if ((u32)k < nd) mac128(hi, lo, x[k], hat[(u64)k * hat_stride + j]);
      out[(u64)J.map.out_limb[j] * n + i] = barrett128(hi, lo, c.primes[J.map.prime[j]]);
    }
  } else {
    for (int jj = 0; jj < kConvTargets; ++jj) {
      u32 j = j0 + jj;
      if (j >= nc) break;
      const DevPrime P = c.primes[J.map.prime[j]];
      u64 hi = 0, lo = 0;
      for (u32 k = 0; k < nd; ++k) {
        mac128(hi, lo, t[(u64)k * n + i], hat[(u64)k * hat_stride + j]);
        if ((k & 7) == 7) { lo = barrett128(hi, lo, P); hi = 0; }  // keep the sum below 2^128
      }
      out[(u64)J.map.out_limb[j] * n + i] = barrett128(hi, lo, P);
    }
  }
}

// ---- the same conversion on the matrix cores ------------------------------------------------------------------
// out_j = sum_k x_k * hat_kj (mod m_j) is a matrix product over the bytes of the source words: with the signed bytes
// d_ka of x_k (x_k = sum_a d_ka 2^(8a), d in [-128, 127]) and the constants C_kaj = hat_kj * 2^(8a) mod m_j cut
// into signed bytes the same way (C = sum_p e_kajp 2^(8p)), V_j = sum_p 2^(8p) sum_(k,a) d_ka e_kajp is congruent to
// the sum mod m_j.  The inner sums are one int8 MFMA product: rows (target, p), columns = coefficients, inner index
// (k, a) -- a source word as it lies in memory is eight consecutive inner indices.  |V_j| < 2^14 m_j, so the
// quotient has 15 bits, an FP64 estimate of it is off by less than one, and V_j - Q m_j is taken in wrapping 64-bit
// arithmetic: the canonical residue, the same word the multiply-accumulate path gives.
// v_mfma_i32_32x32x32_i8: lane l holds row (column) l % 32 and inner indices 16 (l / 32) .. + 15 of the A (B) operand;
// result register r of lane l is row 8 (r / 4) + 4 (l / 32) + r % 4 of column l % 32.  The table's rows are permuted so
// that registers 0-7 of a lane are the eight byte sums of target 2 (l / 32) of the quad, registers 8-15 those of target
// 2 (l / 32) + 1.
// Source words must be below 2^63 - 2^56 (residues of primes below 2^61 are).
constexpr u32 kMxThreads = 256, kMxCoefPerBlock = 64 * (kMxThreads / 64);

// one quad of targets for the wave's two tiles; FULL: all four targets exist (no lane is left out, so the stores
// are unconditional and the waits the compiler places do not have to allow for a path without them)
template <int STEPS, bool FULL>
__device__ __forceinline__ void conv_mx_quad(const uint4 (&row)[STEPS], const ConvTarget (&tg)[2],
                                             const conv_v4i (&x)[2][STEPS], u64* __restrict__ out, u32 first_target,
                                             u32 nc) {
  conv_v16i acc[2];
#pragma unroll
  for (u32 tile = 0; tile < 2; ++tile) {
    acc[tile] = conv_v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const conv_v4i a = {(int)row[s].x, (int)row[s].y, (int)row[s].z, (int)row[s].w};
      acc[tile] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, x[tile][s], acc[tile], 0, 0, 0);
    }
  }
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    const u64 m = tg[w].m;
    u64 res[2];
#pragma unroll
    for (u32 tile = 0; tile < 2; ++tile) res[tile] = conv_mx_residue(acc[tile], w, m, tg[w].minv);
    if (FULL || first_target + w < nc)
    {
      typedef u64 u64x2 __attribute__((ext_vector_type(2)));
      const u64x2 pr = {res[0], res[1]};
      stn<8>(reinterpret_cast<u64x2*>(out + tg[w].out_off), pr);
    }
  }
}

// A wave converts 64 coefficients as two tiles of 32 (lane column c of tile e is coefficient 2 c + e, so a lane
// loads and stores its two coefficients as one 16-byte word), one quad of targets after the other; the table rows of
// the next quad are requested before the current one is worked on (the tables end with a spare quad).
template <int STEPS>
__global__ __launch_bounds__(kMxThreads) void baseconv_mx_kernel(DevCtx c, u64* __restrict__ out_base,
                                                                 const u64* __restrict__ t_base, ConvBatch b,
                                                                 u32 quads_per_block) {
  const u64 n = c.N;
  const u32 lane = threadIdx.x & 63, half = lane >> 5;
  const u64 i = ((u64)blockIdx.x * (kMxThreads / 64) + (threadIdx.x >> 6)) * 64 + 2 * (lane & 31);
  const u32 jobi = blockIdx.z % b.n_jobs, op = blockIdx.z / b.n_jobs;
  const ConvJob& J = b.job[jobi];
  const u32 nd = J.nd, nc = J.nc;
  const u32 quad0 = blockIdx.y * quads_per_block;
  if (quad0 * 4 >= nc) return;
  const u32 quad1 = min(quad0 + quads_per_block, (nc + 3) / 4);
  const u32 full1 = min(quad1, nc / 4);  // quads below this one have all four targets
  const u64* __restrict__ t = t_base + op * b.t_stride + J.t_off + i;
  u64* __restrict__ out = out_base + op * b.out_stride + J.out_off + i;
  conv_v4i x[2][STEPS];
  {
    ulonglong2 v[STEPS][2];
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const u32 k = 4 * s + 2 * half + w;
        {
          typedef u64 u64x2 __attribute__((ext_vector_type(2)));
          const u64x2 pr = ldn<8>(reinterpret_cast<const u64x2*>(t + (u64)min(k, nd - 1) * n));
          v[s][w] = make_ulonglong2(pr.x, pr.y);
        }
      }
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const bool live = 4 * s + 2 * half + w < nd;
        int lo, hi;
        conv_mx_signed(v[s][w].x, live, lo, hi);
        x[0][s][2 * w] = lo;
        x[0][s][2 * w + 1] = hi;
        conv_mx_signed(v[s][w].y, live, lo, hi);
        x[1][s][2 * w] = lo;
        x[1][s][2 * w + 1] = hi;
      }
  }
  const uint4* __restrict__ mx = J.mx + (u64)quad0 * kMxSteps * 64 + lane;
  const ConvTarget* __restrict__ mt = J.mt + quad0 * 4 + 2 * half;
  uint4 row[STEPS];
  ConvTarget tg[2];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) row[s] = mx[s * 64];
  tg[0] = mt[0];
  tg[1] = mt[1];
  u32 quad = quad0;
  for (; quad < full1; ++quad) {
    mx += kMxSteps * 64;
    mt += 4;
    uint4 row_next[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) row_next[s] = mx[s * 64];
    const ConvTarget tg_next[2] = {mt[0], mt[1]};
    conv_mx_quad<STEPS, true>(row, tg, x, out, quad * 4 + 2 * half, nc);
#pragma unroll
    for (int s = 0; s < STEPS; ++s) row[s] = row_next[s];
    tg[0] = tg_next[0];
    tg[1] = tg_next[1];
  }
  if (quad < quad1) conv_mx_quad<STEPS, false>(row, tg, x, out, quad * 4 + 2 * half, nc);
}

// register-array size used for nd source limbs (0: the looped kernel)
static int conv_padded_sources(u32 nd) { return nd <= 4 ? 4 : nd <= 8 ? 8 : nd <= 12 ? 12 : nd <= 16 ? 16 : 0; }

void launch_baseconv(hipStream_t st, const DevCtx& c, u64* out, const u64* t, const ConvBatch& b, u32 n_ops) {
  if (!b.n_jobs || !n_ops) return;
  u32 max_nc = 0, max_nd = 0;
  bool fp = true;  // jobs without FP64 tables keep the launch to integer arithmetic
  for (u32 k = 0; k < b.n_jobs; ++k) {
    max_nc = b.job[k].nc > max_nc ? b.job[k].nc : max_nc;
    max_nd = b.job[k].nd > max_nd ? b.job[k].nd : max_nd;
    fp &= b.job[k].fw != nullptr;
  }
  if (!max_nc) return;
  bool mx = b.matrix && c.N % kMxCoefPerBlock == 0 && max_nd <= 4 * kMxSteps &&
            ((uintptr_t)out | (uintptr_t)t) % 16 == 0 && (b.out_stride | b.t_stride) % 2 == 0;
  for (u32 k = 0; k < b.n_jobs; ++k) mx &= b.job[k].mx != nullptr;
  if (mx) {
    const u32 quads = (max_nc + 3) / 4, steps = (max_nd + 3) / 4;
    // all targets of a job in one block (the source words are loaded once) unless that leaves the machine empty
    const u32 blocks = (u32)(c.N / kMxCoefPerBlock) * b.n_jobs * n_ops;
    u32 split = blocks >= 1024 ? 1 : (1024 + blocks - 1) / blocks;
    split = split > quads ? quads : split;
    const u32 per_block = (quads + split - 1) / split;
    dim3 g((u32)(c.N / kMxCoefPerBlock), (quads + per_block - 1) / per_block, b.n_jobs * n_ops);
#define ACE_BCX(S) hipLaunchKernelGGL((baseconv_mx_kernel<S>), g, dim3(kMxThreads), 0, st, c, out, t, b, per_block)
    switch (steps) {
      case 1: ACE_BCX(1); break;
      case 2: ACE_BCX(2); break;
      case 3: ACE_BCX(3); break;
      default: ACE_BCX(4); break;
    }
#undef ACE_BCX
    return;
  }
  const int maxs = conv_padded_sources(max_nd);
  dim3 g((c.N + kThreads - 1) / kThreads, (max_nc + kConvTargets - 1) / kConvTargets, b.n_jobs * n_ops);
#define ACE_BC(S, M) hipLaunchKernelGGL((baseconv_kernel<S, M>), g, dim3(kThreads), 0, st, c, out, t, b)
#define ACE_BC_MODES(S) \
  do { if (fp) ACE_BC(S, 1); else ACE_BC(S, 0); } while (0)
  switch (maxs) {
    case 4: ACE_BC_MODES(4); break;
    case 8: ACE_BC_MODES(8); break;
    case 12: ACE_BC_MODES(12); break;
    case 16: ACE_BC_MODES(16); break;
    default: ACE_BC(0, 0); break;
  }
#undef ACE_BC_MODES
#undef ACE_BC
}

// copies the digit limbs of `src` (level limbs per operand) into their places
// in the raised polynomials: limb t of digit d = t / part_size goes to
// res + op*res_stride + d*digit_stride + t*N  (Decomp, rns_poly.c:74-105)
__global__ __launch_bounds__(kThreads) void digit_copy_kernel(u64* __restrict__ res, const u64* __restrict__ src,
                                                              u64 n, u32 part_size, u32 n_digits, u64 digit_stride,
                                                              u64 res_stride, u64 src_stride) {
  const u32 limb = blockIdx.y, op = blockIdx.z;
  u32 d = limb / part_size;
  if (d >= n_digits) d = n_digits - 1;
  const u64* __restrict__ s = src + op * src_stride + (u64)limb * n;
  u64* __restrict__ r = res + op * res_stride + d * digit_stride + (u64)limb * n;
#pragma unroll
  ACE_EW_LOOP(i, n) r[i] = s[i];
}
void launch_digit_copy(hipStream_t st, const DevCtx& c, u64* res, const u64* src, u32 level, u32 part_size,
                       u32 n_digits, u64 digit_stride, u64 res_stride, u64 src_stride, u32 n_ops) {
  if (!level || !n_ops) return;
  hipLaunchKernelGGL(digit_copy_kernel, ew_grid(c.N, level, n_ops), dim3(kThreads), 0, st, res, src, (u64)c.N,
                     part_size, n_digits, digit_stride, res_stride, src_stride);
}

__global__ __launch_bounds__(kThreads) void order_check_kernel(const i64* __restrict__ order, u32 n, u32* report) {
  const u32 i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= n) return;
  const i64 v = order[i], first = order[i & ~4095u];
  if (v < 0 || v >= (i64)n || first < 0 || (v >> 12) != (first >> 12)) report[0] = 1;
  if ((i & 4095u) == 0) report[1 + (i >> 12)] = (u32)((u64)v >> 12);
}
void launch_order_check(hipStream_t st, const DevCtx& c, const i64* order, u32* report) {
  hipLaunchKernelGGL(order_check_kernel, dim3((c.N + kThreads - 1) / kThreads), dim3(kThreads), 0, st, order, c.N,
                     report);
}

// ---- Dot_prod (rns_poly.c:502-529, rns_poly_impl.c:102-162) ----------------
// Both key halves in one pass so the digits are read once.  Products of residues are accumulated in 128 bits
// (the reference's Fast_dotprod_poly) and reduced by one single-word Barrett step while the sum stays below
// 2^(shift + 64); the result equals the reference's multiply-reduce-add chain because canonical residues are unique.
template <bool TWO>
__global__ __launch_bounds__(kThreads) void dotprod_kernel(DevCtx c, u64* __restrict__ out0, u64* __restrict__ out1,
                                                           u64 out_stride, const u64* __restrict__ digits,
                                                           u64 digit_stride, u64 digits_op_stride, KeySet keys,
                                                           u64 key1_off, u64 key_stride, u32 n_parts, LimbMap lm,
                                                           LimbMap key_limb, Lift lift) {
  const u32 limb = blockIdx.y, op = blockIdx.z;
  const bool lifted = TWO && lift.cst && limb < lift.level;
  const u64 lw = lifted ? lift.cst[2 * limb] : 0, lwp = lifted ? lift.cst[2 * limb + 1] : 0;
  const u64* __restrict__ add0 = lifted ? lift.addend.at(2 * op) + (u64)limb * c.N : nullptr;
  const u64* __restrict__ add1 = lifted ? lift.addend.at(2 * op + 1) + (u64)limb * c.N : nullptr;
  const DevPrime P = c.primes[lm.prime[limb]];
  const u64 n = c.N, dbase = (u64)limb * n, kbase = (u64)key_limb.prime[limb] * n;
  const u64* __restrict__ key0 = keys.p[keys.n == 1 ? 0 : op];
  const u64* __restrict__ key1 = key0 + key1_off;
  digits += op * digits_op_stride;
  out0 += op * out_stride;
  if (TWO) out1 += op * out_stride;
  const u32 max_terms = sum_terms(P);
#pragma unroll
  ACE_EW_LOOP(i, n) {
    u64 h0 = 0, l0 = 0, h1 = 0, l1 = 0;
    u32 terms = 0;
    for (u32 d = 0; d < n_parts; ++d) {
      u64 x = ldn<256>(digits + d * digit_stride + dbase + i);
      mac128(h0, l0, x, ldn<256>(key0 + d * key_stride + kbase + i));
      if (TWO) mac128(h1, l1, x, ldn<256>(key1 + d * key_stride + kbase + i));
      if (++terms == max_terms && d + 1 < n_parts) {  // the reduced sum counts as one term
        l0 = barrett_sum(h0, l0, P); h0 = 0;
        if (TWO) { l1 = barrett_sum(h1, l1, P); h1 = 0; }
        terms = 1;
      }
    }
    u64 v0 = barrett_sum(h0, l0, P), v1 = TWO ? barrett_sum(h1, l1, P) : 0;
    if (lifted) {
      v0 = add_mod(v0, shoup_mul(ldn<256>(add0 + i), lw, lwp, P.q), P.q);
      v1 = add_mod(v1, shoup_mul(ldn<256>(add1 + i), lw, lwp, P.q), P.q);
    }
    stn<256>(out0 + dbase + i, v0);
    if (TWO) stn<256>(out1 + dbase + i, v1);
  }
}

// A rotation in the extended basis without its Mod_down (Fast_rotate_ext, evaluator.c:503-566, as bootstrapping
// uses it): both halves of the inner product with the rotation key, an optional addend on the first half, and the
// automorphism, in one pass.  The gather is applied on the way in: out[i] = value at order[i], so writes stay
// coalesced.  NTT form only (no negative index entries).  accumulate: bit 0 adds to what out0 holds, bit 1 to out1.
__global__ __launch_bounds__(kThreads) void ext_rotate_kernel(DevCtx c, u64* __restrict__ out0, u64* __restrict__ out1,
                                                              const u64* __restrict__ digits, u64 digit_stride,
                                                              const u64* __restrict__ key0, u64 key1_off, u64 key_stride,
                                                              u32 n_parts, const u64* __restrict__ addend0,
                                                              const i64* __restrict__ order, int accumulate,
                                                              LimbMap lm, LimbMap key_limb) {
  const u32 limb = blockIdx.y;
  const DevPrime P = c.primes[lm.prime[limb]];
  const u64 n = c.N, dbase = (u64)limb * n, kbase = (u64)key_limb.prime[limb] * n;
  const u64* __restrict__ key1 = key0 + key1_off;
  const u32 max_terms = sum_terms(P);
#pragma unroll
  ACE_EW_LOOP(i, n) {
    const u64 j = (u64)order[i];
    u64 h0 = 0, l0 = 0, h1 = 0, l1 = 0;
    u32 terms = 0;
    for (u32 d = 0; d < n_parts; ++d) {
      const u64 x = digits[d * digit_stride + dbase + j];
      mac128(h0, l0, x, ldn<64>(key0 + d * key_stride + kbase + j));
      mac128(h1, l1, x, ldn<64>(key1 + d * key_stride + kbase + j));
      if (++terms == max_terms && d + 1 < n_parts) {  // the reduced sum counts as one term
        l0 = barrett_sum(h0, l0, P); h0 = 0;
        l1 = barrett_sum(h1, l1, P); h1 = 0;
        terms = 1;
      }
    }
    u64 v0 = barrett_sum(h0, l0, P), v1 = barrett_sum(h1, l1, P);
    if (addend0) v0 = add_mod(v0, addend0[dbase + j], P.q);
    if (accumulate & 1) v0 = add_mod(v0, out0[dbase + i], P.q);
    if (accumulate & 2) v1 = add_mod(v1, out1[dbase + i], P.q);
    stn<64>(out0 + dbase + i, v0);
    stn<64>(out1 + dbase + i, v1);
  }
}
void launch_ext_rotate(hipStream_t st, const DevCtx& c, u64* out0, u64* out1, const u64* digits, u64 digit_stride,
                       const u64* key0, u64 key1_off, u64 key_stride, u32 n_parts, const u64* addend0, const i64* order,
                       int accumulate, const LimbMap& lm, const LimbMap& key_limb, u32 n_limbs) {
  if (!n_limbs) return;
  hipLaunchKernelGGL(ext_rotate_kernel, ew_grid(c.N, n_limbs, 1), dim3(kThreads), 0, st, c, out0, out1, digits,
                     digit_stride, key0, key1_off, key_stride, n_parts, addend0, order, accumulate, lm, key_limb);
}

// The same for operands that share one key: each thread keeps its 2*NP key
// words in registers and walks the operands blockIdx.z, blockIdx.z + gridDim.z, ...
// so the key, the largest stream of a key switch, is fetched gridDim.z times
// instead of once per operand.
// coefficients per thread of the kernel below: one (60-106 registers, four to eight waves per SIMD) serves the batched
// key switch best: 377 us against 396 with two and 431 with four, whose 170 registers leave two waves per SIMD
constexpr int kKeyUnroll = 1;
template <int NP>
__global__ __launch_bounds__(kThreads) void dotprod_shared_key_kernel(
    DevCtx c, u64* __restrict__ out0, u64* __restrict__ out1, u64 out_stride, const u64* __restrict__ digits,
    u64 digit_stride, u64 digits_op_stride, const u64* __restrict__ key0, u64 key1_off, u64 key_stride, LimbMap lm,
    LimbMap key_limb, u32 n_ops, OwnLimbs own, Lift lift, u32 blocks_x, u32 n_limbs, u32 split) {
  // one-dimensional grid: the `split` work-groups that share a tile of the key are neighbours on one XCD (see
  // dotprod_shared_digits_kernel)
  const u32 xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  const u32 tile = (local / split) * 8 + xcd, first_op = local % split;
  if (tile >= blocks_x * n_limbs) return;
  const u32 limb = tile / blocks_x, bx = tile % blocks_x;
  const DevPrime P = c.primes[lm.prime[limb]];
  const bool lifted = lift.cst && limb < lift.level;
  const u64 lw = lifted ? lift.cst[2 * limb] : 0, lwp = lifted ? lift.cst[2 * limb + 1] : 0;
  const u64 n = c.N, dbase = (u64)limb * n, kbase = (u64)key_limb.prime[limb] * n;
  const u64* __restrict__ key1 = key0 + key1_off;
  // the digit this limb is an own limb of (NP: none, or the digits hold their own limbs)
  const int own_d = ((own.src || own.product) && limb < own.level) ? min((int)(limb / own.part_size), NP - 1) : NP;
  // ... whose words are the product a1 b1 of the operands the lifted terms are formed from (never stored)
  const bool own_product = own.product && own_d < NP;
  // the thread's kKeyUnroll coefficients are handled together so that every operand has
  // kKeyUnroll * NP independent loads in flight
  const u64 i0 = (u64)bx * (kThreads * kKeyUnroll) + threadIdx.x;
  u64 k0[kKeyUnroll][NP], k1[kKeyUnroll][NP];
#pragma unroll
  for (int u = 0; u < kKeyUnroll; ++u) {
    const u64 i = i0 + u * kThreads;
#pragma unroll
    for (int d = 0; d < NP; ++d) {
      k0[u][d] = i < n ? ldn<16>(key0 + d * key_stride + kbase + i) : 0;
      k1[u][d] = i < n ? ldn<16>(key1 + d * key_stride + kbase + i) : 0;
    }
  }
  for (u32 op = first_op; op < n_ops; op += split) {
    const u64* __restrict__ dg = digits + op * digits_op_stride + dbase;
    u64 x[kKeyUnroll][NP];
#pragma unroll
    for (int u = 0; u < kKeyUnroll; ++u) {
      const u64 i = i0 + u * kThreads;
#pragma unroll
      for (int d = 0; d < NP; ++d)
        x[u][d] = (i >= n || (d == own_d && own_product)) ? 0
                  : d == own_d ? ldn<2>(own.src + op * own.op_stride + dbase + i) : ldn<2>(dg + d * digit_stride + i);
    }
#pragma unroll
    for (int u = 0; u < kKeyUnroll; ++u) {
      const u64 i = i0 + u * kThreads;
      u64 h0 = 0, l0 = 0, h1 = 0, l1 = 0;
      // The lifted tensor terms P a0 b0 and P (a0 b1 + a1 b0) join the sums before their one reduction where the sums
      // have room for two more products: P a0 and P a1 are reduced (two Shoup products), the three products with
      // b0 / b1 are not.  The residue of the whole sum is the same word as the sum of the residues.
      const bool fold = lifted && lift.a0 && sum_terms(P) >= NP + 2;
      u64 x0 = 0, x1 = 0, y0 = 0, y1 = 0;
      if (fold && i < n) {
        const u64 o = op * lift.in_stride + dbase + i;
        x0 = ldn<2>(lift.a0 + o), x1 = ldn<2>(lift.a1 + o), y0 = ldn<2>(lift.b0 + o), y1 = ldn<2>(lift.b1 + o);
      }
      const u64 own_word = own_product ? mulmod(x1, y1, P) : 0;  // (the host asks for it only where every limb folds)
#pragma unroll
      for (int d = 0; d < NP; ++d) {
        const u64 xd = (own_product && d == own_d) ? own_word : x[u][d];
        mac128(h0, l0, xd, k0[u][d]);
        mac128(h1, l1, xd, k1[u][d]);
      }
      if (fold && i < n) {
        const u64 px0 = shoup_mul(x0, lw, lwp, P.q), px1 = shoup_mul(x1, lw, lwp, P.q);
        mac128(h0, l0, px0, y0);
        mac128(h1, l1, px0, y1);
        mac128(h1, l1, px1, y0);
      }
      if (i < n) {  // NP <= 4 products: below 2^(shift + 64) for every prime below 2^61
        u64 v0 = barrett_sum(h0, l0, P), v1 = barrett_sum(h1, l1, P);
        if (fold) {
        } else if (lifted && lift.a0) {
          const u64 o = op * lift.in_stride + dbase + i;
          const u64 x0 = ldn<2>(lift.a0 + o), x1 = ldn<2>(lift.a1 + o), y0 = ldn<2>(lift.b0 + o), y1 = ldn<2>(lift.b1 + o);
          u64 h = 0, l = 0;  // two products of residues stay below 2^(shift + 64)
          mac128(h, l, x0, y1);
          mac128(h, l, x1, y0);
          v0 = add_mod(v0, shoup_mul(mulmod(x0, y0, P), lw, lwp, P.q), P.q);
          v1 = add_mod(v1, shoup_mul(barrett_sum(h, l, P), lw, lwp, P.q), P.q);
        } else if (lifted) {
          v0 = add_mod(v0, shoup_mul(ldn<2>(lift.addend.at(2 * op) + dbase + i), lw, lwp, P.q), P.q);
          v1 = add_mod(v1, shoup_mul(ldn<2>(lift.addend.at(2 * op + 1) + dbase + i), lw, lwp, P.q), P.q);
        }
        stn<2>(out0 + op * out_stride + dbase + i, v0);
        stn<2>(out1 + op * out_stride + dbase + i, v1);
      }
    }
  }
}

// The mirror case, rotations of one ciphertext: every operand multiplies the
// same digits by its own key.  The NP digit words stay in registers while the
// thread walks the operands, so the digits are fetched gridDim.z times instead
// of once per rotation (they do not survive in L2 between rotations: each
// rotation streams a whole key through it).
constexpr int kDigitsUnroll = 4;  // coefficients per thread of the kernel below (two: 754 us against 732 for the 32-rotation batch)
template <int NP>
__global__ __launch_bounds__(kThreads) void dotprod_shared_digits_kernel(
    DevCtx c, u64* __restrict__ out0, u64* __restrict__ out1, u64 out_stride, const u64* __restrict__ digits,
    u64 digit_stride, KeySet keys, u64 key1_off, u64 key_stride, LimbMap lm, LimbMap key_limb, u32 n_ops,
    u32 blocks_x, u32 n_limbs, u32 split) {
  // The grid is one-dimensional.  Hardware hands consecutive work-groups to the 8 XCDs in turn, each with its own L2:
  // the `split` work-groups that share a tile of the digits (same coefficients, same limb, different keys) are
  // consecutive work-groups of one XCD, so the tile comes from memory once and from that L2 for the others.
  const u32 xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  const u32 tile = (local / split) * 8 + xcd, first_op = local % split;
  if (tile >= blocks_x * n_limbs) return;
  const u32 limb = tile / blocks_x, bx = tile % blocks_x;
  const DevPrime P = c.primes[lm.prime[limb]];
  const u64 n = c.N, dbase = (u64)limb * n, kbase = (u64)key_limb.prime[limb] * n;
  const u64 i0 = (u64)bx * (kThreads * kDigitsUnroll) + threadIdx.x;
  u64 x[kDigitsUnroll][NP];
#pragma unroll
  for (int u = 0; u < kDigitsUnroll; ++u) {
    const u64 i = i0 + u * kThreads;
#pragma unroll
    for (int d = 0; d < NP; ++d) x[u][d] = i < n ? ldn<32>(digits + d * digit_stride + dbase + i) : 0;
  }
  for (u32 op = first_op; op < n_ops; op += split) {
    const u64* __restrict__ key0 = keys.p[op] + kbase;
    const u64* __restrict__ key1 = key0 + key1_off;
    u64 k0[kDigitsUnroll][NP], k1[kDigitsUnroll][NP];
#pragma unroll
    for (int u = 0; u < kDigitsUnroll; ++u) {
      const u64 i = i0 + u * kThreads;
#pragma unroll
      for (int d = 0; d < NP; ++d) {
        k0[u][d] = i < n ? ldn<4>(key0 + d * key_stride + i) : 0;
        k1[u][d] = i < n ? ldn<4>(key1 + d * key_stride + i) : 0;
      }
    }
#pragma unroll
    for (int u = 0; u < kDigitsUnroll; ++u) {
      const u64 i = i0 + u * kThreads;
      u64 h0 = 0, l0 = 0, h1 = 0, l1 = 0;
#pragma unroll
      for (int d = 0; d < NP; ++d) {
        mac128(h0, l0, x[u][d], k0[u][d]);
        mac128(h1, l1, x[u][d], k1[u][d]);
      }
      if (i < n) {  // NP <= 4 products: below 2^(shift + 64) for every prime below 2^61
        stn<4>(out0 + op * out_stride + dbase + i, barrett_sum(h0, l0, P));
        stn<4>(out1 + op * out_stride + dbase + i, barrett_sum(h1, l1, P));
      }
    }
  }
}

// How many blocks share the walk over the operands of a batch (blockIdx.z): the shared operand is fetched that many
// times.  A key is 93 MiB, so the kernel that shares it splits the operands two ways only; the digits that
// rotations share are a twentieth of one key, and sixteen blocks walking two keys each keep more of the machine's
// memory channels busy than four walking eight (rotations +2 %; eight walking four and thirty-two walking one are
// slower again: 773 and 754 us against 732 for the 32-rotation batch).
constexpr u32 kSharedKeySplit = 2, kSharedDigitsSplit = 16;
bool dotprod_reads_own(u32 n_keys, u32 n_ops, bool two_halves, u32 n_parts) {
  return n_keys == 1 && n_ops > 1 && two_halves && n_parts >= 1 && n_parts <= 4;
}

void launch_dotprod(hipStream_t st, const DevCtx& c, u64* out0, u64* out1, u64 out_stride, const u64* digits,
                    u64 digit_stride, u64 digits_op_stride, const KeySet& keys, u64 key1_off, u64 key_stride,
                    u32 n_parts, const LimbMap& lm, const LimbMap& key_limb, u32 n_limbs, u32 n_ops,
                    const OwnLimbs* own, const Lift* lift) {
  if (!n_limbs || !n_ops) return;
  const Lift lf = lift ? *lift : Lift{PolySeq{{nullptr, nullptr}, 0}, nullptr, 0, nullptr, nullptr, nullptr, nullptr, 0};
  if (dotprod_reads_own(keys.n, n_ops, out1 != nullptr, n_parts)) {
    const OwnLimbs ol = own ? *own : OwnLimbs{nullptr, 0, 1, 0, 0};
    // NP <= 4 products of residues below 2^61 fit 128 bits without an intermediate reduction
    const u32 blocks_x = (u32)((c.N + kThreads * kKeyUnroll - 1) / (kThreads * kKeyUnroll));
    const u32 split = n_ops < kSharedKeySplit ? n_ops : kSharedKeySplit;
    dim3 g(((blocks_x * n_limbs + 7) / 8) * 8 * split);
#define ACE_DP_CASE(NP)                                                                                          \
  case NP:                                                                                                       \
    hipLaunchKernelGGL(dotprod_shared_key_kernel<NP>, g, dim3(kThreads), 0, st, c, out0, out1, out_stride,       \
                       digits, digit_stride, digits_op_stride, keys.p[0], key1_off, key_stride, lm, key_limb,    \
                       n_ops, ol, lf, blocks_x, n_limbs, split);                                                 \
    break;
    switch (n_parts) { ACE_DP_CASE(1) ACE_DP_CASE(2) ACE_DP_CASE(3) ACE_DP_CASE(4) }
#undef ACE_DP_CASE
    return;
  }
  if (!lift && keys.n == n_ops && n_ops > 1 && digits_op_stride == 0 && out1 && n_parts >= 1 && n_parts <= 4) {
    const u32 blocks_x = (u32)((c.N + kThreads * kDigitsUnroll - 1) / (kThreads * kDigitsUnroll));
    const u32 split = n_ops < kSharedDigitsSplit ? n_ops : kSharedDigitsSplit;
    dim3 g(((blocks_x * n_limbs + 7) / 8) * 8 * split);
#define ACE_DP_CASE(NP)                                                                                          \
  case NP:                                                                                                       \
    hipLaunchKernelGGL(dotprod_shared_digits_kernel<NP>, g, dim3(kThreads), 0, st, c, out0, out1, out_stride,    \
                       digits, digit_stride, keys, key1_off, key_stride, lm, key_limb, n_ops, blocks_x, n_limbs, \
                       split);                                                                                   \
    break;
    switch (n_parts) { ACE_DP_CASE(1) ACE_DP_CASE(2) ACE_DP_CASE(3) ACE_DP_CASE(4) }
#undef ACE_DP_CASE
    return;
  }
  dim3 g = ew_grid(c.N, n_limbs, n_ops);
  if (out1)
    hipLaunchKernelGGL(dotprod_kernel<true>, g, dim3(kThreads), 0, st, c, out0, out1, out_stride, digits,
                       digit_stride, digits_op_stride, keys, key1_off, key_stride, n_parts, lm, key_limb, lf);
  else
    hipLaunchKernelGGL(dotprod_kernel<false>, g, dim3(kThreads), 0, st, c, out0, out1, out_stride, digits,
                       digit_stride, digits_op_stride, keys, key1_off, key_stride, n_parts, lm, key_limb, lf);
}

// ---- Mod_down tail (rns_poly.c:292-303): (src - y) * P^-1 [+ addend] --------
// blockIdx.z = polynomial; src/out/addend are addressed as PolySeq.  With index
// tables (orders.n != 0) the automorphism that ends a rotation is applied on the
// way out: out[i] = value at order[i] (polynomials 2r and 2r+1 use table r),
// negative entries as in gather_kernel.
__global__ __launch_bounds__(kThreads) void moddown_tail_kernel(DevCtx c, PolySeq outs, PolySeq srcs,
                                                                const u64* __restrict__ y_base, u64 y_stride,
                                                                PolySeq addends, int addend_mode,
                                                                const u64* __restrict__ cst, LimbMap lm,
                                                                OrderSet orders) {
  const u32 limb = blockIdx.y, p = blockIdx.z;
  const u64 q = c.primes[lm.prime[limb]].q;
  const u64 w = cst[2 * limb], wp = cst[2 * limb + 1];
  const u64 n = c.N, base = (u64)limb * n;
  u64* out = outs.at(p);  // may be the addend itself (in-place relinearisation): no restrict
  const u64* __restrict__ src = srcs.at(p);
  const u64* __restrict__ y = y_base + p * y_stride;
  // addend_mode: 0 none, 1 every polynomial, 2 even polynomials only
  const u64* addend = (addend_mode == 1 || (addend_mode == 2 && !(p & 1))) ? addends.at(p) : nullptr;
  const i64* __restrict__ order = orders.n ? orders.p[orders.n == 1 ? 0 : (p >> 1)] : nullptr;
#pragma unroll
  ACE_EW_LOOP(i, n) {
    i64 k = order ? order[i] : (i64)i;
    u64 j = base + (u64)(k < 0 ? -k : k);
    u64 v = shoup_mul(sub_mod(src[j], y[j], q), w, wp, q);
    if (addend) v = add_mod(v, addend[j], q);
    out[base + i] = k < 0 ? q - v : v;
  }
}

void launch_moddown_tail(hipStream_t st, const DevCtx& c, const PolySeq& out, const PolySeq& src, const u64* y,
                         u64 y_stride, const PolySeq* addend, int addend_mode, const u64* cst, const LimbMap& lm,
                         u32 n_limbs, u32 n_polys, const OrderSet* orders) {
  if (!n_limbs || !n_polys) return;
  PolySeq ad = addend ? *addend : out;
  OrderSet os{};
  if (orders) os = *orders;
  hipLaunchKernelGGL(moddown_tail_kernel, ew_grid(c.N, n_limbs, n_polys), dim3(kThreads), 0, st, c, out, src, y,
                     y_stride, ad, addend ? addend_mode : 0, cst, lm, os);
}

// ---- Rescale (rns_poly.c:310-404) ------------------------------------------
// Switch_modulus (include/util/modular.h:296-322): centred lift q_l -> q_t.
// cst per limb: K, K' (Shoup), diff = q_t - (q_l mod q_t)
__global__ __launch_bounds__(kThreads) void rescale_switch_kernel(DevCtx c, u64* __restrict__ u_base, u64 u_stride,
                                                                  const u64* __restrict__ last_base, u64 last_stride,
                                                                  u32 last_prime, const u64* __restrict__ cst,
                                                                  LimbMap lm) {
  const u32 limb = blockIdx.y, p = blockIdx.z;
  const DevPrime P = c.primes[lm.prime[limb]];
  const u64 ql = c.primes[last_prime].q, half = ql >> 1;
  const u64 K = cst[3 * limb], Kp = cst[3 * limb + 1], diff = cst[3 * limb + 2];
  const u64 n = c.N, base = (u64)limb * n;
  u64* __restrict__ u = u_base + p * u_stride;
  const u64* __restrict__ last = last_base + p * last_stride;
#pragma unroll
  ACE_EW_LOOP(i, n) {
    u64 v = last[i];
    if (P.q > ql) {
      if (v > half) v += P.q - ql;
    } else {
      if (v > half) v += diff;
      if (v >= P.q) v = barrett128(0, v, P);
    }
    u[base + i] = shoup_mul(v, K, Kp, P.q);
  }
}
void launch_rescale_switch(hipStream_t st, const DevCtx& c, u64* u, u64 u_stride, const u64* last, u64 last_stride,
                           u32 last_prime, const u64* cst, const LimbMap& lm, u32 n_limbs, u32 n_polys) {
  if (!n_limbs || !n_polys) return;
  hipLaunchKernelGGL(rescale_switch_kernel, ew_grid(c.N, n_limbs, n_polys), dim3(kThreads), 0, st, c, u, u_stride,
                     last, last_stride, last_prime, cst, lm);
}

__global__ __launch_bounds__(kThreads) void rescale_tail_kernel(DevCtx c, PolySeq outs, PolySeq srcs,
                                                                const u64* __restrict__ u_base, u64 u_stride,
                                                                const u64* __restrict__ cst, LimbMap lm) {
  const u32 limb = blockIdx.y, p = blockIdx.z;
  const u64 q = c.primes[lm.prime[limb]].q;
  const u64 w = cst[2 * limb], wp = cst[2 * limb + 1];
  const u64 n = c.N, base = (u64)limb * n;
  u64* __restrict__ out = outs.at(p);
  const u64* __restrict__ src = srcs.at(p);
  const u64* __restrict__ u = u_base + p * u_stride;
#pragma unroll
  ACE_EW_LOOP(i, n) out[base + i] = add_mod(shoup_mul(src[base + i], w, wp, q), u[base + i], q);
}
void launch_rescale_tail(hipStream_t st, const DevCtx& c, const PolySeq& out, const PolySeq& src, const u64* u,
                         u64 u_stride, const u64* cst, const LimbMap& lm, u32 n_limbs, u32 n_polys) {
  if (!n_limbs || !n_polys) return;
  hipLaunchKernelGGL(rescale_tail_kernel, ew_grid(c.N, n_limbs, n_polys), dim3(kThreads), 0, st, c, out, src, u,
                     u_stride, cst, lm);
}

// coefficient form (rns_poly.c:380-400): plain residue of the last limb
__global__ __launch_bounds__(kThreads) void rescale_coef_kernel(DevCtx c, u64* __restrict__ out,
                                                                const u64* __restrict__ src,
                                                                const u64* __restrict__ last,
                                                                const u64* __restrict__ cst, LimbMap lm) {
  const u32 limb = blockIdx.y;
  const DevPrime P = c.primes[lm.prime[limb]];
  const u64 w = cst[2 * limb], wp = cst[2 * limb + 1];
  const u64 n = c.N, base = (u64)limb * n;
#pragma unroll
  ACE_EW_LOOP(i, n) {
    u64 lc = barrett128(0, last[i], P);
    out[base + i] = shoup_mul(sub_mod(src[base + i], lc, P.q), w, wp, P.q);
  }
}
void launch_rescale_coef(hipStream_t st, const DevCtx& c, u64* out, const u64* src, const u64* last,
                         const u64* cst, const LimbMap& lm, u32 n_limbs) {
  if (!n_limbs) return;
  hipLaunchKernelGGL(rescale_coef_kernel, ew_grid(c.N, n_limbs), dim3(kThreads), 0, st, c, out, src, last, cst, lm);
}

// ---- Mod_down_rescale / Reduce_and_rescale_modup tail (rns_poly.c:555-590,
// rns_poly_impl.c:549-607), coefficient form ---------------------------------
// y holds the P part converted to the Q basis (level limbs).  For limb i < level-1:
//   last = (poly_last - y_last) * P^-1 mod q_last
//   out_i = (((poly_i - y_i) * P^-1 mod q_i) - last) * q_last^-1 mod q_i
// with Sub_mul_const_mod's exact semantics.  When last_out is given, the blocks of
// limb 0 also store `last` there; it must not alias y (every block reads y_last).
// pinv / qlinv: (constant, Shoup) pairs per limb.
__global__ __launch_bounds__(kThreads) void moddown_rescale_kernel(DevCtx c, u64* __restrict__ out,
                                                                   const u64* __restrict__ poly,
                                                                   const u64* __restrict__ y,
                                                                   u64* __restrict__ last_out,
                                                                   const u64* __restrict__ pinv,
                                                                   const u64* __restrict__ qlinv, u32 level) {
  const u32 limb = blockIdx.y, last = level - 1;
  const u64 q = c.primes[limb].q, ql = c.primes[last].q;
  const u64 w = pinv[2 * limb], wp = pinv[2 * limb + 1], wl = pinv[2 * last], wlp = pinv[2 * last + 1];
  const u64 v = qlinv[2 * limb], vp = qlinv[2 * limb + 1];
  const u64 n = c.N, base = (u64)limb * n, lbase = (u64)last * n;
#pragma unroll
  ACE_EW_LOOP(i, n) {
    u64 lastv = sub_mul_const(poly[lbase + i], y[lbase + i], wl, wlp, ql);
    u64 t = sub_mul_const(poly[base + i], y[base + i], w, wp, q);
    out[base + i] = sub_mul_const(t, lastv, v, vp, q);
    if (last_out && limb == 0) last_out[i] = lastv;
  }
}
void launch_moddown_rescale(hipStream_t st, const DevCtx& c, u64* out, const u64* poly, const u64* y, u64* last_out,
                            const u64* pinv, const u64* qlinv, u32 level) {
  if (level < 2) return;
  hipLaunchKernelGGL(moddown_rescale_kernel, ew_grid(c.N, level - 1), dim3(kThreads), 0, st, c, out, poly, y,
                     last_out, pinv, qlinv, level);
}

// ---- Transform_values_from_level0 (rns_poly.c:1101-1125) ---------------------
// out limb 0 = src; out limb i = Switch_modulus(src, q_0 -> q_i) (modular.h:296-322)
__global__ __launch_bounds__(kThreads) void from_level0_kernel(DevCtx c, u64* __restrict__ out,
                                                               const u64* __restrict__ src) {
  const u32 limb = blockIdx.y;
  const DevPrime P = c.primes[limb];
  const u64 q0 = c.primes[0].q, half = q0 >> 1;
  const u64 n = c.N, base = (u64)limb * n;
#pragma unroll
  ACE_EW_LOOP(i, n) {
    u64 v = src[i];
    if (limb != 0) {
      if (P.q > q0) {
        if (v > half) v += P.q - q0;
      } else {
        if (v > half) v += P.q - (q0 % P.q);
        if (v >= P.q) v = barrett128(0, v, P);
      }
    }
    out[base + i] = v;
  }
}
void launch_from_level0(hipStream_t st, const DevCtx& c, u64* out, const u64* src, u32 level) {
  if (!level) return;
  hipLaunchKernelGGL(from_level0_kernel, ew_grid(c.N, level), dim3(kThreads), 0, st, c, out, src);
}

// ---- multiply every limb by its own constant (Extend, rns_poly.c:483-500) ---
__global__ __launch_bounds__(kThreads) void mul_const_kernel(DevCtx c, u64* __restrict__ out,
                                                             const u64* __restrict__ src,
                                                             const u64* __restrict__ cst, LimbMap lm) {
  const u32 limb = blockIdx.y;
  const u64 q = c.primes[lm.prime[limb]].q;
  const u64 w = cst[2 * limb], wp = cst[2 * limb + 1];
  const u64 n = c.N, base = (u64)limb * n;
#pragma unroll
  ACE_EW_LOOP(i, n) out[base + i] = shoup_mul(src[base + i], w, wp, q);
}
void launch_mul_const(hipStream_t st, const DevCtx& c, u64* out, const u64* src, const u64* cst, const LimbMap& lm,
                      u32 n_limbs) {
  if (!n_limbs) return;
  hipLaunchKernelGGL(mul_const_kernel, ew_grid(c.N, n_limbs), dim3(kThreads), 0, st, c, out, src, cst, lm);
}

__global__ __launch_bounds__(kThreads) void fill_zero_kernel(u64* __restrict__ p, u64 n) {
  for (u64 i = (u64)blockIdx.x * kThreads + threadIdx.x; i < n; i += (u64)gridDim.x * kThreads) p[i] = 0;
}
void launch_fill_zero(hipStream_t st, u64* p, u64 n) {
  if (!n) return;
  u64 blocks = (n + kThreads - 1) / kThreads;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, st, p, n);
}

}  // namespace ace
