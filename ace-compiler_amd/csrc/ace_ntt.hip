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
//            chunk per workgroup: 256 threads x 16 registers, three rounds of
//            four stages with two LDS transposes (LDS index padded by e>>4 so
//            the 16-word-strided accesses are conflict-free), and a last
//            transpose so the global store is coalesced.
//   inverse  the same two kernels mirrored (chunk first, strided last).
// Inside a kernel values are kept lazily reduced (forward < 4q, inverse < 2q,
// Harvey butterflies); the last kernel of a transform stores canonical
// residues.  N <= 4096 uses one workgroup per limb with the limb in LDS.
#include "ace_kernels.h"

namespace ace {

constexpr int kChunk = 4096;
constexpr int kLogChunk = 12;

__device__ __forceinline__ int lds_pos(int e) { return e + (e >> 4); }

// forward butterfly, Harvey: x,y < 4q -> x' , y' < 4q
__device__ __forceinline__ void ct_bfly(u64& x, u64& y, u64 w, u64 wp, u64 q, u64 q2) {
  u64 a = csub(x, q2);
  u64 t = shoup_lazy(y, w, wp, q);
  x = a + t;
  y = a - t + q2;
}
// inverse butterfly: x,y < 2q -> x', y' < 2q
__device__ __forceinline__ void gs_bfly(u64& x, u64& y, u64 w, u64 wp, u64 q, u64 q2) {
  u64 s = csub(x + y, q2);
  u64 d = x - y + q2;
  x = s;
  y = shoup_lazy(d, w, wp, q);
}

// ---------------------------------------------------------------------------
// forward, strided pass: stages 0..LOGR-1
// grid = (N/R/256, n_limbs, n_polys)
template <int LOGR>
__global__ __launch_bounds__(256) void ntt_fwd_strided(DevCtx c, u64* __restrict__ dst, const u64* __restrict__ src,
                                                       LimbMap lm, LimbMap pos, u64 poly_stride) {
  constexpr int R = 1 << LOGR;
  const u32 col = blockIdx.x * 256 + threadIdx.x;
  const u32 limb = blockIdx.y, pi = lm.prime[limb];
  const u64 rs = c.N >> LOGR;  // row stride
  const u64 off = blockIdx.z * poly_stride + (u64)pos.prime[limb] * c.N + col;
  const u64 q = c.primes[pi].q, q2 = q << 1;
  const u64* w = c.rou + (u64)pi * c.N;
  const u64* wp = c.rou_p + (u64)pi * c.N;
  u64 v[R];
#pragma unroll
  for (int r = 0; r < R; ++r) v[r] = src[off + r * rs];
#pragma unroll
  for (int ls = 0; ls < LOGR; ++ls) {
    const int half = R >> (ls + 1);
#pragma unroll
    for (int g = 0; g < (1 << ls); ++g) {
      u64 W = w[(1 << ls) + g], Wp = wp[(1 << ls) + g];
#pragma unroll
      for (int j = 0; j < half; ++j) ct_bfly(v[g * 2 * half + j], v[g * 2 * half + j + half], W, Wp, q, q2);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) dst[off + r * rs] = v[r];
}

// forward, chunk pass: stages logr..logN-1 on 4096 contiguous words.
// grid = (N/4096, n_limbs, n_polys); in place on `data`, or src -> data when
// logr == 0 is impossible here (N > 4096 always has a strided pass first).
__global__ __launch_bounds__(256) void ntt_fwd_chunk(DevCtx c, u64* __restrict__ data, LimbMap lm, LimbMap pos, u64 poly_stride,
                                                     u32 logr) {
  __shared__ u64 lds[kChunk + kChunk / 16];
  const int t = threadIdx.x;
  const u32 chunk = blockIdx.x, limb = blockIdx.y, pi = lm.prime[limb];
  u64* base = data + blockIdx.z * poly_stride + (u64)pos.prime[limb] * c.N + (u64)chunk * kChunk;
  const u64 q = c.primes[pi].q, q2 = q << 1;
  const u64* w = c.rou + (u64)pi * c.N;
  const u64* wp = c.rou_p + (u64)pi * c.N;
  u64 v[16];
  // round A: element e = t + 256 r, local stages 0..3; twiddles are uniform
#pragma unroll
  for (int r = 0; r < 16; ++r) v[r] = base[t + 256 * r];
#pragma unroll
  for (int ls = 0; ls < 4; ++ls) {
    const int half = 8 >> ls;
    const u32 m = 1u << (logr + ls);
#pragma unroll
    for (int g = 0; g < (1 << ls); ++g) {
      u32 ti = m + (chunk << ls) + g;
      u64 W = w[ti], Wp = wp[ti];
#pragma unroll
      for (int j = 0; j < half; ++j) ct_bfly(v[g * 2 * half + j], v[g * 2 * half + j + half], W, Wp, q, q2);
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) lds[lds_pos(t + 256 * r)] = v[r];
  __syncthreads();
  // round B: e = hi*256 + r*16 + lo, local stages 4..7
  const int hi = t >> 4, lo = t & 15;
#pragma unroll
  for (int r = 0; r < 16; ++r) v[r] = lds[lds_pos(hi * 256 + r * 16 + lo)];
#pragma unroll
  for (int ls = 4; ls < 8; ++ls) {
    const int half = 8 >> (ls - 4);
    const u32 m = 1u << (logr + ls);
#pragma unroll
    for (int g = 0; g < (1 << (ls - 4)); ++g) {
      u32 ti = m + (chunk << ls) + (hi << (ls - 4)) + g;
      u64 W = w[ti], Wp = wp[ti];
#pragma unroll
      for (int j = 0; j < half; ++j) ct_bfly(v[g * 2 * half + j], v[g * 2 * half + j + half], W, Wp, q, q2);
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) lds[lds_pos(hi * 256 + r * 16 + lo)] = v[r];
  __syncthreads();
  // round C: e = t*16 + r, local stages 8..11
#pragma unroll
  for (int r = 0; r < 16; ++r) v[r] = lds[lds_pos(t * 16 + r)];
#pragma unroll
  for (int ls = 8; ls < 12; ++ls) {
    const int half = 8 >> (ls - 8);
    const u32 m = 1u << (logr + ls);
#pragma unroll
    for (int g = 0; g < (1 << (ls - 8)); ++g) {
      u32 ti = m + (chunk << ls) + (t << (ls - 8)) + g;
      u64 W = w[ti], Wp = wp[ti];
#pragma unroll
      for (int j = 0; j < half; ++j) ct_bfly(v[g * 2 * half + j], v[g * 2 * half + j + half], W, Wp, q, q2);
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) lds[lds_pos(t * 16 + r)] = csub(csub(v[r], q2), q);
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 16; ++r) base[t + 256 * r] = lds[lds_pos(t + 256 * r)];
}

// ---------------------------------------------------------------------------
// inverse, chunk pass: spans 1..2048 on 4096 contiguous words; src -> dst.
// Nothing is scaled here: 1/N (times an optional per-limb constant) is applied
// by the strided pass that always follows.
__global__ __launch_bounds__(256) void ntt_inv_chunk(DevCtx c, u64* __restrict__ dst, const u64* __restrict__ src,
                                                     LimbMap lm, LimbMap pos, u64 poly_stride) {
  __shared__ u64 lds[kChunk + kChunk / 16];
  const int t = threadIdx.x;
  const u32 chunk = blockIdx.x, limb = blockIdx.y, pi = lm.prime[limb];
  const u64 off = blockIdx.z * poly_stride + (u64)pos.prime[limb] * c.N + (u64)chunk * kChunk;
  const u64 q = c.primes[pi].q, q2 = q << 1;
  const u64* w = c.irou + (u64)pi * c.N;
  const u64* wp = c.irou_p + (u64)pi * c.N;
  const u32 logN = c.logN;
  u64 v[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) lds[lds_pos(t + 256 * r)] = src[off + t + 256 * r];
  __syncthreads();
  // round C': e = t*16 + r, spans 2^u, u = 0..3
#pragma unroll
  for (int r = 0; r < 16; ++r) v[r] = lds[lds_pos(t * 16 + r)];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int span = 1 << u;
    const u32 m = 1u << (logN - u - 1);
#pragma unroll
    for (int g = 0; g < (8 >> u); ++g) {
      u32 ti = m + (chunk << (11 - u)) + (t << (3 - u)) + g;
      u64 W = w[ti], Wp = wp[ti];
#pragma unroll
      for (int j = 0; j < span; ++j) gs_bfly(v[g * 2 * span + j], v[g * 2 * span + j + span], W, Wp, q, q2);
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) lds[lds_pos(t * 16 + r)] = v[r];
  __syncthreads();
  // round B': e = hi*256 + r*16 + lo, u = 4..7
  const int hi = t >> 4, lo = t & 15;
#pragma unroll
  for (int r = 0; r < 16; ++r) v[r] = lds[lds_pos(hi * 256 + r * 16 + lo)];
#pragma unroll
  for (int u = 4; u < 8; ++u) {
    const int span = 1 << (u - 4);
    const u32 m = 1u << (logN - u - 1);
#pragma unroll
    for (int g = 0; g < (8 >> (u - 4)); ++g) {
      u32 ti = m + (chunk << (11 - u)) + (hi << (7 - u)) + g;
      u64 W = w[ti], Wp = wp[ti];
#pragma unroll
      for (int j = 0; j < span; ++j) gs_bfly(v[g * 2 * span + j], v[g * 2 * span + j + span], W, Wp, q, q2);
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) lds[lds_pos(hi * 256 + r * 16 + lo)] = v[r];
  __syncthreads();
  // round A': e = t + 256 r, u = 8..11; twiddles uniform
#pragma unroll
  for (int r = 0; r < 16; ++r) v[r] = lds[lds_pos(t + 256 * r)];
#pragma unroll
  for (int u = 8; u < 12; ++u) {
    const int span = 1 << (u - 8);
    const u32 m = 1u << (logN - u - 1);
#pragma unroll
    for (int g = 0; g < (8 >> (u - 8)); ++g) {
      u32 ti = m + (chunk << (11 - u)) + g;
      u64 W = w[ti], Wp = wp[ti];
#pragma unroll
      for (int j = 0; j < span; ++j) gs_bfly(v[g * 2 * span + j], v[g * 2 * span + j + span], W, Wp, q, q2);
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) dst[off + t + 256 * r] = v[r];
}

// inverse, strided pass: spans 4096..N/2, then scale every word by
// scale[limb] (default 1/N) and store canonical residues.  In place.
// scale: nullptr or 2*n_limbs words (constant, Shoup companion) per limb.
template <int LOGR>
__global__ __launch_bounds__(256) void ntt_inv_strided(DevCtx c, u64* __restrict__ data, LimbMap lm, LimbMap pos, u64 poly_stride,
                                                       const u64* __restrict__ scale) {
  constexpr int R = 1 << LOGR;
  const u32 col = blockIdx.x * 256 + threadIdx.x;
  const u32 limb = blockIdx.y, pi = lm.prime[limb];
  const u64 rs = c.N >> LOGR;
  const u64 off = blockIdx.z * poly_stride + (u64)pos.prime[limb] * c.N + col;
  const DevPrime P = c.primes[pi];
  const u64 q = P.q, q2 = q << 1;
  const u64* w = c.irou + (u64)pi * c.N;
  const u64* wp = c.irou_p + (u64)pi * c.N;
  u64 v[R];
#pragma unroll
  for (int r = 0; r < R; ++r) v[r] = data[off + r * rs];
#pragma unroll
  for (int u = 0; u < LOGR; ++u) {  // span 2^u rows, m = R >> (u+1) groups
    const int span = 1 << u;
#pragma unroll
    for (int g = 0; g < (R >> (u + 1)); ++g) {
      u64 W = w[(R >> (u + 1)) + g], Wp = wp[(R >> (u + 1)) + g];
#pragma unroll
      for (int j = 0; j < span; ++j) gs_bfly(v[g * 2 * span + j], v[g * 2 * span + j + span], W, Wp, q, q2);
    }
  }
  u64 s = P.ninv, sp = P.ninv_p;
  if (scale) { s = scale[2 * limb]; sp = scale[2 * limb + 1]; }
#pragma unroll
  for (int r = 0; r < R; ++r) data[off + r * rs] = shoup_mul(v[r], s, sp, q);
}

// ---------------------------------------------------------------------------
// N <= 4096: one workgroup per limb, the limb in LDS, one butterfly per
// thread per step.  grid = (1, n_limbs, n_polys)
__global__ __launch_bounds__(256) void ntt_small(DevCtx c, u64* __restrict__ dst, const u64* __restrict__ src,
                                                 LimbMap lm, LimbMap pos, u64 poly_stride, int inverse,
                                                 const u64* __restrict__ scale) {
  __shared__ u64 a[kChunk];
  const u32 N = c.N, logN = c.logN, limb = blockIdx.y, pi = lm.prime[limb];
  const u64 off = blockIdx.z * poly_stride + (u64)pos.prime[limb] * N;
  const DevPrime P = c.primes[pi];
  const u64 q = P.q, q2 = q << 1;
  for (u32 i = threadIdx.x; i < N; i += 256) a[i] = src[off + i];
  __syncthreads();
  if (!inverse) {
    const u64* w = c.rou + (u64)pi * N;
    const u64* wp = c.rou_p + (u64)pi * N;
    for (u32 s = 0; s < logN; ++s) {
      const u32 tspan = N >> (s + 1);
      for (u32 b = threadIdx.x; b < (N >> 1); b += 256) {
        u32 g = b / tspan, j = b - g * tspan, i0 = g * 2 * tspan + j;
        ct_bfly(a[i0], a[i0 + tspan], w[(1u << s) + g], wp[(1u << s) + g], q, q2);
      }
      __syncthreads();
    }
    for (u32 i = threadIdx.x; i < N; i += 256) dst[off + i] = csub(csub(a[i], q2), q);
  } else {
    const u64* w = c.irou + (u64)pi * N;
    const u64* wp = c.irou_p + (u64)pi * N;
    for (u32 u = 0; u < logN; ++u) {
      const u32 span = 1u << u, m = N >> (u + 1);
      for (u32 b = threadIdx.x; b < (N >> 1); b += 256) {
        u32 g = b >> u, j = b & (span - 1), i0 = g * 2 * span + j;
        gs_bfly(a[i0], a[i0 + span], w[m + g], wp[m + g], q, q2);
      }
      __syncthreads();
    }
    u64 s = P.ninv, sp = P.ninv_p;
    if (scale) { s = scale[2 * limb]; sp = scale[2 * limb + 1]; }
    for (u32 i = threadIdx.x; i < N; i += 256) dst[off + i] = shoup_mul(a[i], s, sp, q);
  }
}

// ---------------------------------------------------------------------------
template <int LOGR>
static void fwd_large(hipStream_t st, const DevCtx& c, u64* dst, const u64* src, const LimbMap& lm, const LimbMap& pos,
                      u32 n_limbs, u32 n_polys, u64 poly_stride) {
  dim3 g1((c.N >> LOGR) / 256, n_limbs, n_polys), g2(c.N / kChunk, n_limbs, n_polys);
  hipLaunchKernelGGL(ntt_fwd_strided<LOGR>, g1, dim3(256), 0, st, c, dst, src, lm, pos, poly_stride);
  hipLaunchKernelGGL(ntt_fwd_chunk, g2, dim3(256), 0, st, c, dst, lm, pos, poly_stride, (u32)LOGR);
}
template <int LOGR>
static void inv_large(hipStream_t st, const DevCtx& c, u64* dst, const u64* src, const LimbMap& lm, const LimbMap& pos,
                      u32 n_limbs, u32 n_polys, u64 poly_stride, const u64* scale) {
  dim3 g1(c.N / kChunk, n_limbs, n_polys), g2((c.N >> LOGR) / 256, n_limbs, n_polys);
  hipLaunchKernelGGL(ntt_inv_chunk, g1, dim3(256), 0, st, c, dst, src, lm, pos, poly_stride);
  hipLaunchKernelGGL(ntt_inv_strided<LOGR>, g2, dim3(256), 0, st, c, dst, lm, pos, poly_stride, scale);
}

bool launch_ntt(hipStream_t st, const DevCtx& c, u64* dst, const u64* src, const LimbMap& lm, const LimbMap* pos_in,
                u32 n_limbs, u32 n_polys, u64 poly_stride, bool inverse, const u64* scale) {
  if (n_limbs == 0 || n_polys == 0) return true;
  LimbMap pos{};
  if (pos_in) pos = *pos_in;
  else
    for (u32 t = 0; t < n_limbs; ++t) pos.prime[t] = (uint8_t)t;
  if (c.logN <= kLogChunk) {
    hipLaunchKernelGGL(ntt_small, dim3(1, n_limbs, n_polys), dim3(256), 0, st, c, dst, src, lm, pos,
                       poly_stride, inverse ? 1 : 0, scale);
    return true;
  }
  switch (c.logN - kLogChunk) {
#define ACE_NTT_CASE(LR)                                                                  \
  case LR:                                                                                \
    if (inverse) inv_large<LR>(st, c, dst, src, lm, pos, n_limbs, n_polys, poly_stride, scale); \
    else         fwd_large<LR>(st, c, dst, src, lm, pos, n_limbs, n_polys, poly_stride);        \
    return true;
    ACE_NTT_CASE(1)
    ACE_NTT_CASE(2)
    ACE_NTT_CASE(3)
    ACE_NTT_CASE(4)
    ACE_NTT_CASE(5)
#undef ACE_NTT_CASE
    default:
      return false;  // ring degree above 2^17 not supported
  }
}

}  // namespace ace
