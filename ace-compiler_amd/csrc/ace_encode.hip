// CKKS encoder on the device (Encode_impl, ckks/src/encoder.c:234-326): inverse
// canonical embedding (Embedding_inv, util/src/ntt.c:631-675) in FP64, scaling,
// rounding, and the split into RNS residues.  Every floating-point step is the
// reference's operation in the reference's order with contraction off, so the
// rounded integers -- and with them every residue -- are the same bits.
#include "ace_kernels.h"

namespace ace {

constexpr int kEncThreads = 256;

// stages logm_hi .. logm_lo of Embedding_inv in one launch: a work-group keeps a tile of up to 2048 elements in
// LDS -- all 2^S values of the S index bits the stages pair up (bits logm_lo-1 .. logm_hi-1), times W consecutive
// values of the bits below them -- and runs the stages on it with a barrier in between.  Stage logm pairs elements (j+i, j+i+2^(logm-1)) of
// every block j of 2^logm elements with the twiddle of rot[i]; running the stages in the reference's order on each
// butterfly keeps the result the same bits however the butterflies are grouped.
constexpr u32 kTileLog = 11;
constexpr int kTileThreads = 1024;  // one butterfly per thread and stage on a full tile: the stages are latency-bound
__global__ __launch_bounds__(kTileThreads) void embed_inv_tile_kernel(double2* __restrict__ r,
                                                                     const double2* __restrict__ rou,
                                                                     const u32* __restrict__ rot, u32 M, u32 logm_hi,
                                                                     u32 logm_lo, u32 log_w) {
#pragma clang fp contract(off)
  __shared__ double2 tile[1u << kTileLog];
  const u32 S = logm_hi - logm_lo + 1, low_bits = logm_lo - 1;  // low_bits index bits lie below the paired ones
  const u32 tile_elems = 1u << (S + log_w);
  // blockIdx.x enumerates (high part, group of W low values)
  const u32 groups_lo = 1u << (low_bits - log_w);
  const u32 g_lo0 = (blockIdx.x & (groups_lo - 1)) << log_w, g_hi = blockIdx.x >> (low_bits - log_w);
  auto global_of = [&](u32 local) {
    const u32 w = local & ((1u << log_w) - 1), k = local >> log_w;
    return (g_hi << logm_hi) | (k << low_bits) | (g_lo0 + w);
  };
  for (u32 e = threadIdx.x; e < tile_elems; e += blockDim.x) tile[e] = r[global_of(e)];
  __syncthreads();
  for (u32 logm = logm_hi; logm >= logm_lo; --logm) {
    const u32 bitpos = log_w + (logm - logm_lo);
    const u32 num2 = 1u << (logm - 1), idx_mod = 1u << (logm + 2), gap = M / idx_mod;
    for (u32 t = threadIdx.x; t < (tile_elems >> 1); t += blockDim.x) {
      const u32 lo = t & ((1u << bitpos) - 1), le = ((t >> bitpos) << (bitpos + 1)) | lo, lodd = le | (1u << bitpos);
      const u32 i = global_of(le) & (num2 - 1);
      const u32 rou_idx = (idx_mod - (rot[i] & (idx_mod - 1))) * gap;
      const double2 x = tile[le], y = tile[lodd], w = rou[rou_idx];
      const double pr = x.x + y.x, pi = x.y + y.y, mr = x.x - y.x, mi = x.y - y.y;
      const double qr = mr * w.x - mi * w.y, qi = mr * w.y + mi * w.x;
      tile[le] = make_double2(pr, pi);
      tile[lodd] = make_double2(qr, qi);
    }
    __syncthreads();
    if (logm == logm_lo) break;  // unsigned loop variable
  }
  for (u32 e = threadIdx.x; e < tile_elems; e += blockDim.x) r[global_of(e)] = tile[e];
}

// all stages of Embedding_inv over `len` elements: the top stages in tiles of strided runs, then the rest
static void launch_embed_inv_stages(hipStream_t st, double2* r, const double2* rou, const u32* rot, u32 M, u32 len) {
  u32 loglen = 0;
  while ((1u << loglen) < len) ++loglen;
  u32 hi = loglen;
  const u32 tile = 1u << (loglen < kTileLog ? loglen : kTileLog), half = tile >> 1;
  const u32 threads = half >= (u32)kTileThreads ? (u32)kTileThreads : (half < 64 ? 64 : half);
  while (hi > kTileLog) {  // stages hi .. lo on tiles of 2^S x W elements, W >= 16 for coalesced runs
    const u32 S = (hi - kTileLog) < 7 ? (hi - kTileLog) : 7, lo = hi - S + 1, log_w = kTileLog - S;
    hipLaunchKernelGGL(embed_inv_tile_kernel, dim3(len >> kTileLog), dim3(threads), 0, st, r, rou, rot, M, hi, lo,
                       log_w);
    hi = lo - 1;
  }
  if (hi >= 1) {
    const u32 tile_log = hi;  // hi <= kTileLog: stages hi .. 1 on tiles of 2^hi consecutive elements
    hipLaunchKernelGGL(embed_inv_tile_kernel, dim3(len >> tile_log), dim3(threads), 0, st, r, rou, rot, M, hi, 1u,
                       0u);
  }
}

// Max_64bit_value (include/util/modular.h:279-281)
__device__ __forceinline__ i64 max_64bit_value() { return (i64)(((u64)1 << 63) - ((u64)1 << 9)) - 1; }
__device__ __forceinline__ i64 mod_int64(i64 v, i64 m) {
  i64 r = v % m;
  return r < 0 ? r + m : r;
}

// bit reversal and 1/len of Embedding_inv, then encoder.c:268-291 and
// Transform_values_to_dcrt (util/src/crt.c:1153-1184): coefficient n of limb t.
// Slot i lands its real part at coefficient i*gap and its imaginary part at
// (i+slots)*gap; all other coefficients are zero.  err: set to 1 where the
// reference asserts (value out of range for the level, or not an int64).
__global__ __launch_bounds__(kEncThreads) void encode_round_kernel(DevCtx c, u64* __restrict__ out,
                                                                   const double2* __restrict__ r, u32 slots,
                                                                   u32 logslots, double scaling_factor, double scale,
                                                                   double round_add, double range_bound, LimbMap lm,
                                                                   int* err) {
#pragma clang fp contract(off)
  const u32 n = blockIdx.x * kEncThreads + threadIdx.x;
  if (n >= c.N) return;
  const u32 limb = blockIdx.y;
  const i64 q = (i64)c.primes[lm.prime[limb]].q;
  const u32 gap = c.N / (slots * 2);
  i64 res = 0;
  if (n % gap == 0) {
    u32 i = n / gap;
    const bool imag = i >= slots;
    if (imag) i -= slots;
    const u32 src = logslots ? (__brev(i) >> (32 - logslots)) : 0;
    const double2 z = r[src];
    const double v = (imag ? z.y : z.x) * (1.0 / (double)slots);  // slots is a power of two: exact, as the division is
    if (fabs(v * scale) >= range_bound) *err = 1;
    const double up = v * scaling_factor + round_add;  // 0.5 in Encode_impl, 0 in Encode_impl_with_scale
    if (!(up <= 9223372036854775807.0 && up >= -9223372036854775807.0)) {
      *err = 1;
    } else {
      const i64 m = llround(up);
      const i64 big = max_64bit_value();
      const i64 msg = m < 0 ? big + m : m;
      res = msg > (big >> 1) ? mod_int64(msg - (big - q), q) : mod_int64(msg, q);
    }
  }
  out[(u64)limb * c.N + n] = (u64)res;
}

// the inverse embedding alone: r (len complex values, overwritten) -> out[i] = r[bitrev(i)] / len
__global__ __launch_bounds__(kEncThreads) void embed_inv_finish_kernel(double2* __restrict__ out,
                                                                       const double2* __restrict__ r, u32 len,
                                                                       u32 loglen) {
  const u32 i = blockIdx.x * kEncThreads + threadIdx.x;
  if (i >= len) return;
  const double2 z = r[loglen ? (__brev(i) >> (32 - loglen)) : 0];
  const double inv = 1.0 / (double)len;
  out[i] = make_double2(z.x * inv, z.y * inv);
}
void launch_embedding_inv(hipStream_t st, const DevCtx& c, double2* out, double2* r, const double2* rou,
                          const u32* rot, u32 len) {
  u32 loglen = 0;
  while ((1u << loglen) < len) ++loglen;
  launch_embed_inv_stages(st, r, rou, rot, 2 * c.N, len);
  hipLaunchKernelGGL(embed_inv_finish_kernel, dim3((len + kEncThreads - 1) / kEncThreads), dim3(kEncThreads), 0, st,
                     out, r, len, loglen);
}

__global__ __launch_bounds__(256) void widen_real_kernel(double2* __restrict__ z, const void* __restrict__ raw,
                                                         int is_f32, u32 n_values, u32 slots) {
  const u32 i = blockIdx.x * 256 + threadIdx.x;
  if (i >= slots) return;
  double v = 0.0;
  if (i < n_values) v = is_f32 ? (double)static_cast<const float*>(raw)[i] : static_cast<const double*>(raw)[i];
  z[i] = make_double2(v, 0.0);
}
void launch_widen_real(hipStream_t st, double2* z, const void* raw, bool is_f32, u32 n_values, u32 slots) {
  hipLaunchKernelGGL(widen_real_kernel, dim3((slots + 255) / 256), dim3(256), 0, st, z, raw, is_f32 ? 1 : 0, n_values,
                     slots);
}

void launch_encode(hipStream_t st, const DevCtx& c, u64* out, double2* r, const double2* rou, const u32* rot,
                   u32 slots, double scaling_factor, double scale, double round_add, double range_bound,
                   const LimbMap& lm, u32 n_limbs, int* err) {
  u32 logslots = 0;
  while ((1u << logslots) < slots) ++logslots;
  launch_embed_inv_stages(st, r, rou, rot, 2 * c.N, slots);
  hipLaunchKernelGGL(encode_round_kernel, dim3((c.N + kEncThreads - 1) / kEncThreads, n_limbs), dim3(kEncThreads), 0,
                     st, c, out, r, slots, logslots, scaling_factor, scale, round_add, range_bound, lm, err);
}

}  // namespace ace
