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
                                                                     u32 logm_lo, u32 log_w, u32 len) {
#pragma clang fp contract(off)
  __shared__ double2 tile[1u << kTileLog];
  r += (u64)blockIdx.y * len;  // blockIdx.y: which of the vectors of a batch
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
static void launch_embed_inv_stages(hipStream_t st, double2* r, const double2* rou, const u32* rot, u32 M, u32 len,
                                    u32 n_vec = 1) {
  u32 loglen = 0;
  while ((1u << loglen) < len) ++loglen;
  u32 hi = loglen;
  const u32 tile = 1u << (loglen < kTileLog ? loglen : kTileLog), half = tile >> 1;
  const u32 threads = half >= (u32)kTileThreads ? (u32)kTileThreads : (half < 64 ? 64 : half);
  while (hi > kTileLog) {  // stages hi .. lo on tiles of 2^S x W elements, W >= 16 for coalesced runs
    const u32 S = (hi - kTileLog) < 7 ? (hi - kTileLog) : 7, lo = hi - S + 1, log_w = kTileLog - S;
    hipLaunchKernelGGL(embed_inv_tile_kernel, dim3(len >> kTileLog, n_vec), dim3(threads), 0, st, r, rou, rot, M, hi,
                       lo, log_w, len);
    hi = lo - 1;
  }
  if (hi >= 1) {
    const u32 tile_log = hi;  // hi <= kTileLog: stages hi .. 1 on tiles of 2^hi consecutive elements
    hipLaunchKernelGGL(embed_inv_tile_kernel, dim3(len >> tile_log, n_vec), dim3(threads), 0, st, r, rou, rot, M, hi,
                       1u, 0u, len);
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
                                                                   int* err, u64 out_stride) {
#pragma clang fp contract(off)
  const u32 n = blockIdx.x * kEncThreads + threadIdx.x;
  if (n >= c.N) return;
  out += blockIdx.z * out_stride;  // blockIdx.z: which of the vectors of a batch
  r += (u64)blockIdx.z * slots;
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
  const u64 at = (u64)blockIdx.y * n_values + i;  // blockIdx.y: which of the vectors of a batch, stored back to back
  double v = 0.0;
  if (i < n_values) v = is_f32 ? (double)static_cast<const float*>(raw)[at] : static_cast<const double*>(raw)[at];
  z[(u64)blockIdx.y * slots + i] = make_double2(v, 0.0);
}
void launch_widen_real(hipStream_t st, double2* z, const void* raw, bool is_f32, u32 n_values, u32 slots, u32 n_vec) {
  hipLaunchKernelGGL(widen_real_kernel, dim3((slots + 255) / 256, n_vec), dim3(256), 0, st, z, raw, is_f32 ? 1 : 0,
                     n_values, slots);
}

void launch_encode(hipStream_t st, const DevCtx& c, u64* out, double2* r, const double2* rou, const u32* rot,
                   u32 slots, double scaling_factor, double scale, double round_add, double range_bound,
                   const LimbMap& lm, u32 n_limbs, int* err, u32 n_vec, u64 out_stride) {
  u32 logslots = 0;
  while ((1u << logslots) < slots) ++logslots;
  launch_embed_inv_stages(st, r, rou, rot, 2 * c.N, slots, n_vec);
  hipLaunchKernelGGL(encode_round_kernel, dim3((c.N + kEncThreads - 1) / kEncThreads, n_limbs, n_vec),
                     dim3(kEncThreads), 0, st, c, out, r, slots, logslots, scaling_factor, scale, round_add,
                     range_bound, lm, err, out_stride);
}

// ---- decoding (Decode, ckks/src/encoder.c:657-704) ------------------------------------------------------
// Reconstruct (util/src/crt.c:1247-1275) followed by mpz_get_d: the centred integer behind the residues of one
// coefficient as a double, truncated towards zero.  Mixed-radix digits (x = d0 + d1 q0 + d2 q0 q1 + ...) from the
// table garner[i*stride + j] = q0..q(j-1) mod qi and inv[i] = (q0..q(i-1))^-1 mod qi, then the exact value by
// Horner's rule in `level` 64-bit words (primes are below 2^61, so it fits), compared with Q = q0..q(level-1).
__device__ double crt_to_double(const DevCtx& c, const u64* __restrict__ poly, u32 coef, u32 level,
                                const u64* __restrict__ inv, const u64* __restrict__ garner, u32 stride,
                                const u64* __restrict__ big_q) {
  u64 d[kDecodeWords], x[kDecodeWords];
  for (u32 i = 0; i < level; ++i) {
    const DevPrime p = c.primes[i];
    u64 hi = 0, lo = 0;
    for (u32 j = 0; j < i; ++j) mac128(hi, lo, d[j], garner[(u64)i * stride + j]);
    const u64 acc = barrett128(hi, lo, p);
    u64 v = poly[(u64)i * c.N + coef];
    if (v >= p.q) v %= p.q;
    const u64 t = v >= acc ? v - acc : v + p.q - acc;
    d[i] = i ? mulmod(t, inv[i], p) : t;
  }
  for (u32 k = 0; k < level; ++k) x[k] = 0;
  for (u32 i = level; i-- > 0;) {  // x = x * q_i + d_i
    const u64 q = c.primes[i].q;
    u64 carry = d[i];
    for (u32 k = 0; k < level; ++k) {
      const u64 lo = x[k] * q, hi = __umul64hi(x[k], q), s = lo + carry;
      x[k] = s;
      carry = hi + (s < lo);
    }
  }
  // negative when 2x > Q (Q is odd); 2x still fits the words: x < 2^(61 level)
  bool neg = false;
  for (u32 k = level; k-- > 0;) {
    const u64 twice = (x[k] << 1) | (k ? x[k - 1] >> 63 : 0);
    if (twice != big_q[k]) {
      neg = twice > big_q[k];
      break;
    }
  }
  if (neg) {  // x = Q - x
    u64 borrow = 0;
    for (u32 k = 0; k < level; ++k) {
      const u64 a = big_q[k], b = x[k], t = a - b - borrow;
      borrow = (a < b) || (a == b && borrow);
      x[k] = t;
    }
  }
  u32 top = level;
  while (top > 0 && x[top - 1] == 0) --top;
  if (!top) return 0.0;
  const u32 hb = 63 - (u32)__clzll((long long)x[top - 1]), bitlen = (top - 1) * 64 + hb + 1;
  double r;
  if (bitlen <= 53) {
    r = (double)x[0];
  } else {  // the 53 leading bits, the rest cut off
    const u32 sh = bitlen - 53, w = sh / 64, b = sh % 64;
    u64 m = x[w] >> b;
    if (b && w + 1 < top) m |= x[w + 1] << (64 - b);
    m &= ((u64)1 << 53) - 1;
    r = ldexp((double)m, (int)sh);
  }
  return neg ? -r : r;
}

// thread n < slots: the real part of slot n (coefficient n*gap), n >= slots: the imaginary part (coefficient
// (n-slots)*gap + N/2); each divided by the plaintext's scale and stored where the embedding's bit reversal
// wants it
__global__ __launch_bounds__(kEncThreads) void decode_crt_kernel(DevCtx c, double2* __restrict__ r,
                                                                 const u64* __restrict__ poly, u32 level, u32 slots,
                                                                 u32 logslots, double factor,
                                                                 const u64* __restrict__ inv,
                                                                 const u64* __restrict__ garner, u32 stride,
                                                                 const u64* __restrict__ big_q) {
  const u32 n = blockIdx.x * kEncThreads + threadIdx.x;
  if (n >= 2 * slots) return;
  const bool imag = n >= slots;
  const u32 i = imag ? n - slots : n, gap = c.N / (2 * slots);
  const double v = crt_to_double(c, poly, i * gap + (imag ? c.N / 2 : 0), level, inv, garner, stride, big_q) / factor;
  double* out = reinterpret_cast<double*>(r + (logslots ? (__brev(i) >> (32 - logslots)) : 0));
  out[imag ? 1 : 0] = v;
}

// stage logm of Embedding (util/src/ntt.c:598-629) on bit-reversed input: (x, y) -> (x + w y, x - w y)
__global__ __launch_bounds__(kEncThreads) void embed_fwd_stage_kernel(double2* __restrict__ r,
                                                                      const double2* __restrict__ rou,
                                                                      const u32* __restrict__ rot, u32 M, u32 logm,
                                                                      u32 len) {
#pragma clang fp contract(off)
  const u32 t = blockIdx.x * kEncThreads + threadIdx.x;
  if (t >= (len >> 1)) return;
  const u32 num = 1u << (logm - 1), i = t & (num - 1), ie = ((t >> (logm - 1)) << logm) | i, io = ie + num;
  const u32 idx_mod = 1u << (logm + 2), gap = M / idx_mod;
  const double2 w = rou[(rot[i] & (idx_mod - 1)) * gap], x = r[ie], y = r[io];
  const double pr = w.x * y.x, qr = w.y * y.y, pi = w.x * y.y, qi = w.y * y.x;
  const double omr = pr - qr, omi = pi + qi;
  r[ie] = make_double2(x.x + omr, x.y + omi);
  r[io] = make_double2(x.x - omr, x.y - omi);
}

void launch_decode(hipStream_t st, const DevCtx& c, double2* r, const u64* poly, u32 level, u32 slots, double factor,
                   const u64* inv, const u64* garner, u32 stride, const u64* big_q, const double2* rou,
                   const u32* rot) {
  u32 logslots = 0;
  while ((1u << logslots) < slots) ++logslots;
  hipLaunchKernelGGL(decode_crt_kernel, dim3((2 * slots + kEncThreads - 1) / kEncThreads), dim3(kEncThreads), 0, st, c,
                     r, poly, level, slots, logslots, factor, inv, garner, stride, big_q);
  for (u32 logm = 1; logm <= logslots; ++logm)
    hipLaunchKernelGGL(embed_fwd_stage_kernel, dim3(((slots >> 1) + kEncThreads - 1) / kEncThreads),
                       dim3(kEncThreads), 0, st, r, rou, rot, 2 * c.N, logm, slots);
}

}  // namespace ace
