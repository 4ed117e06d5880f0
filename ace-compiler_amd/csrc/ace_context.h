// Host-side CRT/NTT context of the MI355X CKKS runtime: prime chain, 2N-th
// roots, twiddle tables and base-conversion constants, built once on the CPU
// and uploaded to HBM by the caller.  Follows the reference's rules so that
// every table is value-identical (fhe-cmplr/rtlib/ant/util/src/crt.c:42-582,
// ntt.c:34-138, number_theory.c:97-162).
#pragma once
#include <cstddef>
#include <cstdint>
#include <vector>

namespace ace {

using u64  = uint64_t;
using i64  = int64_t;
using u128 = unsigned __int128;

// One RNS modulus with every per-prime constant the kernels need.
struct PrimeInfo {
  u64 q;          // the prime
  u64 mu_lo;      // floor(2^128 / q), low / high word (Mod_barrett_128's mu)
  u64 mu_hi;
  u64 mu_sh;      // floor(2^(shift+64) / q) for products of two residues
  uint32_t shift; // bitlen(q) - 1
  i64 br_k, br_m; // MODULUS::_br_k/_br_m (include/util/modular.h:67-72)
  u64 root;       // primitive 2N-th root psi
  u64 ninv;       // N^-1 mod q
};

struct ShoupConst {
  u64 w, wp;  // value and floor(w * 2^64 / q)
};

// Tables for raising digit `part` at `level` (Decomp_modup).
struct ModUpTable {
  std::vector<int> digit;        // prime indices of the digit limbs
  std::vector<int> compl_idx;    // prime indices of the target limbs, reference order
  std::vector<u64> hat_inv;      // [nd]  (D/q_i)^-1 mod q_i
  std::vector<u64> hat;          // [nd][nc]  (D/q_i) mod m_j
};

struct HostContext {
  uint32_t N = 0, logN = 0;
  size_t L = 0, K = 0, parts = 0, part_size = 0;
  std::vector<PrimeInfo> primes;            // [L+K]
  // twiddles, [L+K][N] each: psi^bitrev powers, their Shoup companions, inverses
  std::vector<u64> rou, rou_p, irou, irou_p;
  // P -> Q conversion (Mod_down)
  std::vector<u64> phat_inv;   // [K]
  std::vector<u64> phat_modq;  // [L][K]
  std::vector<u64> pinv_modq;  // [L]
  std::vector<u64> pmodq;      // [L]

  void build(uint32_t degree, const std::vector<i64>& q, size_t num_parts);
  size_t num_decomp(size_t level) const;
  ModUpTable modup_table(size_t level, size_t part) const;
  // rescale constants at `level`: q_l^-1 mod q_i and -q_l^-1 mod q_i, i < level-1
  void rescale_table(size_t level, std::vector<u64>& ql_inv, std::vector<u64>& neg_ql_inv) const;
};

// prime chain of Init_crtcontext_with_prime_size
std::vector<i64> generate_q_primes(uint32_t degree, size_t num_q, size_t q0_bits, size_t sf_bits);

u64 mul_mod(u64 a, u64 b, u64 q);
u64 pow_mod(u64 a, u64 e, u64 q);
u64 inv_mod_prime(u64 a, u64 q);
u64 shoup(u64 w, u64 q);
uint32_t find_automorphism_index(int32_t rot_idx, uint32_t degree);
// Precompute_fft (util/src/ntt.c:559-587) for fft_length = 2*degree: rou[2i], rou[2i+1] = cos, sin of
// 2 pi i / (2*degree) for i < 2*degree; rot[i] = 5^i mod 2*degree for i < degree/2.
// This file is built with the host C++ compiler, not hipcc, so that cos and sin are the C library's,
// as in the reference: the encoder's results depend on the last bit of these tables.
void fft_tables(uint32_t degree, std::vector<double>& rou, std::vector<uint32_t>& rot);
void automorphism_order(i64* order, uint32_t k, uint32_t degree, bool is_ntt);

}  // namespace ace
