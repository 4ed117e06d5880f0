// Host-side context construction (see ace_context.h).
#include "ace_context.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <stdexcept>

namespace ace {

u64 mul_mod(u64 a, u64 b, u64 q) { return (u64)(((u128)a * b) % q); }

u64 pow_mod(u64 a, u64 e, u64 q) {
  u64 r = 1 % q;
  a %= q;
  for (; e; e >>= 1) {
    if (e & 1) r = mul_mod(r, a, q);
    a = mul_mod(a, a, q);
  }
  return r;
}

u64 inv_mod_prime(u64 a, u64 q) { return pow_mod(a, q - 2, q); }

u64 shoup(u64 w, u64 q) { return (u64)(((u128)w << 64) / q); }

// Deterministic Miller-Rabin, exact for every 64-bit input (the reference
// uses 200 random rounds, number_theory.c:164-189; same verdicts).
static bool is_prime(u64 n) {
  if (n < 2) return false;
  static const u64 bases[] = {2, 3, 5, 7, 11, 13, 17, 19, 23, 29, 31, 37};
  for (u64 b : bases) {
    if (n == b) return true;
    if (n % b == 0) return false;
  }
  u64 d = n - 1;
  int s = 0;
  while (!(d & 1)) { d >>= 1; ++s; }
  for (u64 b : bases) {
    u64 x = pow_mod(b, d, n);
    if (x == 1 || x == n - 1) continue;
    bool witness = true;
    for (int r = 1; r < s && witness; ++r) {
      x = mul_mod(x, x, n);
      if (x == n - 1) witness = false;
    }
    if (witness) return false;
  }
  return true;
}

// crt.c:42-67.  Candidates are 1 mod 2N.  "next" starts two steps above its
// argument, as the reference does.
static i64 first_prime(uint32_t N, size_t bits) {
  i64 step = 2 * (i64)N, p = ((i64)1 << bits) + step + 1;
  while (!is_prime((u64)p)) p += step;
  return p;
}
static i64 previous_prime(i64 from, i64 step) {
  i64 p = from - step;
  while (!is_prime((u64)p)) p -= step;
  return p;
}
static i64 next_prime(i64 from, i64 step) {
  i64 p = from + 2 * step;
  while (!is_prime((u64)p)) p += step;
  return p;
}

// crt.c:112-148: the last prime is the first one above 2^sf_bits; going down
// the chain, primes alternate below / above it; q0 has its own size.
std::vector<i64> generate_q_primes(uint32_t N, size_t n, size_t q0_bits, size_t sf_bits) {
  std::vector<i64> q(n);
  i64 step = 2 * (i64)N;
  i64 lo = first_prime(N, sf_bits), hi = lo;
  q[n - 1] = lo;
  bool below = true;
  for (size_t i = n - 1; i-- > 1;) {
    if (below) { lo = previous_prime(lo, step); q[i] = lo; }
    else       { hi = next_prime(hi, step);     q[i] = hi; }
    below = !below;
  }
  q[0] = (q0_bits == sf_bits) ? previous_prime(lo, step)
                              : previous_prime(first_prime(N, q0_bits), step);
  return q;
}

// Smallest primitive root (number_theory.c:97-139).
static u64 smallest_generator(u64 q) {
  u64 phi = q - 1, rest = phi;
  std::vector<u64> fac;
  for (u64 f = 2; f * f <= rest; ++f) {
    if (rest % f == 0) {
      fac.push_back(f);
      while (rest % f == 0) rest /= f;
    }
  }
  if (rest > 1) fac.push_back(rest);
  for (u64 g = 2; g <= phi; ++g) {
    bool ok = true;
    for (u64 f : fac)
      if (pow_mod(g, phi / f, q) == 1) { ok = false; break; }
    if (ok) return g;
  }
  throw std::runtime_error("no generator");
}

// (order, prime, root) triples that override the computed root, as the
// reference's table does for ring degrees 16 and 16384 (std_param.c:229-300).
struct RootOverride { i64 order, prime, root; };
static const RootOverride kRootOverrides[] = {
#include "rou_overrides.inc"
};

static u64 root_of_unity(u64 order, u64 q) {
  if ((q - 1) % order) throw std::runtime_error("prime is not 1 mod 2N");
  for (const auto& e : kRootOverrides)
    if ((u64)e.order == order && (u64)e.prime == q) return (u64)e.root;
  return pow_mod(smallest_generator(q), (q - 1) / order, q);
}

static inline u64 bitrev(u64 v, unsigned w) {
  u64 r = 0;
  for (unsigned i = 0; i < w; ++i, v >>= 1) r = (r << 1) | (v & 1);
  return r;
}

// bit length of the product of a run of primes (crt.c:436-456)
static size_t product_bits(const i64* p, size_t n) {
  std::vector<u64> w{1};
  for (size_t i = 0; i < n; ++i) {
    u64 carry = 0;
    for (auto& limb : w) {
      u128 t = (u128)limb * (u64)p[i] + carry;
      limb  = (u64)t;
      carry = (u64)(t >> 64);
    }
    if (carry) w.push_back(carry);
  }
  size_t bits = (w.size() - 1) * 64;
  for (u64 t = w.back(); t; t >>= 1) ++bits;
  return bits;
}

void HostContext::build(uint32_t degree, const std::vector<i64>& q, size_t num_parts) {
  if (degree < 2 || (degree & (degree - 1))) throw std::runtime_error("invalid poly degree");
  if (q.empty() || num_parts == 0) throw std::runtime_error("empty modulus chain");
  N = degree;
  logN = 0;
  while ((1u << logN) < N) ++logN;
  L = q.size();
  parts = num_parts;
  part_size = (L + parts - 1) / parts;
  if (L <= part_size * (parts - 1)) throw std::runtime_error("invalid number of q parts");
  // the device arithmetic keeps lazily reduced words below 8q in 64 bits (the reference's parameter sets stop at
  // 60-bit primes)
  for (i64 v : q)
    if (v < 3 || v >= ((i64)1 << 61)) throw std::runtime_error("primes must be below 2^61");
  size_t max_bits = 0;
  for (size_t j = 0; j < parts; ++j) {
    size_t lo = j * part_size, hi = std::min(L, lo + part_size);
    max_bits = std::max(max_bits, product_bits(q.data() + lo, hi - lo));
  }
  K = (max_bits + 59) / 60;  // 60-bit special primes (AUXBITS)
  if (L + K > 96) throw std::runtime_error("more than 96 RNS primes are not supported");

  // crt.c:71-103: P primes walk down from the first 60-bit prime, skipping Q
  std::vector<i64> all(q);
  i64 step = 2 * (i64)N, prev = first_prime(N, 60);
  for (size_t i = 0; i < K; ++i) {
    i64 cand;
    bool clash;
    do {
      cand = previous_prime(prev, step);
      clash = false;
      for (i64 v : q) clash |= (v == cand);
      prev = cand;
    } while (clash);
    all.push_back(cand);
  }

  size_t T = L + K;
  primes.resize(T);
  rou.assign(T * N, 0); rou_p.assign(T * N, 0);
  irou.assign(T * N, 0); irou_p.assign(T * N, 0);
  for (size_t i = 0; i < T; ++i) {
    PrimeInfo& p = primes[i];
    p.q = (u64)all[i];
    u128 full = ~(u128)0, mu = full / p.q;
    if (full - mu * p.q == (u128)p.q - 1) ++mu;
    p.mu_lo = (u64)mu;
    p.mu_hi = (u64)(mu >> 64);
    unsigned bl = 64 - __builtin_clzll(p.q);
    p.shift = bl - 1;
    p.mu_sh = (u64)((((u128)1) << (p.shift + 64)) / p.q);
    p.br_k = 2 * ((i64)std::log2((double)all[i]) + 1);
    p.br_m = (i64)((((__int128)1) << p.br_k) / all[i]);
    p.root = root_of_unity(2ull * N, p.q);
    p.ninv = inv_mod_prime(N, p.q);
    u64 psi = p.root, ipsi = inv_mod_prime(psi, p.q);
    u64 *r = &rou[i * N], *rp = &rou_p[i * N], *ir = &irou[i * N], *irp = &irou_p[i * N];
    u64 pw = 1, ipw = 1;
    for (uint32_t e = 0; e < N; ++e) {
      u64 pos = bitrev(e, logN);
      r[pos] = pw;   rp[pos] = shoup(pw, p.q);
      ir[pos] = ipw; irp[pos] = shoup(ipw, p.q);
      pw = mul_mod(pw, psi, p.q);
      ipw = mul_mod(ipw, ipsi, p.q);
    }
  }

  // P -> Q tables (crt.c:264-291, 354-420)
  phat_inv.resize(K); phat_modq.resize(L * K); pinv_modq.resize(L); pmodq.resize(L);
  auto phat_mod = [&](size_t skip, u64 m) {
    u64 v = 1 % m;
    for (size_t t = 0; t < K; ++t)
      if (t != skip) v = mul_mod(v, primes[L + t].q % m, m);
    return v;
  };
  for (size_t j = 0; j < K; ++j) phat_inv[j] = inv_mod_prime(phat_mod(j, primes[L + j].q), primes[L + j].q);
  for (size_t i = 0; i < L; ++i) {
    u64 qi = primes[i].q;
    for (size_t j = 0; j < K; ++j) phat_modq[i * K + j] = phat_mod(j, qi);
    pmodq[i] = phat_mod((size_t)-1, qi);
    pinv_modq[i] = inv_mod_prime(pmodq[i], qi);
  }
}

size_t HostContext::num_decomp(size_t level) const {
  size_t n = (level + part_size - 1) / part_size;
  return n > parts ? parts : n;
}

// crt.c:459-566: cofactors of the digit's primes (restricted to `level`),
// modulo every prime of the complement basis [other Q limbs < level | P].
ModUpTable HostContext::modup_table(size_t level, size_t part) const {
  ModUpTable t;
  size_t nd_total = num_decomp(level);
  if (part >= nd_total) throw std::runtime_error("digit index out of range");
  size_t start = part_size * part;
  size_t len = (part == nd_total - 1) ? level - start : part_size;
  for (size_t i = 0; i < len; ++i) t.digit.push_back((int)(start + i));
  for (size_t i = 0; i < level; ++i)
    if (i < start || i >= start + len) t.compl_idx.push_back((int)i);
  for (size_t j = 0; j < K; ++j) t.compl_idx.push_back((int)(L + j));
  size_t nc = t.compl_idx.size();
  t.hat_inv.resize(len);
  t.hat.resize(len * nc);
  auto cof = [&](size_t skip, u64 m) {
    u64 v = 1 % m;
    for (size_t k = 0; k < len; ++k)
      if (k != skip) v = mul_mod(v, primes[t.digit[k]].q % m, m);
    return v;
  };
  for (size_t i = 0; i < len; ++i) {
    u64 qi = primes[t.digit[i]].q;
    t.hat_inv[i] = inv_mod_prime(cof(i, qi), qi);
    for (size_t j = 0; j < nc; ++j) t.hat[i * nc + j] = cof(i, primes[t.compl_idx[j]].q);
  }
  return t;
}

// crt.c:299-349.  The second table, floor(H*(H^-1 mod q_l)/q_l) mod q_i with H
// the cofactor of q_l in the full Q, is congruent to -q_l^-1 because q_i | H.
void HostContext::rescale_table(size_t level, std::vector<u64>& ql_inv, std::vector<u64>& neg_ql_inv) const {
  u64 ql = primes[level - 1].q;
  ql_inv.resize(level - 1);
  neg_ql_inv.resize(level - 1);
  for (size_t i = 0; i + 1 < level; ++i) {
    u64 qi = primes[i].q;
    ql_inv[i] = inv_mod_prime(ql % qi, qi);
    neg_ql_inv[i] = qi - ql_inv[i];
  }
}

// number_theory.c:192-204
uint32_t find_automorphism_index(int32_t rot_idx, uint32_t degree) {
  u64 m = 2ull * degree;
  if (rot_idx == 0) return 1;
  if (rot_idx == (int32_t)(m - 1)) return (uint32_t)rot_idx;
  u64 gen = 5;
  if (rot_idx < 0) {
    // 5^-1 mod 2N by extended Euclid (2N is not prime)
    i64 a = 5, b = (i64)m, x0 = 1, x1 = 0;
    while (b) { i64 qq = a / b, t = a % b; a = b; b = t; t = x0 - qq * x1; x0 = x1; x1 = t; }
    gen = (u64)((x0 % (i64)m + (i64)m) % (i64)m);
  }
  return (uint32_t)pow_mod(gen, (u64)std::llabs((long long)rot_idx), m);
}

// number_theory.c:206-231
void automorphism_order(i64* order, uint32_t k, uint32_t n, bool is_ntt) {
  u64 m = 2ull * n;
  unsigned logn = 0;
  while ((1u << logn) < n) ++logn;
  if (is_ntt) {
    for (u64 j = 0; j < n; ++j) {
      u64 idx = (((2 * j + 1) * k) % m) >> 1;
      order[bitrev(j, logn)] = (i64)bitrev(idx, logn);
    }
  } else {
    for (u64 j = 0; j < n; ++j) {
      u64 e = (j * k) % m;
      if (e < n) order[e] = (i64)j;
      else       order[e - n] = -(i64)j;
    }
  }
}

void fft_tables(uint32_t degree, std::vector<double>& rou, std::vector<uint32_t>& rot) {
  const size_t M = 2 * (size_t)degree, ns = M / 4;
  rou.resize(2 * M);
  for (size_t i = 0; i < M; ++i) {
    double angle = 2 * M_PI * i / M;
    rou[2 * i] = cos(angle);
    rou[2 * i + 1] = sin(angle);
  }
  rot.assign(ns ? ns : 1, 1);
  for (size_t i = 1; i < ns; ++i) rot[i] = (uint32_t)((5ull * rot[i - 1]) % M);
}

}  // namespace ace
