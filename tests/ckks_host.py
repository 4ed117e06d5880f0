"""Host-side CKKS around the polynomial hot path, for end-to-end tests only: key generation,
canonical-embedding encode/decode, public-key encryption and decryption, in numpy and Python integers.

The evaluation (rotations, plaintext and ciphertext products, rescale) runs on the implementation under
test; this module only produces its inputs and reads its outputs.  Conventions follow the reference:
  * switch key per digit d: b_d = -a_d*s_res + e_d + P*s_src on the limbs of digit d (nothing added on the
    other limbs), a_d uniform, both over all L+k primes in NTT form, stored [digit][b | a][(L+k) limbs][N]
    (Generate_switching_key, fhe-cmplr/rtlib/ant/ckks/src/key_gen.c:127-200);
  * relinearisation key: s_src = s^2, s_res = s (key_gen.c:204-214);
  * rotation keys are "fast" keys: the evaluator switches the un-rotated c1 and applies the automorphism
    last, so the key for index k takes s to sigma_k^-1(s) (key_gen.c:216-262);
  * rotation r uses k = 5^r mod 2N (Find_automorphism_index, util/src/number_theory.c:192-204), and slot j
    of the embedding is the evaluation at zeta^(5^j), so sigma_k moves slot j+r to slot j.
"""
import numpy as np

import seeded


class CkksHost:
    def __init__(self, oracle, seed, hamming_weight=192, sigma=3.2):
        self.o = oracle
        self.N, self.L, self.K, self.parts = oracle.N, oracle.L, oracle.K, oracle.parts
        self.primes = [int(q) for q in oracle.primes]
        self.all_idx = list(range(self.L + self.K))
        self.rng = np.random.Generator(np.random.PCG64(seed))
        self.seed = seed
        self.sigma = sigma
        self._uniform_ctr = 0
        self.part_size = -(-self.L // self.parts)
        self.P = 1
        for p in self.primes[self.L:]:
            self.P *= p
        s = np.zeros(self.N, np.int64)
        pos = self.rng.choice(self.N, size=min(hamming_weight, self.N), replace=False)
        s[pos] = self.rng.choice(np.array([-1, 1], np.int64), size=pos.size)
        self.s = s
        self.s_ntt = self.small_to_ntt(s, self.all_idx)
        # slot j <-> odd power 5^j mod 2N
        n2 = 2 * self.N
        pw = [1]
        for _ in range(self.N // 2 - 1):
            pw.append(pw[-1] * 5 % n2)
        self.slot_u = (np.array(pw, np.int64) - 1) // 2  # index into the N odd-power evaluations
        self.twist = np.exp(1j * np.pi * np.arange(self.N) / self.N)

    # ---- small helpers
    def small_to_ntt(self, v, prime_idx):
        """Signed small coefficients -> residues per prime, NTT form."""
        limbs = np.concatenate([np.mod(v, self.primes[i]).astype(np.int64) for i in prime_idx])
        return self.o.ntt(limbs, prime_idx)

    def big_to_ntt(self, coeffs, prime_idx):
        """Python-integer coefficients -> residues per prime, NTT form."""
        limbs = np.concatenate([np.array([c % self.primes[i] for c in coeffs], np.int64) for i in prime_idx])
        return self.o.ntt(limbs, prime_idx)

    def uniform(self, prime_idx):
        self._uniform_ctr += 1
        return seeded.uniform_poly(self.seed * 1000003 + self._uniform_ctr, [self.primes[i] for i in prime_idx], self.N)

    def error(self):
        return np.rint(self.rng.normal(0.0, self.sigma, self.N)).astype(np.int64)

    def limbwise(self, name, a, b, prime_idx):
        n = self.N
        return np.concatenate([self.o.hw(name, a[t * n:(t + 1) * n], b[t * n:(t + 1) * n], i)
                               for t, i in enumerate(prime_idx)])

    def automorphism_coeffs(self, v, k):
        """sigma_k on a signed coefficient vector: X^i -> X^(i*k mod 2N) with the negacyclic sign."""
        out = np.zeros_like(v)
        i = np.arange(self.N)
        j = (i * k) % (2 * self.N)
        out[j % self.N] = np.where(j >= self.N, -v, v)
        return out

    # ---- keys
    def public_key(self):
        idx = list(range(self.L))
        a = self.uniform(idx)
        b = self.limbwise("modadd", self.neg(self.limbwise("modmul", a, self.s_ntt[:self.L * self.N], idx), idx),
                          self.small_to_ntt(self.error(), idx), idx)
        return b, a

    def neg(self, a, prime_idx):
        return self.limbwise("modsub", np.zeros_like(a), a, prime_idx)

    def switch_key(self, s_res_ntt, s_src_ntt, a_given=None, e_given=None):
        """Key taking a polynomial multiplying s_src to a pair decrypting under s_res (all L+k limbs, NTT).
        a_given / e_given: per digit, the uniform polynomial (NTT form) and the small error (signed coefficients)
        to use instead of drawing them."""
        n, T = self.N, self.L + self.K
        out = []
        for d in range(self.parts):
            a = a_given[d] if a_given is not None else self.uniform(self.all_idx)
            e = e_given[d] if e_given is not None else self.error()
            b = self.limbwise("modadd", self.neg(self.limbwise("modmul", a, s_res_ntt, self.all_idx), self.all_idx),
                              self.small_to_ntt(e, self.all_idx), self.all_idx)
            for i in range(d * self.part_size, min((d + 1) * self.part_size, self.L)):
                lift = self.o.hw("modmul_scalar", s_src_ntt[i * n:(i + 1) * n], self.P % self.primes[i], i)
                b[i * n:(i + 1) * n] = self.o.hw("modadd", b[i * n:(i + 1) * n], lift, i)
            out += [b, a]
        key = np.concatenate(out)
        assert key.size == 2 * self.parts * T * n
        return key

    def relin_key(self):
        s2 = self.limbwise("modmul", self.s_ntt, self.s_ntt, self.all_idx)
        return self.switch_key(self.s_ntt, s2)

    def rotation_key(self, k):
        """Fast rotation key of automorphism index k."""
        k_inv = pow(int(k), -1, 2 * self.N)
        s_res = self.small_to_ntt(self.automorphism_coeffs(self.s, k_inv), self.all_idx)
        return self.switch_key(s_res, self.s_ntt)

    # ---- encode / decode
    def embed_inverse(self, slots):
        """N/2 complex slot values -> real coefficient vector (float64)."""
        E = np.zeros(self.N, np.complex128)
        E[self.slot_u] = slots
        E[self.N - 1 - self.slot_u] = np.conj(slots)
        a = np.fft.fft(E) / self.N
        return np.real(a * np.conj(self.twist))

    def embed(self, coeffs):
        """Real coefficient vector -> N/2 complex slot values."""
        E = self.N * np.fft.ifft(np.asarray(coeffs, np.float64) * self.twist)
        return E[self.slot_u]

    def encode(self, values, scale, level):
        """values (length dividing N/2, tiled over all slots) -> plaintext, `level` limbs, NTT form."""
        values = np.asarray(values, np.complex128)
        slots = np.tile(values, (self.N // 2) // values.size)
        coeffs = np.rint(self.embed_inverse(slots) * scale)
        assert np.abs(coeffs).max() < 2.0 ** 62
        return self.small_to_ntt(coeffs.astype(np.int64), list(range(level)))

    def decode(self, coeffs, scale):
        return self.embed(np.asarray(coeffs, np.float64) / scale)

    # ---- encrypt / decrypt
    def encrypt(self, pt, pk, level):
        """Public-key encryption at `level` (pt and the result in NTT form)."""
        idx = list(range(level))
        n = level * self.N
        u = self.rng.integers(-1, 2, self.N).astype(np.int64)
        u_ntt = self.small_to_ntt(u, idx)
        c0 = self.limbwise("modadd", self.limbwise("modmul", pk[0][:n], u_ntt, idx), self.small_to_ntt(self.error(), idx), idx)
        c0 = self.limbwise("modadd", c0, pt, idx)
        c1 = self.limbwise("modadd", self.limbwise("modmul", pk[1][:n], u_ntt, idx), self.small_to_ntt(self.error(), idx), idx)
        return c0, c1

    def decrypt(self, c0, c1, level):
        """c0 + c1*s at `level` -> centred Python-integer coefficients."""
        idx = list(range(level))
        n = level * self.N
        m = self.limbwise("modadd", c0[:n], self.limbwise("modmul", c1[:n], self.s_ntt[:n], idx), idx)
        m = self.o.intt(m, idx)
        q = self.primes[:level]
        Q = 1
        for v in q:
            Q *= v
        hat = [Q // v for v in q]
        w = [h * pow(h % v, -1, v) % Q for h, v in zip(hat, q)]
        limbs = [m[t * self.N:(t + 1) * self.N].tolist() for t in range(level)]
        out = []
        for i in range(self.N):
            x = sum(limbs[t][i] * w[t] for t in range(level)) % Q
            out.append(x - Q if x > Q // 2 else x)
        return out

    def decrypt_decode(self, c0, c1, level, scale):
        return self.decode([float(v) for v in self.decrypt(c0, c1, level)], scale)
