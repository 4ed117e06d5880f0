"""Decrypt-level pins of the oracle's ciphertext operations: with real keys from a ternary secret, the
oracle's HMult+relinearise+rescale, hoisted rotation and conjugation decrypt to the product, the rotated
and the conjugated message (what the reference's ut_ckks_arithmetic / ut_ckks_rotation tests check)."""
import numpy as np
import pytest

from ckks_host import CkksHost
from oracle_lib import Oracle

CFGS = [(1024, 4, 50, 40, 2), (256, 7, 45, 40, 3)]


@pytest.fixture(scope="module", params=CFGS, ids=lambda c: "N%d_L%d" % (c[0], c[1]))
def setup(request):
    o = Oracle(*request.param)
    h = CkksHost(o, seed=7)
    rng = np.random.default_rng(1)
    z = rng.uniform(-1, 1, o.N // 2) + 1j * rng.uniform(-1, 1, o.N // 2)
    sc = 2.0 ** request.param[3]
    ct = h.encrypt(h.encode(z, sc, o.L), h.public_key(), o.L)
    yield o, h, z, sc, ct
    o.close()


def test_encrypt_decrypt(setup):
    o, h, z, sc, (c0, c1) = setup
    assert np.abs(h.decrypt_decode(c0, c1, o.L, sc) - z).max() < 1e-6


@pytest.mark.parametrize("rot", [1, -1, 5, 100])
def test_rotation_decrypts_to_rotated_slots(setup, rot):
    o, h, z, sc, (c0, c1) = setup
    k = o.find_automorphism_index(rot)
    r0, r1 = o.fast_rotate(c0, o.precomp(c1, o.L, True), h.rotation_key(k), o.automorphism_order(k, True), o.L)
    assert np.abs(h.decrypt_decode(r0, r1, o.L, sc) - np.roll(z, -rot)).max() < 1e-6


def test_conjugation_decrypts_to_conjugate(setup):
    o, h, z, sc, (c0, c1) = setup
    k = 2 * o.N - 1
    r0, r1 = o.fast_rotate(c0, o.precomp(c1, o.L, True), h.rotation_key(k), o.automorphism_order(k, True), o.L)
    assert np.abs(h.decrypt_decode(r0, r1, o.L, sc) - np.conj(z)).max() < 1e-6


def test_hmult_relin_rescale_decrypts_to_product(setup):
    o, h, z, sc, (c0, c1) = setup
    m0, m1 = o.mul_relin_rescale(c0, c1, c0, c1, h.relin_key(), o.L)
    got = h.decrypt_decode(m0, m1, o.L - 1, sc * sc / o.primes[o.L - 1])
    assert np.abs(got - z * z).max() < 1e-6


def test_lower_level_rotation(setup):
    o, h, z, sc, (c0, c1) = setup
    level = o.L - 1  # a ciphertext that has lost one limb: keys are viewed at the lower level
    n = level * o.N
    k = o.find_automorphism_index(3)
    r0, r1 = o.fast_rotate(c0[:n], o.precomp(c1[:n], level, True), h.rotation_key(k), o.automorphism_order(k, True), level)
    assert np.abs(h.decrypt_decode(r0, r1, level, sc) - np.roll(z, -3)).max() < 1e-6
