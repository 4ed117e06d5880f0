"""End-to-end Gemm layer (encrypt -> rotations / plaintext products / rescale -> decrypt) at N=8192, 5 limbs.

CPU part: the oracle's evaluation decrypts to W x within 1e-3 (a decrypt-level pin of the oracle's key
switching, rotation and rescale that is independent of the reference's own arithmetic).
GPU part: the HIP path returns the very same ciphertext, bit for bit, and so the same decrypted result."""
import numpy as np
import pytest

import gemm_e2e as ge
from ckks_host import CkksHost
from oracle_lib import Oracle


@pytest.fixture(scope="module")
def problem():
    o = Oracle(*ge.CFG)
    host = CkksHost(o, seed=2024)
    x, w = ge.make_problem(99)
    prob = ge.prepare(host, x, w)
    want_ct = ge.evaluate(ge.OracleEval(o), prob, o.L)
    yield o, host, x, w, prob, want_ct
    o.close()


def test_oracle_gemm_decrypts_to_the_product(problem):
    o, host, x, w, prob, (r0, r1) = problem
    scale_out = prob["scale"] ** 2 / o.primes[o.L - 1]
    y = ge.decode_result(host, r0, r1, o.L - 1, scale_out)
    ref = w.astype(np.float64) @ x.astype(np.float64)
    assert np.abs(y - ref).max() < 1e-3, np.abs(y - ref).max()
    assert np.abs(y - (w @ x)).max() < 1e-3  # the fp32 product, as the reference's Validate_output_data compares


@pytest.mark.gpu
def test_gpu_gemm_matches_oracle_and_plain_product(problem):
    import acefhe

    o, host, x, w, prob, (w0, w1) = problem
    g = acefhe.Context(*ge.CFG)
    assert g.has_device, "no GPU visible"
    r0, r1 = ge.evaluate(ge.GpuEval(g), prob, g.L)
    g.close()
    assert np.array_equal(r0, w0) and np.array_equal(r1, w1), "ciphertext differs from the oracle's"
    scale_out = prob["scale"] ** 2 / o.primes[o.L - 1]
    y = ge.decode_result(host, r0, r1, o.L - 1, scale_out)
    assert np.abs(y - (w @ x)).max() < 1e-3
