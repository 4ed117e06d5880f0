"""Whole programs on the HIP-backed runtime: context, key generation, encoding, encryption, the evaluation
graph, decryption and decoding (needs an MI355X).

  * tests/programs/gemm_program: y = (W x + b)^2 with plaintext weights encoded by the program, checked
    against the floating-point result to 1e-3, plus the reference's encode test
    (rtlib/ant/test/test_ant_encode.c: Encode_float, Get_msg_from_plain within 1e-7);
  * the reference's own examples (rtlib/ant/example/eg_fhertlib_*.c: a generated program and a harness that
    holds the expected output and compares to 1e-3), compiled unchanged against this runtime where the
    reference tree was present at build time.  Their binaries live under oracle/_ref/examples.
"""
import os
import subprocess

import pytest

import rt_program

pytestmark = pytest.mark.gpu

GEMM = os.path.join(rt_program.ROOT, "tests", "programs", "gemm_program")
EXAMPLES_DIR = os.path.join(rt_program.ROOT, "oracle", "_ref", "examples")
EXAMPLES = ["add", "add_const", "avg_pool", "conv2d", "gemm", "gemm_02", "mul_const", "relin", "relin_02", "rotate",
            "rotate_02"]


def run(cmd, seed):
    env = dict(os.environ, RT_HIP_SEED=str(seed))
    print("running", " ".join(cmd), "seed", seed, flush=True)
    return subprocess.run(cmd, capture_output=True, text=True, timeout=110, env=env)


@pytest.mark.parametrize("degree,dim", [(4096, 8), (16384, 16), (65536, 32)])
def test_gemm_square_program(degree, dim):
    assert os.path.exists(GEMM), "tests/programs/gemm_program is not built"
    r = run([GEMM, str(degree), str(dim), str(1000 + dim)], 0)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "max_err" in r.stdout


@pytest.mark.parametrize("name", EXAMPLES)
def test_reference_example(name):
    exe = os.path.join(EXAMPLES_DIR, "eg_fhertlib_" + name)
    if not os.path.exists(exe):
        pytest.skip("built only where the reference tree is present")
    r = run([exe], 77)
    assert r.returncode == 0 and "SUCESS" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
