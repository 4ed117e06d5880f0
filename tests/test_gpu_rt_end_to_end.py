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
from fractions import Fraction

import pytest

import rt_program

pytestmark = pytest.mark.gpu

GEMM = os.path.join(rt_program.ROOT, "tests", "programs", "gemm_program")
EXAMPLES_DIR = os.path.join(rt_program.ROOT, "oracle", "_ref", "examples")
EXAMPLES = ["add", "add_const", "avg_pool", "bootstrap", "bootstrap_02", "conv2d", "gemm", "gemm_02", "mul_const", "relin",
            "relin_02", "relu", "rotate", "rotate_02"]


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


def test_reference_example_that_expects_its_validation_to_fail():
    """eg_fhertlib_mul_const_rtv.c:62-68 is the reference's negative test of the run-time validation: the generated
    code calls Validate() on a value that cannot match (20 * 2^60 wraps under its 63-bit modulus), the harness
    compares the output with data that must not match either, prints EXPECTED FAILED! and returns 0."""
    exe = os.path.join(EXAMPLES_DIR, "eg_fhertlib_mul_const_rtv")
    if not os.path.exists(exe):
        pytest.skip("built only where the reference tree is present")
    r = run([exe], 77)
    assert r.returncode == 0 and "EXPECTED FAILED!" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
    assert "NOT EXPECTED" not in r.stdout
    assert "ERROR: validation failed" in r.stderr, r.stderr[-2000:]


def test_reference_generated_sine_program():
    """rtlib/ant/dataset/bootstrap_full.cxx: a C++ program the reference's EDSL generated (N=16384, depth 23, key
    switches open-coded with Decomp_modup / Set_pk0 / Hw_modmul / Mod_down), built unchanged with g++.  Its harness
    holds sin(8x) for eight inputs and compares to 1e-2; its side-file is the header-only one the reference ships."""
    exe = os.path.join(EXAMPLES_DIR, "bootstrap_full")
    if not os.path.exists(exe):
        pytest.skip("built only where the reference tree is present")
    env = dict(os.environ, RT_HIP_SEED="5",
               RT_HIP_DATA_FILE=os.path.join(rt_program.ROOT, "tests", "golden", "bootstrap_full_data.msg"))
    print("running", exe, flush=True)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=110, env=env)
    assert r.returncode == 0 and "SUCCESS" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


CODEC = os.path.join(rt_program.ROOT, "tests", "programs", "codec_program")


@pytest.mark.parametrize("cfg,level,sf_degree,n_values",
                         [((64, 4, 45, 40, 2), 4, 1, 32), ((4096, 4, 60, 50, 2), 3, 2, 100),
                          ((65536, 6, 50, 50, 3), 6, 1, 32768)],
                         ids=["N64", "N4096_sf2", "N65536"])
def test_plaintext_codec_matches_the_oracle(cfg, level, sf_degree, n_values, tmp_path):
    """Encode_dcmplx, the one-value form of Encode_double and Get_dcmplx_msg_from_plain, bit for bit."""
    import numpy as np

    from oracle_lib import Oracle

    assert os.path.exists(CODEC), "tests/programs/codec_program is not built"
    N, L, q0, sf, parts = cfg
    rng = np.random.Generator(np.random.PCG64(900 + N))
    values = (rng.uniform(-1, 1, n_values) + 1j * rng.uniform(-1, 1, n_values)).astype(np.complex128)
    head = np.array([N, L - 1, q0, sf, parts, level, sf_degree, n_values], np.int64)
    in_path, out_path = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(in_path, "wb") as f:
        f.write(head.tobytes() + values.tobytes())
    r = run([CODEC, in_path, out_path], 0)
    assert r.returncode == 0, r.stdout + r.stderr
    raw = open(out_path, "rb").read()
    words = level * N
    enc = np.frombuffer(raw, np.int64, words)
    dec = np.frombuffer(raw, np.complex128, N // 2, offset=8 * words)
    one = np.frombuffer(raw, np.int64, words, offset=8 * words + 16 * (N // 2))
    o = Oracle(*cfg)
    want = o.encode(values, 0, level, sf_degree)
    assert want is not None and np.array_equal(enc, want)
    want_dec = o.decode(want, level, N // 2, float(2.0 ** (sf * sf_degree)))
    assert np.array_equal(dec.view(np.float64), want_dec.view(np.float64))
    assert np.abs(dec[:n_values] - values).max() < 1e-7
    # Encode_val_at_level: a constant polynomial (constant in NTT form too) whose residues recombine to the
    # scaled value, truncated to 61 significant bits when it is larger than that
    primes = [int(q) for q in o.primes[:level]]
    o.close()
    res = one.reshape(level, N)
    assert (res == res[:, :1]).all()
    Q = 1
    for q in primes:
        Q *= q
    x = sum(int(res[t, 0]) * (Q // q) * pow(Q // q, -1, q) for t, q in enumerate(primes)) % Q
    x = x - Q if x > Q // 2 else x
    exact = Fraction(float(values[0].real)) * 2 ** (sf * sf_degree)
    assert abs(x - exact) <= max(1, abs(exact) / 2 ** 60)


BOOTSTRAP = os.path.join(rt_program.ROOT, "tests", "programs", "bootstrap_program")


@pytest.mark.parametrize("args,env", [
    ("16 25 60 51 0 8 0 1", {}),               # the reference example's ring, fully packed
    ("256 25 60 51 0 128 0 2", {}),            # uniform ternary secret: K = 512, six double-angle steps
    ("256 25 60 51 0 16 5 3", {}),             # sparsely packed, to a requested level
    ("1024 20 60 51 64 512 0 4", {}),          # Hamming weight <= 192: K = 32, three double-angle steps
    ("1024 20 60 51 64 512 0 5", {"RTLIB_BTS_EVEN_POLY": "1"}),   # the even series
    ("256 25 60 51 0 128 0 6", {"RT_BTS_CLEAR_IMAG": "1"}),       # imaginary parts cleared by conjugation
    ("16384 23 60 56 192 8192 0 7", {}),       # the reference's bootstrap_full parameters
], ids=["N16", "N256", "N256_sparse", "N1024_hw64", "N1024_even", "N256_clear_imag", "N16384"])
def test_bootstrap_refreshes_levels(args, env):
    """Encrypt at level 1, bootstrap, check the message (1e-3), the level, and one multiplication at the new level."""
    assert os.path.exists(BOOTSTRAP), "tests/programs/bootstrap_program is not built"
    e = dict(os.environ, **env)
    print("running bootstrap_program", args, env, flush=True)
    r = subprocess.run([BOOTSTRAP] + args.split(), capture_output=True, text=True, timeout=110, env=e)
    assert r.returncode == 0, r.stdout + r.stderr


RESNET20 = os.path.join(rt_program.ROOT, "oracle", "_ref", "models", "resnet20_cifar10_pre.onnx")


def bootstrap_error(args):
    """max_err printed by bootstrap_program (its exit status says whether that is below 1e-3)."""
    print("running bootstrap_program", args, flush=True)
    r = subprocess.run([BOOTSTRAP] + args.split(), capture_output=True, text=True, timeout=200)
    assert r.returncode in (0, 1) and "max_err" in r.stdout, r.stdout + r.stderr
    f = r.stdout.split()
    return float(f[f.index("max_err") + 1]), r.returncode


def test_bootstrap_on_two_lanes_equals_one_lane():
    """A fully packed bootstrap issues its two sine evaluations on the library's two lanes; with RT_HIP_ONE_LANE=1 it
    issues them one after the other.  Same keys, same input: the decrypted results are the same numbers to the last
    printed digit (the ciphertexts are bit-identical, the arithmetic being exact)."""
    assert os.path.exists(BOOTSTRAP), "tests/programs/bootstrap_program is not built"
    lines = []
    for one in ("0", "1"):
        print("running bootstrap_program, RT_HIP_ONE_LANE=" + one, flush=True)
        r = subprocess.run([BOOTSTRAP] + "1024 20 60 51 64 512 0 4".split(), capture_output=True, text=True, timeout=110,
                           env=dict(os.environ, RT_HIP_ONE_LANE=one))
        assert r.returncode == 0, r.stdout + r.stderr
        f = r.stdout.split()
        lines.append((f[f.index("max_err") + 1], f[f.index("square_err") + 1], f[f.index("level") + 1]))
    assert lines[0] == lines[1], lines


def test_bootstrap_precision_at_the_model_ring():
    """N = 65536, 34 limbs, Hamming weight 192, 32768 slots, refreshed to level 15 (the call of the ResNet programs).
    On the chain the reference's build scripts compile the models with (q0 = 60, scale = 56 bits:
    scripts/build_resnet20_cifar10.sh:13-14,32) the error stays below 1e-3.  The scale is tracked nominally, as in the
    reference (Rescale_ciphertext divides the recorded scale by 2^scale_bits, ckks/src/evaluator.c:342-362, with
    _scaling_factor = 1 << scaling_mod_size, ckks/src/param.c:68), so every rescale leaves the relative error
    d_l = q_l / 2^scale_bits - 1 of its prime in the value; the sine evaluation sees it multiplied by the integer
    part, q0 / scale and, after the slot transform, sqrt(N).  d_l is the distance of the primes = 1 mod 2N from
    2^scale_bits, so it grows with N and falls with 2^scale_bits: the error follows that law across rings and
    chains, and the defaults compiled into the committed programs (51 / 46 bits) are far outside 1e-3 at this ring."""
    assert os.path.exists(BOOTSTRAP), "tests/programs/bootstrap_program is not built"
    good, rc = bootstrap_error("65536 33 60 56 192 32768 15 1")
    assert rc == 0 and good < 1e-3, good
    e46, _ = bootstrap_error("65536 33 51 46 192 32768 15 1")
    e50, _ = bootstrap_error("65536 33 55 50 192 32768 15 1")
    e46_small, _ = bootstrap_error("16384 33 51 46 192 8192 15 1")
    print("max_err: 60/56 %.3g  55/50 %.3g  51/46 %.3g  51/46 at N=16384 %.3g" % (good, e50, e46, e46_small), flush=True)
    assert 1e-2 < e46 < 1.0
    # 4 more scale bits: d_l / 16; a quarter of the ring: d_l / 4 and sqrt(N) / 2 -- each within a factor 3
    assert 16 / 3 < e46 / e50 < 16 * 3, (e46, e50)
    assert 8 / 3 < e46 / e46_small < 8 * 3, (e46, e46_small)


# Synthetic weights of this amplitude give logits of a few tenths with every ReLU input inside the range of the
# compiler's polynomial (at 0.15 the logits are below 0.02; at 0.4 they reach 3 and two runs under different keys
# differ by 8e-4; at 0.6 the activations leave the range and the outputs are noise of size 10^3).
AMPLITUDE = "0.33"


def resnet20_run(chain, key_seed, images=1, threads=1, amplitude=AMPLITUDE, late_threads=False):
    """logits of each image, in the order of the images"""
    env = dict(os.environ, RT_HIP_SYNTHETIC_WEIGHTS=amplitude, MODEL_Q0_BITS=str(chain[0]), MODEL_SF_BITS=str(chain[1]),
               MODEL_KEY_SEED=str(key_seed), MODEL_THREADS=str(threads))
    if late_threads:
        env["MODEL_LATE_THREADS"] = "1"
    print("running", RESNET20, "chain", chain, "key seed", key_seed, "images", images, "threads", threads, flush=True)
    r = subprocess.run([RESNET20, "3", "32", "32", "10", "1", str(images)], capture_output=True, text=True, timeout=230,
                       env=env)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    rows = [l.split("output:")[1].split() for l in r.stdout.splitlines() if l.startswith("output:")]
    rows += [l.split("output:")[1].split() for l in sorted(
        (l for l in r.stdout.splitlines() if l.startswith("image ") and "output:" in l), key=lambda l: int(l.split()[1]))]
    assert len(rows) == images and all(len(row) == 10 for row in rows), r.stdout[-2000:]
    return [[float(v) for v in row] for row in rows]


def test_bootstrap_precision_over_seeds_and_slot_counts():
    """The bootstrap has no bit-level counterpart here, so its margin against the 1e-3 bound is shown over the keys
    and messages rather than on one draw: five seeds at the full slot count of the model ring on the published
    chain (60 / 56 bits, refreshed to level 15 as the ResNet programs ask), and the sparse slot counts a packed
    model uses (a sparsely packed message is raised, summed over its copies and refreshed through the shorter
    transforms)."""
    assert os.path.exists(BOOTSTRAP), "tests/programs/bootstrap_program is not built"
    worst = 0.0
    for seed in (1, 2, 3, 4, 5):
        err, rc = bootstrap_error("65536 33 60 56 192 32768 15 %d" % seed)
        print("seed", seed, "max_err %.3g" % err, flush=True)
        assert rc == 0 and err < 1e-3, (seed, err)
        worst = max(worst, err)
    for slots in (16384, 8192, 4096):
        err, rc = bootstrap_error("65536 33 60 56 192 %d 15 1" % slots)
        print("slots", slots, "max_err %.3g" % err, flush=True)
        assert rc == 0 and err < 1e-3, (slots, err)
        worst = max(worst, err)
    print("worst max_err %.3g" % worst, flush=True)


def resnet20_logits(chain, key_seed, amplitude=AMPLITUDE):
    return resnet20_run(chain, key_seed, amplitude=amplitude)[0]


def test_reference_resnet20_program_is_stable_under_the_keys():
    """The compiler's ResNet-20 program (7000 lines of generated C at N=65536, 34 limbs, 197 rotation keys, 19
    bootstraps, 1038 weight plaintexts encoded on the fly), unchanged, on the chain the reference's build script
    compiles it with (60 / 56 bits).  The weight file is not part of the reference tree, so weights and image are
    pseudo-random and there is no expected output; what is checked is that the ten logits do not depend on the
    secret key, the encryption randomness or the key-switching noise: two runs that differ in all of those agree
    within 1e-3 (a numerically meaningless run, as on the compiled-in 51 / 46 chain, fails this by orders of
    magnitude).  The operators the program is made of are checked with expected values by the reference's examples."""
    if not os.path.exists(RESNET20):
        pytest.skip("built only where the reference tree is present")
    a, b = resnet20_logits((60, 56), 11), resnet20_logits((60, 56), 22)
    spread = max(abs(x - y) for x, y in zip(a, b))
    print("logits", a, "spread", spread, flush=True)
    assert all(v == v and abs(v) < 10 for v in a)
    assert max(abs(v) for v in a) > 0.1, "the logits carry no signal"
    assert spread < 1e-3 and spread < 0.01 * max(abs(v) for v in a), spread


MODELS_DIR = os.path.join(rt_program.ROOT, "oracle", "_ref", "models")


def model_logits(exe, images, env):
    print("running", exe, "images", images, flush=True)
    r = subprocess.run([exe, "3", "32", "32", "10", "1", str(images)], capture_output=True, text=True, timeout=140, env=env)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    rows = [[float(v) for v in l.split("output:")[1].split()] for l in r.stdout.splitlines() if l.startswith("output:")]
    assert len(rows) == images and all(len(row) == 10 for row in rows), r.stdout[-2000:]
    return rows


@pytest.mark.parametrize("model,images", [("resnet20_cifar10_pre.onnx", 2), ("resnet32_cifar10_pre.onnx", 1),
                                          ("resnet32_cifar100_pre.onnx", 1), ("resnet44_cifar10_pre.onnx", 1),
                                          ("resnet56_cifar10_pre.onnx", 1), ("resnet110_cifar10_pre.onnx", 1)])
def test_reference_models_decrypt_to_their_plain_float_run(model, images):
    """The value-level check of the whole models.  The reference's weight files and expected logits are not in its
    tree, so the expected output is made here: the same generated program (unchanged) is compiled a second time
    over a plain-float stand-in for the runtime (tests/programs/shadow/rt_ant/rt_ant.h: a ciphertext is its message,
    Hw_* act slot by slot, rotations permute slots, Rescale and Bootstrap copy) and run on the host with the same
    image and the same pseudo-random weights.  The encrypted run on the GPU -- 34 limbs at N = 65536, 197 to 268
    rotation keys, 19 to 109 bootstraps, the compiler's polynomial ReLUs -- must decrypt to the same ten logits within
    1e-3, the bound of the reference's own drivers (measured 2e-4 on logits of 0.1 to 1.8).  A rotation by a wrong
    amount, a plaintext at a wrong level or scale, a lost limb or a wrong key anywhere in the 7 000 to 25 000 lines
    fails this; so does a bootstrap outside its precision."""
    gpu, host = os.path.join(MODELS_DIR, model), os.path.join(MODELS_DIR, model + "_shadow")
    if not (os.path.exists(gpu) and os.path.exists(host)):
        pytest.skip("built only where the reference tree is present")
    env = dict(os.environ, RT_HIP_SYNTHETIC_WEIGHTS=AMPLITUDE, MODEL_Q0_BITS="60", MODEL_SF_BITS="56", MODEL_KEY_SEED="11")
    want = model_logits(host, images, env)
    got = model_logits(gpu, images, env)
    for i, (g, w) in enumerate(zip(got, want)):
        d = max(abs(x - y) for x, y in zip(g, w))
        print("image", i + 1, "plain float", w, "encrypted", g, "difference %.3g" % d, flush=True)
        assert max(abs(v) for v in w) > 0.05, "the logits carry no signal"
        assert d < 1e-3, (i, d)


def test_reference_resnet20_program_on_three_threads():
    """Images of a batch on several host threads at once, as the reference's driver runs them
    (dataset/resnet_cifar.main.inc:81-112: `#pragma omp parallel for`, input and output sections critical): one set
    of keys, tables and kept plaintexts, a context of the family per thread.  Every image's logits are those of the
    run that takes the images one after the other, up to the encryption randomness (each thread draws its own).
    (A random network of this depth barely follows its input: two images' logits differ by some 6e-4 at this
    amplitude, so nothing is asserted about that.)"""
    if not os.path.exists(RESNET20):
        pytest.skip("built only where the reference tree is present")
    one = resnet20_run((60, 56), 11, images=4)
    # the second run's other threads first call in after the first image: they meet a runtime that has worked alone
    # (no waiting after publishing, weight plaintexts of the next run still on their way on its second stream)
    for late in (False, True):
        three = resnet20_run((60, 56), 11, images=4, threads=3, late_threads=late)
        for i, (a, b) in enumerate(zip(one, three)):
            d = max(abs(x - y) for x, y in zip(a, b))
            print("image", i + 1, "one thread", a, "difference on three threads", d, "late" if late else "", flush=True)
            assert d < 1e-3 and d < 0.01 * max(abs(v) for v in a), (i, d, late)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_operator_block_at_the_model_ring(seed, tmp_path):
    """One block of a compiled model at the size the whole models run at (N=65536, 34 limbs, 60/56 bits), with weights
    the test program knows (tests/programs/operator_program.c): a 3x3 convolution over four channels laid out as the
    compiler lays out ResNet-20's first one, its plaintexts read by Pt_from_msg from a side-file the program writes,
    then Bootstrap to level 15 and the compiler's own App_relu / Rotate / Relinearize from the included ResNet-20
    program.  Expected values are the validation mode's float models (Conv_impl, Relu_impl), which are pinned to the
    reference's rt_validate.c.  Bounds: the convolution 1e-5 (measured 8e-10), the bootstrapped values 1e-3 (5e-4),
    the ReLU 1e-3 where |x| >= 0.1 as in the reference's relu example (4e-4) and 1e-2 everywhere (3e-3: the
    polynomial's fit is loosest around zero)."""
    exe = os.path.join(rt_program.ROOT, "oracle", "_ref", "models", "operator_block")
    if not os.path.exists(exe):
        pytest.skip("built only where the reference tree is present")
    print("running", exe, seed, flush=True)
    r = subprocess.run([exe, str(tmp_path / "block.msg"), str(seed)], capture_output=True, text=True, timeout=200)
    print(r.stdout, flush=True)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    f = r.stdout.split()
    v = {f[i]: float(f[i + 1]) for i in range(0, 12, 2)}
    assert v["conv_err"] < 1e-5 and v["bootstrap_err"] < 1e-3 and v["relu_err_away_from_zero"] < 1e-3
    assert v["relu_err"] < 1e-2 and v["level"] == 15


def test_reference_resnet20_program_runs_on_its_compiled_in_chain():
    """The same program with the parameters it carries (51 / 46 bits): runs to the end.  Its bootstraps are far
    outside their precision on this chain (test_bootstrap_precision_at_the_model_ring), in the reference's arithmetic
    as here, so nothing is asserted about the values beyond their being numbers."""
    if not os.path.exists(RESNET20):
        pytest.skip("built only where the reference tree is present")
    env = dict(os.environ, RT_HIP_SYNTHETIC_WEIGHTS="0.05")
    print("running", RESNET20, flush=True)
    r = subprocess.run([RESNET20, "3", "32", "32", "10", "1"], capture_output=True, text=True, timeout=230, env=env)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    out = [l for l in r.stdout.splitlines() if l.startswith("output:")][0].split()[1:]
    assert len(out) == 10 and all(v == v and abs(v) != float("inf") for v in map(float, out))


CONV_PROGRAMS = ["conv_3x16x32x3", "conv_16x16x32x3", "conv_32x32x16x3", "conv_64x64x8x3", "conv_128x128x28x3",
                 "conv_256x256x14x3", "conv_512x512x7x3"]


@pytest.mark.parametrize("name", CONV_PROGRAMS)
def test_reference_conv_programs_run(name, tmp_path):
    """The reference's single-layer convolution programs (rtlib/ant/dataset/conv_*.cxx: the compiler's output plus a
    driver with the input, the expected output and, in three of them, the comparison), built unchanged, run to the end.  Their
    weight files are not in the reference tree, so the weights are pseudo-random and the comparison with the expected
    output cannot succeed: what is checked is that every runtime call of these programs is there and works (they
    use the per-event timing marks, whose table must list the convolution), and that the output is finite."""
    exe = os.path.join(rt_program.ROOT, "oracle", "_ref", "models", name)
    if not os.path.exists(exe):
        pytest.skip("built only where the reference tree is present")
    table = tmp_path / "timing.txt"
    env = dict(os.environ, RT_HIP_SYNTHETIC_WEIGHTS="0.05", RTLIB_TIMING_OUTPUT=str(table), PRINT_ALL="1")
    print("running", exe, flush=True)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=200, env=env)
    assert r.returncode in (0, 1), r.stdout[-1500:] + r.stderr[-1500:]
    # some of the drivers have their comparison commented out and only run the graph
    if "expect absolute error" in r.stdout:
        assert "FAILED!" in r.stdout or "SUCCESS!" in r.stdout, r.stdout[-1500:]
        values = [float(l.split("result: ")[1].split(",")[0]) for l in r.stdout.splitlines() if l.startswith("index: ") and "result: " in l]
        assert len(values) >= 1024 and all(v == v and abs(v) < 1e6 for v in values)
    else:
        assert r.returncode == 0
    text = table.read_text()
    assert "RTLib functions" in text and "NN_CONV" in text, text


MSG = os.path.join(rt_program.ROOT, "tests", "programs", "msg_program")


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_plaintexts_from_a_weight_file(dtype, tmp_path):
    """Pt_from_msg / Pt_from_msg_ofst read the right entry of a side-file and encode it like Encode_float."""
    import numpy as np

    import msgfile
    from oracle_lib import Oracle

    assert os.path.exists(MSG), "tests/programs/msg_program is not built"
    cfg, level = (4096, 4, 60, 50, 2), 3
    N = cfg[0]
    rng = np.random.Generator(np.random.PCG64(31))
    np_type = np.float32 if dtype == "f32" else np.float64
    entries = [("w%d" % i, rng.uniform(-1, 1, n).astype(np_type), 1, level) for i, n in enumerate((5, 2048, 77, 1000))]
    path, out_path = str(tmp_path / "weights.msg"), str(tmp_path / "out.bin")
    msgfile.write(path, entries, np_type)
    # the last three repeat earlier ones: served from the encoded plaintexts kept in HBM
    picks = [(1, 0, 2048), (3, 0, 900), (2, 10, 60), (0, 0, 5), (3, 0, 900), (1, 0, 2048), (2, 10, 60)]
    args = [MSG, path, str(N), str(cfg[1] - 1), str(cfg[2]), str(cfg[3]), str(cfg[4]), str(level), out_path]
    for p in picks:
        args += [str(v) for v in p]
    r = run(args, 0)
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(out_path, np.int64).reshape(len(picks), level * N)
    if dtype == "f64":  # and with nothing kept
        env = dict(os.environ, RT_HIP_PLAINTEXT_CACHE_GB="0")
        r2 = subprocess.run(args, capture_output=True, text=True, timeout=110, env=env)
        assert r2.returncode == 0, r2.stdout + r2.stderr
        assert np.array_equal(np.fromfile(out_path, np.int64).reshape(len(picks), level * N), got)
    o = Oracle(*cfg)
    for row, (index, ofst, n) in zip(got, picks):
        values = np.asarray(entries[index][1][ofst:ofst + n], np.float64).astype(np.complex128)
        assert np.array_equal(row, o.encode(values, 0, level, 1)), (index, ofst, n)
    o.close()
    if dtype == "f32":  # an index past the table is refused the way the reference refuses it
        bad = run(args[:9] + ["9", "0", "4"], 0)
        assert bad.returncode != 0 and "index out of entry range" in bad.stderr


SURFACE = os.path.join(rt_program.ROOT, "tests", "programs", "surface_program")


@pytest.mark.parametrize("args", [
    "4096 5 60 50 11",
    "65536 4 60 50 12",
    "1024 20 60 51 13 bootstrap",
], ids=["N4096", "N65536", "N1024_staged_bootstrap"])
def test_less_used_entry_points(args):
    """One-limb polynomials, per-limb scalars, Alloc_precomp's list, Automorphism_transform, Upscale / Downscale /
    Raise_mod, Reset_ciph, Encode_float_with_scale, Prepare_input_dup, a file of pre-encoded plaintexts read by
    Pt_get, and the three staged bootstrap operators: each against the entry points the committed programs use
    (bit for bit) or the message it must decrypt to."""
    assert os.path.exists(SURFACE), "tests/programs/surface_program is not built"
    print("running surface_program", args, flush=True)
    r = subprocess.run([SURFACE] + args.split(), capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and "surface ok" in r.stdout, r.stdout + r.stderr


KEYGEN = os.path.join(rt_program.ROOT, "tests", "programs", "keygen_program")


@pytest.mark.parametrize("cfg,hw", [((8192, 5, 40, 40, 3), 192), ((65536, 6, 60, 50, 3), 192), ((2048, 4, 50, 40, 2), 0)],
                         ids=["N8192", "N65536", "N2048_uniform_secret"])
def test_device_built_keys_satisfy_their_defining_equations(cfg, hw, tmp_path):
    """Keys built in HBM by Rt_generate_keys against Generate_switching_key (key_gen.c:127-262): for every digit,
    b + a*s_res - P*s_src*[limb in the digit] must be ONE small polynomial (coefficients -1, 0, 1) seen through all
    L+k limbs -- a dropped term, a wrong sign, the lift on the wrong limbs or a wrong automorphism of the secret
    leaves residues that are large or differ between limbs -- and rebuilding b on the CPU from the same (a, e, s)
    gives the device's words bit for bit.  Relinearisation, two rotations, the conjugation, and the public key."""
    import numpy as np

    from ckks_host import CkksHost
    from oracle_lib import Oracle

    assert os.path.exists(KEYGEN), "tests/programs/keygen_program is not built"
    N, num_q, q0_bits, sf_bits, parts = cfg
    rots = [1, -3, 2 * N - 1]
    out_path = str(tmp_path / "keys.bin")
    args = [KEYGEN, out_path, str(N), str(num_q - 1), str(q0_bits), str(sf_bits), str(hw), "77"] + [str(r) for r in rots]
    print("running keygen_program", args[2:], flush=True)
    r = subprocess.run(args, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stdout + r.stderr
    o = Oracle(*cfg)
    L, K, T = o.L, o.K, o.L + o.K
    raw = np.fromfile(out_path, np.int64)
    key_words = 2 * parts * T * N
    assert raw.size == N + 2 * L * N + (1 + len(rots)) * key_words
    s = raw[:N]
    assert set(np.unique(s)) <= {-1, 0, 1}
    if hw:
        assert int(np.abs(s).sum()) == hw and abs(int((s == 1).sum()) - hw // 2) <= 1
    else:
        assert N // 2 < int(np.abs(s).sum()) < 3 * N // 4  # uniform over {-1, 0, 1}
    h = CkksHost(o, 5, hamming_weight=min(192, N))
    h.s, h.s_ntt = s, h.small_to_ntt(s, h.all_idx)
    all_idx, q_idx = h.all_idx, list(range(L))

    def small_poly(res_ntt, idx, what):
        """the polynomial whose residues res_ntt holds: must be small and the same through every limb"""
        c = o.intt(res_ntt, idx).reshape(len(idx), N)
        qs = np.array([o.primes[i] for i in idx], np.int64)[:, None]
        c = np.where(c > qs // 2, c - qs, c)
        assert np.abs(c).max() <= 1, "%s: residual is not small (max %d)" % (what, int(np.abs(c).max()))
        assert (c == c[0]).all(), "%s: residual differs between limbs" % what
        assert N // 4 < int(np.abs(c[0]).sum()) < 3 * N // 4, "%s: not the triangle distribution" % what
        return c[0]

    pk0, pk1 = raw[N:N + L * N], raw[N + L * N:N + 2 * L * N]
    small_poly(h.limbwise("modadd", pk0, h.limbwise("modmul", pk1, h.s_ntt[:L * N], q_idx), q_idx), q_idx, "public key")
    s2 = h.limbwise("modmul", h.s_ntt, h.s_ntt, all_idx)
    cases = [("relin", h.s_ntt, s2)]
    for rot in rots:
        k = 2 * N - 1 if rot == 2 * N - 1 else o.find_automorphism_index(rot)
        s_res = h.small_to_ntt(h.automorphism_coeffs(s, pow(int(k), -1, 2 * N)), all_idx)
        cases.append(("rotation %d" % rot, s_res, h.s_ntt))
    seen_a = []
    for ci, (name, s_res, s_src) in enumerate(cases):
        key = raw[N + 2 * L * N + ci * key_words:N + 2 * L * N + (ci + 1) * key_words]
        a_list, e_list = [], []
        for d in range(parts):
            b, a = key[2 * d * T * N:(2 * d + 1) * T * N], key[(2 * d + 1) * T * N:(2 * d + 2) * T * N]
            assert all((a[t * N:(t + 1) * N] < o.primes[i]).all() and (a[t * N:(t + 1) * N] >= 0).all() for t, i in enumerate(all_idx))
            res = h.limbwise("modadd", b, h.limbwise("modmul", a, s_res, all_idx), all_idx)
            for i in range(d * h.part_size, min((d + 1) * h.part_size, L)):
                lift = o.hw("modmul_scalar", s_src[i * N:(i + 1) * N], h.P % o.primes[i], i)
                res[i * N:(i + 1) * N] = o.hw("modsub", res[i * N:(i + 1) * N], lift, i)
            e_list.append(small_poly(res, all_idx, "%s digit %d" % (name, d)))
            a_list.append(a)
            seen_a.append(a[:64].tobytes())
        assert np.array_equal(h.switch_key(s_res, s_src, a_list, e_list), key), name
    assert len(set(seen_a)) == len(seen_a), "the uniform polynomials of two digits or keys coincide"
    o.close()
