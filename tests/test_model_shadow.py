"""The plain-float stand-in for the runtime (tests/programs/shadow/rt_ant/rt_ant.h), on the host: the generated
ResNet-20 program (rtlib/ant/dataset/resnet20_cifar10_pre.onnx.inc), included unchanged over it, runs to the end,
is a function of the image and of the weights' amplitude only, and follows its input.  What the encrypted run on the
GPU is compared with (tests/test_gpu_rt_end_to_end.py::test_reference_models_decrypt_to_their_plain_float_run)."""
import os
import subprocess

import pytest

import rt_program

SHADOW = os.path.join(rt_program.ROOT, "oracle", "_ref", "models", "resnet20_cifar10_pre.onnx_shadow")


def logits(seed, amplitude, images=1):
    env = dict(os.environ, RT_HIP_SYNTHETIC_WEIGHTS=amplitude)
    r = subprocess.run([SHADOW, "3", "32", "32", "10", str(seed), str(images)], capture_output=True, text=True,
                       timeout=120, env=env)
    assert r.returncode == 0, r.stdout[-1000:] + r.stderr[-1000:]
    rows = [[float(v) for v in l.split()[1:]] for l in r.stdout.splitlines() if l.startswith("output:")]
    assert len(rows) == images and all(len(x) == 10 for x in rows)
    return rows


def test_plain_float_run_of_the_generated_resnet20_program():
    if not os.path.exists(SHADOW):
        pytest.skip("built only where the reference tree is present")
    a = logits(1, "0.33", images=2)
    assert a == logits(1, "0.33", images=2), "the run depends on something besides its arguments"
    assert all(v == v and abs(v) < 10 for row in a for v in row)
    assert max(abs(v) for v in a[0]) > 0.1, "the logits carry no signal"
    assert a[0] != a[1] and a[0] != logits(2, "0.33")[0], "the logits do not follow the image"
    assert a[0] != logits(1, "0.30")[0], "the logits do not follow the weights"
    # without weights there is nothing to run on
    r = subprocess.run([SHADOW, "3", "32", "32", "10", "1"], capture_output=True, text=True, timeout=60,
                       env={k: v for k, v in os.environ.items() if k != "RT_HIP_SYNTHETIC_WEIGHTS"})
    assert r.returncode == 2
