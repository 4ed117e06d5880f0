"""A compiler-shaped C program run on the HIP-backed runtime (rt_hip.h) and compared, limb by limb,
with the CPU oracle's evaluation of the same graph (needs an MI355X)."""
import os

import numpy as np
import pytest

import rt_program
from oracle_lib import Oracle

pytestmark = pytest.mark.gpu

CASES = [((64, 4, 45, 40, 2), [1, -1, 5]), ((8192, 5, 40, 40, 3), [1, 7, -3]), ((65536, 6, 50, 50, 3), [1, -1])]


@pytest.mark.parametrize("cfg,rots", CASES, ids=lambda v: "N%d_L%d" % (v[0], v[1]) if isinstance(v, tuple) else "")
def test_generated_style_program(cfg, rots, tmp_path):
    assert os.path.exists(rt_program.PROGRAM), "tests/programs/keyswitch_program is not built"
    o = Oracle(*cfg)
    blob, data = rt_program.make_inputs(o, cfg, rots, seed=4000 + cfg[0])
    in_path, out_path = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(in_path, "wb") as f:
        f.write(blob)
    print("running keyswitch_program", cfg, rots, flush=True)
    res = rt_program.run_program(in_path, out_path)
    assert res.returncode == 0, res.stdout + res.stderr
    got = rt_program.read_outputs(out_path, cfg[0])
    want = rt_program.expected_outputs(o, data, rots)
    o.close()
    assert len(got) == len(want) == 2 * len(rots) + 2
    names = ["open-coded hmult"] + ["open-coded rotate %d" % r for r in rots] + ["Mul_ciph+Rescale_ciph"] + \
            ["Rotate_batch_ciph %d" % r for r in rots]
    for name, (gl, g0, g1), (wl, w0, w1) in zip(names, got, want):
        assert gl == wl, name
        assert np.array_equal(g0, w0), name + " c0"
        assert np.array_equal(g1, w1), name + " c1"
