"""The per-event timing table (Append_rtlib_timing / Report_rtlib_timing of librt_hip.so) against the reference's own
rtlib_timing.c compiled as it lies (oracle/_ref/libref_timing.so): the same sequence of recorded events prints the
same table, character for character (event names by number, indentation by level, group headers, sub totals, the
nested-time form)."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = os.path.join(ROOT, "oracle", "_ref", "libref_timing.so")
OURS = os.path.join(ROOT, "ace-compiler_amd", "librt_hip.so")

pytestmark = pytest.mark.skipif(not os.path.exists(REF), reason="built only where the reference tree is present")

CHILD = """
import ctypes as C, sys
lib = C.CDLL(sys.argv[1])
lib.Append_rtlib_timing.argtypes = [C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint64]
for event, ident, nsec, sub in eval(sys.argv[2]):
    lib.Append_rtlib_timing(event, ident, nsec, sub)
lib.Report_rtlib_timing()
"""

SEQUENCES = [
    # (event number, id, nanoseconds, nested nanoseconds): NN_CONV twice, FHE_ADDCC, FHE_RESCALE, a bootstrap with
    # nested time, MAIN_GRAPH, the library's bootstrap events at levels 1 to 3, PT_GET
    [(5, 0, 1500000000, 0), (5, 1, 500000000, 0), (12, 0, 1000, 0), (19, 0, 123456789, 0),
     (14, 0, 2000000000, 500000000), (29, 0, 9000000000, 0), (52, 0, 2000000000, 0), (55, 0, 1900000000, 0),
     (58, 0, 600000000, 0), (59, 0, 900000000, 0), (62, 0, 1000, 0)],
    [(29, 0, 1000000, 0)],
    [(1, 0, 5, 0), (10, 0, 7, 0), (21, 0, 9, 0), (22, 0, 11, 0)],
    [(e, 0, 1000 * (e + 1), 0) for e in range(63)],
    [],
]


def _table(lib, seq, out):
    env = dict(os.environ, RTLIB_TIMING_OUTPUT=out)
    r = subprocess.run([sys.executable, "-c", CHILD, lib, repr(seq)], capture_output=True, text=True, env=env, timeout=60)
    assert r.returncode == 0, r.stderr
    return r.stdout, r.stderr


@pytest.mark.parametrize("k", range(len(SEQUENCES)))
def test_same_table_as_the_reference(k):
    assert _table(REF, SEQUENCES[k], "stdout") == _table(OURS, SEQUENCES[k], "stdout")
    assert _table(REF, SEQUENCES[k], "stderr") == _table(OURS, SEQUENCES[k], "stderr")


def test_nothing_without_the_variable():
    env = {k: v for k, v in os.environ.items() if k != "RTLIB_TIMING_OUTPUT"}
    r = subprocess.run([sys.executable, "-c", CHILD, OURS, repr(SEQUENCES[0])], capture_output=True, text=True, env=env, timeout=60)
    assert r.returncode == 0 and r.stdout == "" and r.stderr == ""
