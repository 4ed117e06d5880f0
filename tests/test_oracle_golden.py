"""Oracle vs. the committed golden fixtures (outputs of the reference's own compiled code)."""
import pytest

import golden_replay
from oracle_lib import Oracle


@pytest.mark.parametrize("name", ["small", "gemm", "headline"])
def test_oracle_matches_reference_fixtures(name):
    meta, vec = golden_replay.load()
    o = Oracle(*meta[name]["cfg"])
    golden_replay.check(o, name, meta, vec)
    o.close()
