"""The C oracle must reproduce every golden digest written by RepDL's own C++
CPU backend (tests/golden/golden.json), bit for bit."""
import pytest

import cases
import gen
from oracle import api as oracle


@pytest.mark.parametrize("case", cases.CASES, ids=[c["name"] for c in cases.CASES])
def test_oracle_matches_reference_digest(case, golden):
    g = golden[case["name"]]
    if "error" in g:
        pytest.skip("the reference rejects this input (%s)" % g["error"])
    y = cases.run(case, oracle)
    assert list(y.shape) == g["shape"]
    assert gen.words(y) == g["words"]
    assert gen.sha256(y) == g["sha256"]
