"""GPU parity: every golden case (digests written by RepDL's own C++ CPU backend)
must be reproduced bit for bit by the HIP backend through the C ABI, and must
also equal the C oracle run on the same inputs."""
import pytest
import torch

import cases
import gen
from oracle import api as oracle

pytestmark = pytest.mark.gpu


GEMM_SHAPED = ("mm", "conv2d")


@pytest.mark.parametrize("case", cases.CASES, ids=[c["name"] for c in cases.CASES])
def test_hip_matches_reference_digest(case, golden, matrix_path):
    if matrix_path == "fma" and not case["name"].startswith(GEMM_SHAPED):
        pytest.skip("only one implementation of this operator")
    from hipbackend import backend

    g = golden[case["name"]]
    if "error" in g:
        pytest.skip("the reference rejects this input (%s)" % g["error"])
    print("case", case["name"], flush=True)
    y = cases.run(case, backend)
    assert list(y.shape) == g["shape"]
    assert gen.words(y) == g["words"]
    assert gen.sha256(y) == g["sha256"]
    assert gen.sha256(cases.run(case, oracle)) == g["sha256"]
