import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__)), os.path.join(ROOT, "tests", "golden")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    import json

    with open(os.path.join(ROOT, "tests", "golden", "golden.json")) as f:
        return json.load(f)


@pytest.fixture(params=["matrix", "fma"])
def matrix_path(request):
    """Runs a GPU test twice: on the matrix-instruction kernels (chosen by the library's own
    check of the device, which must pass on an MI355X) and on the v_fma_f32 kernels."""
    from repdl_amd import _lib

    _lib.call("repdl_hip_set_matrix_path", -1 if request.param == "matrix" else 0)
    assert _lib.lib().repdl_hip_matrix_path() == (1 if request.param == "matrix" else 0)
    yield request.param
    _lib.call("repdl_hip_set_matrix_path", -1)
