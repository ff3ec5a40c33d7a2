"""The matrix instructions against chains of single-rounding FMAs, on the device: the
library's own check (mfma_check.hip) at a length well beyond the one it runs before first
use.  Every result of v_mfma_f32_32x32x2_f32 and v_mfma_f32_16x16x4_f32 must have the bits
of fma(a_{K-1}, b_{K-1}, ... fma(a_0, b_0, c)) evaluated with __fmaf_rn."""
import ctypes

import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [1, 0xC0FFEE, 2 ** 63 + 12345])
def test_matrix_instructions_are_fma_chains(seed):
    from repdl_amd import _lib

    bad = (ctypes.c_uint64 * 2)(7, 7)
    # 8192 waves x 140 trials: 1.17e9 results of the 32x32x2 instruction, 2.9e8 of the 16x16x4
    _lib.call("repdl_hip_mfma_selftest", 8192, 140, seed, bad)
    assert list(bad) == [0, 0]


def test_library_selects_the_matrix_path():
    from repdl_amd import _lib

    _lib.call("repdl_hip_set_matrix_path", -1)
    assert _lib.lib().repdl_hip_matrix_path() == 1
    _lib.call("repdl_hip_set_matrix_path", 0)
    assert _lib.lib().repdl_hip_matrix_path() == 0
    _lib.call("repdl_hip_set_matrix_path", -1)
    with pytest.raises(_lib.RepdlHipError):
        _lib.call("repdl_hip_set_matrix_path", 5)
    # mode 1 is "the matrix kernels where the device's check passed": it runs the check, never skips it
    _lib.call("repdl_hip_set_matrix_path", 1)
    assert _lib.lib().repdl_hip_matrix_path() == 1
    _lib.call("repdl_hip_set_matrix_path", -1)


_FIRST_CALL = r"""
import ctypes, sys, torch
sys.path.insert(0, {root!r}); sys.path.insert(0, {root!r} + "/tests")
import gen
from oracle import api as oracle
from repdl_amd import _lib
h = ctypes.CDLL(_lib.LIB_PATH)          # the bare library: nothing has run its start-up check
h.repdl_hip_mm.argtypes = _lib.SIGNATURES["repdl_hip_mm"]
a, b = gen.normal_like(1, 256, 200), gen.normal_like(2, 200, 320)
want = oracle.mm(a, b, False, False)
ad, bd = a.cuda(), b.cuda()
cd = torch.empty(256, 320, device="cuda")
busy = torch.randn(8192, 8192, device="cuda")
torch.cuda.synchronize()
side = torch.cuda.Stream()
for _ in range(6):
    busy = busy @ busy * 1e-4           # tens of milliseconds of work pending on the null stream
with torch.cuda.stream(side):
    rc = h.repdl_hip_mm(ad.data_ptr(), bd.data_ptr(), cd.data_ptr(), 256, 320, 200, 0, 0, side.cuda_stream)
    pending = not torch.cuda.default_stream().query()
side.synchronize()
assert rc == 0, rc
assert torch.equal(cd.cpu(), want)
h.repdl_hip_matrix_path.restype = ctypes.c_int
assert h.repdl_hip_matrix_path() == 1
torch.cuda.synchronize()
print("first-call ok, null stream still busy at return:", pending)
"""


def test_first_gemm_on_a_side_stream_in_a_fresh_process():
    """The first GEMM-shaped call of a process, made on a non-default stream while the null stream
    still has work pending: the check of the matrix instructions runs on its own stream, the call
    neither waits for the null stream nor disturbs it, and the result has the oracle's bits."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-c", _FIRST_CALL.format(root=root)], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "first-call ok" in proc.stdout
