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
