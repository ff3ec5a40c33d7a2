"""ctypes binding of the C-ABI library ``librepdl_hip.so`` (include/repdl_hip.h).

There is no fallback: if the library has not been built, or a call fails, an
exception is raised.  PyTorch is used only for device memory and the current
stream.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "librepdl_hip.so")

_P = ctypes.c_void_p
_I64 = ctypes.c_int64
_INT = ctypes.c_int
_F32 = ctypes.c_float



class AdamTensor(ctypes.Structure):
    """repdl_adam_tensor of repdl_hip.h"""

    _fields_ = [("param", _P), ("grad", _P), ("exp_avg", _P), ("exp_avg_sq", _P), ("max_exp_avg_sq", _P),
                ("n", _I64), ("sqrt_bias_correction2", _F32), ("step_scale", _F32)]


class SgdTensor(ctypes.Structure):
    """repdl_sgd_tensor of repdl_hip.h"""

    _fields_ = [("param", _P), ("grad", _P), ("n", _I64)]


# name -> argument types (all return int), exactly the declarations of repdl_hip.h
SIGNATURES = {
    "repdl_hip_mm": [_P, _P, _P, _I64, _I64, _I64, _INT, _INT, _P],
    "repdl_hip_mm_bias": [_P, _P, _P, _P, _I64, _I64, _I64, _INT, _INT, _P],
    "repdl_hip_conv2d": [_P, _P, _P] + [_I64] * 12 + [_P],
    "repdl_hip_conv2d_bias": [_P, _P, _P, _P] + [_I64] * 12 + [_P],
    "repdl_hip_conv2d_grad_input": [_P, _P, _P] + [_I64] * 13 + [_P],
    "repdl_hip_conv2d_grad_kernel": [_P, _P, _P] + [_I64] * 13 + [_P],
    "repdl_hip_conv2d_ws": [_P, _P, _P, _P] + [_I64] * 12 + [_P, ctypes.c_size_t, _P],
    "repdl_hip_conv2d_grad_input_ws": [_P, _P, _P] + [_I64] * 13 + [_P, ctypes.c_size_t, _P],
    "repdl_hip_conv2d_grad_kernel_ws": [_P, _P, _P] + [_I64] * 13 + [_P, ctypes.c_size_t, _P],
    "repdl_hip_sum1d": [_P, _P, _I64, _INT, _P],
    "repdl_hip_sum1d_ws": [_P, _P, _I64, _INT, _P, ctypes.c_size_t, _P],
    "repdl_hip_sum1d_static": [_P, _P, _I64, _INT, _P],
    "repdl_hip_sum2d_dim0": [_P, _P, _I64, _I64, _INT, _P],
    "repdl_hip_sum2d_dim1": [_P, _P, _I64, _I64, _INT, _P],
    "repdl_hip_sum4d_dim023": [_P, _P, _I64, _I64, _I64, _I64, _INT, _P],
    "repdl_hip_sum2d_dim1_ws": [_P, _P, _I64, _I64, _INT, _P, ctypes.c_size_t, _P],
    "repdl_hip_sum4d_dim023_ws": [_P, _P, _I64, _I64, _I64, _I64, _INT, _P, ctypes.c_size_t, _P],
    "repdl_hip_exp": [_P, _P, _I64, _P],
    "repdl_hip_log": [_P, _P, _I64, _P],
    "repdl_hip_sqrt": [_P, _P, _I64, _P],
    "repdl_hip_div": [_P, _P, _P, _I64, _P],
    "repdl_hip_div_scalar": [_P, _F32, _P, _I64, _P],
    "repdl_hip_softmax": [_P, _P, _I64, _I64, _P],
    "repdl_hip_cross_entropy": [_P, _P, _P, _I64, _I64, _P, _P],
    "repdl_hip_cross_entropy_ws": [_P, _P, _P, _I64, _I64, _P, ctypes.c_size_t, _P],
    "repdl_hip_bn_apply": [_P] * 6 + [_I64] * 3 + [_P],
    "repdl_hip_bn_gvar_term": [_P] * 5 + [_I64] * 3 + [_P],
    "repdl_hip_bn_gweight_term": [_P] * 5 + [_I64] * 3 + [_P],
    "repdl_hip_adam_step": [ctypes.POINTER(AdamTensor), _INT] + [_F32] * 6 + [_P],
    "repdl_hip_sgd_step": [ctypes.POINTER(SgdTensor), _INT, _F32, _P],
    "repdl_hip_mfma_selftest": [_I64, _I64, ctypes.c_uint64, ctypes.POINTER(ctypes.c_uint64)],
    "repdl_hip_set_matrix_path": [_INT],
    "repdl_hip_scratch_trim": [],
}

# name -> argument types of the workspace-size queries (all return size_t)
SIZE_QUERIES = {
    "repdl_hip_sum1d_workspace_bytes": [_I64],
    "repdl_hip_conv2d_workspace_bytes": [_P, _P] + [_I64] * 12,
    "repdl_hip_conv2d_grad_input_workspace_bytes": [_P, _P] + [_I64] * 13,
    "repdl_hip_conv2d_grad_kernel_workspace_bytes": [_P, _P] + [_I64] * 13,
    "repdl_hip_sum2d_dim1_workspace_bytes": [_I64, _I64],
    "repdl_hip_sum4d_dim023_workspace_bytes": [_I64] * 4,
    "repdl_hip_cross_entropy_workspace_bytes": [_I64, _I64],
    "repdl_hip_scratch_bytes": [],
}

_lib = None


class RepdlHipError(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """Load the library (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RepdlHipError(
                "%s is missing: build it with `python -m repdl_amd.build` (there is no CPU fallback)" % LIB_PATH
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = _INT
        handle.repdl_hip_error_string.argtypes = [_INT]
        handle.repdl_hip_error_string.restype = ctypes.c_char_p
        for name, argtypes in SIZE_QUERIES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_size_t
        handle.repdl_hip_matrix_path.argtypes = []
        handle.repdl_hip_matrix_path.restype = _INT
        handle.repdl_hip_abi_version.argtypes = []
        handle.repdl_hip_abi_version.restype = _INT
        handle.repdl_hip_sum1d_static_max_n.argtypes = []
        handle.repdl_hip_sum1d_static_max_n.restype = _I64
        handle.repdl_hip_init.argtypes = []
        handle.repdl_hip_init.restype = _INT
        handle.repdl_hip_routes_taken.argtypes = [_INT]
        handle.repdl_hip_routes_taken.restype = ctypes.c_uint64
        handle.repdl_hip_route_name.argtypes = [_INT]
        handle.repdl_hip_route_name.restype = ctypes.c_char_p
        # Loading touches no device.  The one-time check of the matrix instructions runs inside the first
        # GEMM-shaped call on a device, or in init() below.
        _lib = handle
    return _lib


def init() -> None:
    """Runs the library's one-time check of the matrix instructions for the current device now (otherwise the
    first GEMM-shaped call runs it).  Programs that capture graphs call this before their first capture: the
    check cannot run under capture, and calls made while it has not run take the slower v_fma_f32 kernels."""
    check(lib().repdl_hip_init(), "repdl_hip_init")


def check(code: int, what: str) -> None:
    if code != 0:
        msg = lib().repdl_hip_error_string(code)
        raise RepdlHipError("%s failed with code %d: %s" % (what, code, msg.decode() if msg else "?"))


def call(name: str, *args) -> None:
    check(getattr(lib(), name)(*args), name)
