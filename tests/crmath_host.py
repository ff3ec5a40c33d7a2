"""Builds (gcc) and loads the CPU build of the device math, tests/crmath_check.c."""
from __future__ import annotations

import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libcrmcheck.so")
_lib = None

U32, U64, INT, P = ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int, ctypes.c_void_p


def build() -> str:
    src = os.path.join(_HERE, "crmath_check.c")
    deps = [src] + [os.path.join(_HERE, "..", "repdl_amd", "csrc", f) for f in ("crmath.h", "crmath_tables.h")]
    if os.path.exists(_SO) and all(os.path.getmtime(_SO) >= os.path.getmtime(d) for d in deps):
        return _SO
    os.makedirs(os.path.dirname(_SO), exist_ok=True)
    subprocess.run(
        ["gcc", "-std=gnu11", "-O2", "-fopenmp", "-ffp-contract=off", "-fno-fast-math", "-mfma", "-shared", "-fPIC",
         "-fvisibility=hidden", "-o", _SO, src, "-lm"], check=True)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        L = ctypes.CDLL(build())
        for n in ("crmc_sweep_exp", "crmc_sweep_log", "crmc_sweep_sqrt"):
            f = getattr(L, n)
            f.restype, f.argtypes = U64, [U32, U64, U32, P, INT]
        L.crmc_sweep_div_by.restype, L.crmc_sweep_div_by.argtypes = U64, [U32, U32, U64, U32, P, INT]
        L.crmc_sweep_div_random.restype, L.crmc_sweep_div_random.argtypes = U64, [U64, U64, INT, P, INT]
        for n in ("crmc_exp", "crmc_log", "crmc_sqrt", "crmc_ref_exp", "crmc_ref_log", "crmc_ref_sqrt"):
            f = getattr(L, n)
            f.restype, f.argtypes = U32, [U32]
        for n in ("crmc_div", "crmc_ref_div"):
            f = getattr(L, n)
            f.restype, f.argtypes = U32, [U32, U32]
        _lib = L
    return _lib
