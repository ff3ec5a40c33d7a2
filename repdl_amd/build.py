"""Builds ``repdl_amd/librepdl_hip.so`` (the C-ABI library of include/repdl_hip.h)
from ``repdl_amd/csrc/*.hip`` with hipcc for gfx950.

Flags that matter for reproducibility:
  -ffp-contract=off -fno-fast-math   nothing is fused or reassociated except the
                                     explicit fma calls in the sources;
  (default) denormals preserved      hipcc does not flush fp32 denormals on gfx9;
  -packed-fp32-ops disabled          no v_pk_{fma,mul,add}_f32 is generated.
Run as ``python -m repdl_amd.build``.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from glob import glob

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "librepdl_hip.so")
OBJ = os.path.join(HERE, "csrc", "_obj")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
    "-fvisibility=hidden", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))


def sources() -> list[str]:
    return sorted(glob(os.path.join(CSRC, "*.hip")))


def build(verbose: bool = False, incremental: bool = False, extra_flags: tuple = ()) -> str:
    """Compiles every source (incremental=True: only those newer than their object, or older
    than a header) and links the library."""
    os.makedirs(OBJ, exist_ok=True)
    jobs, objs = [], []
    headers = glob(os.path.join(CSRC, "*.h")) + glob(os.path.join(HERE, "..", "include", "*.h"))
    newest_header = max(os.path.getmtime(h) for h in headers)
    for src in sources():
        obj = os.path.join(OBJ, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        if incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), newest_header):
            continue
        jobs.append([HIPCC] + FLAGS + list(extra_flags) + ["-c", src, "-o", obj])
    with ThreadPoolExecutor(max_workers=6) as ex:
        list(ex.map(_run, jobs))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    if verbose:
        print(LIB)
    return LIB


EXT_NAME = "_hip_ext"


def ext_path() -> str:
    import sysconfig

    return os.path.join(HERE, "backend", EXT_NAME + sysconfig.get_config_var("EXT_SUFFIX"))


def build_ext(verbose: bool = False) -> str:
    """Builds ``repdl_amd/backend/_hip_ext``: csrc/bind.cpp, the PyTorch C++ extension module
    with the function list of RepDL's backend/cuda/bind.cpp, over librepdl_hip.so.  Host C++
    only (g++ against the PyTorch and HIP headers); needs build() first."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension as ce

    out = ext_path()
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-DTORCH_EXTENSION_NAME=" + EXT_NAME, "-DTORCH_API_INCLUDE_EXTENSION_H", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), "-Wno-deprecated-declarations"]
    for inc in ce.include_paths() + [sysconfig.get_paths()["include"], "/opt/rocm/include"]:
        cmd += ["-isystem", inc]
    cmd += [os.path.join(CSRC, "bind.cpp"), "-o", out, "-L" + tlib, "-L" + HERE, "-lrepdl_hip", "-lc10", "-lc10_hip",
            "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-ltorch_python", "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath," + tlib]
    _run(cmd)
    if verbose:
        print(out)
    return out


if __name__ == "__main__":
    build(verbose=True, incremental="--incremental" in sys.argv)
    build_ext(verbose=True)
    sys.exit(0)
