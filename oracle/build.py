"""Build recipes for the CHECKERS (test infrastructure, never product code).

``build_oracle()``  compiles ``oracle/repdl_oracle.c`` (the plain-C restatement)
                    into ``oracle/liboracle.so`` with gcc.
``build_ref()``     compiles RepDL's own C++ CPU backend from the sources where
                    they lie under ``/root/reference/backend/cpu`` (g++ on those
                    files directly, against the PyTorch headers of this image)
                    into ``oracle/_ref/repdl_ref_cpu.so``, a CPython extension
                    exporting exactly what ``backend/cpu/bind.cpp:12-18`` binds,
                    plus ``oracle/_ref/repdl_ref_cpu_math.so`` which binds the two
                    helpers the reference declares in ``backend/cpu/math.h:14-15``
                    but never exports to Python (``exp2d``, ``log1d``).
                    No reference source is copied; outputs go to ``oracle/_ref``
                    only (git-ignored).

Run as ``python oracle/build.py [oracle|ref|all]``.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor
from glob import glob

HERE = os.path.dirname(os.path.abspath(__file__))
REF_ROOT = os.environ.get("REPDL_REFERENCE_ROOT", "/root/reference")
REF_CPU = os.path.join(REF_ROOT, "backend", "cpu")
REF_OUT = os.path.join(HERE, "_ref")
ORACLE_SO = os.path.join(HERE, "liboracle.so")


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))


def build_oracle(force: bool = True) -> str:
    src = os.path.join(HERE, "repdl_oracle.c")
    if not force and os.path.exists(ORACLE_SO) and os.path.getmtime(ORACLE_SO) >= os.path.getmtime(src):
        return ORACLE_SO
    # -mavx2 -mfma: fmaf() becomes one vfmadd instruction (still a single
    # rounding); both this container's and the GPU box's host CPUs have them.
    # -ffp-contract=off: nothing else may be fused.
    _run(
        [
            "gcc", "-std=c11", "-O2", "-fopenmp", "-fPIC", "-shared", "-mavx2", "-mfma",
            "-ffp-contract=off", "-fno-fast-math", "-fvisibility=hidden",
            "-o", ORACLE_SO, src, "-lm",
        ]
    )
    return ORACLE_SO


def reference_available() -> bool:
    return os.path.isdir(REF_CPU) and len(glob(os.path.join(REF_CPU, "*.cpp"))) > 0


def build_ref(force: bool = True) -> str | None:
    """g++ on the reference's own backend/cpu/*.cpp; returns the module path."""
    if not reference_available():
        return None
    from torch.utils import cpp_extension  # headers + library dirs of this image's torch

    os.makedirs(REF_OUT, exist_ok=True)
    out_main = os.path.join(REF_OUT, "repdl_ref_cpu.so")
    out_math = os.path.join(REF_OUT, "repdl_ref_cpu_math.so")
    if not force and os.path.exists(out_main) and os.path.exists(out_math):
        return out_main
    incs = cpp_extension.include_paths() + [sysconfig.get_paths()["include"]]
    libdirs = cpp_extension.library_paths()
    common = ["g++", "-O2", "-fopenmp", "-fPIC", "-std=c++17", "-DTORCH_API_INCLUDE_EXTENSION_H"]
    for i in incs:
        common += ["-isystem", i]
    objdir = os.path.join(REF_OUT, "obj")
    os.makedirs(objdir, exist_ok=True)

    jobs = []
    main_objs = []
    for src in sorted(glob(os.path.join(REF_CPU, "*.cpp"))):
        obj = os.path.join(objdir, os.path.basename(src)[:-4] + ".o")
        main_objs.append(obj)
        jobs.append(common + ["-DTORCH_EXTENSION_NAME=repdl_ref_cpu", "-c", src, "-o", obj])
    bind_obj = os.path.join(objdir, "ref_math_bind.o")
    jobs.append(
        common
        + ["-DTORCH_EXTENSION_NAME=repdl_ref_cpu_math", "-I", REF_CPU, "-c",
           os.path.join(HERE, "ref_math_bind.cpp"), "-o", bind_obj]
    )
    with ThreadPoolExecutor(max_workers=4) as ex:
        list(ex.map(_run, jobs))

    link = ["-shared", "-fopenmp"]
    for d in libdirs:
        link += ["-L" + d, "-Wl,-rpath," + d]
    link += ["-lc10", "-ltorch", "-ltorch_cpu", "-ltorch_python"]
    _run(["g++"] + main_objs + link + ["-o", out_main])
    _run(["g++", bind_obj, os.path.join(objdir, "math.o")] + link + ["-o", out_math])
    shutil.rmtree(objdir, ignore_errors=True)
    return out_main


if __name__ == "__main__":
    what = sys.argv[1] if len(sys.argv) > 1 else "all"
    if what in ("oracle", "all"):
        print(build_oracle())
    if what in ("ref", "all"):
        print(build_ref())
