"""Loader for RepDL's own C++ CPU backend compiled into ``oracle/_ref``.

``load()`` returns ``(cpu, cpu_math)``: ``cpu`` has the ten functions that
``backend/cpu/bind.cpp:12-18`` binds, ``cpu_math`` has ``exp2d`` and ``log1d``
(``backend/cpu/math.h:14-15``).  Returns ``None`` when the build is absent.
"""
from __future__ import annotations

import importlib.util
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_cache = None


def _load_one(name: str):
    path = os.path.join(_HERE, "_ref", name + ".so")
    if not os.path.exists(path):
        return None
    import torch  # noqa: F401  (libtorch must be loaded before the extension)

    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def load():
    global _cache
    if _cache is None:
        cpu = _load_one("repdl_ref_cpu")
        cpu_math = _load_one("repdl_ref_cpu_math")
        if cpu is None or cpu_math is None:
            return None
        _cache = (cpu, cpu_math)
    return _cache
