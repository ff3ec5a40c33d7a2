"""Test helper: the HIP backend behind an adaptor that accepts CPU tensors, moves
them to cuda:0, calls ``repdl_amd.backend.hip`` and brings the result back, so
that the golden-case runner can treat it like any other backend module."""
from __future__ import annotations

import torch

from repdl_amd.backend import hip


class _Adaptor:
    def __init__(self, binding=None):
        self._binding = binding  # None: whatever repdl_amd.backend.hip currently serves

    def __getattr__(self, name):
        if self._binding == "ext":
            from repdl_amd.backend import _hip_ext as mod
        elif self._binding == "ctypes":
            from repdl_amd.backend import hip_ctypes as mod
        else:
            mod = hip
        fn = getattr(mod, name)

        def call(*args):
            moved = [a.cuda() if isinstance(a, torch.Tensor) else a for a in args]
            out = fn(*moved)
            torch.cuda.synchronize()
            return out.cpu()

        return call


backend = _Adaptor()
ext_backend = _Adaptor("ext")
ctypes_backend = _Adaptor("ctypes")
