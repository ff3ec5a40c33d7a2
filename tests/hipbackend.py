"""Test helper: the HIP backend behind an adaptor that accepts CPU tensors, moves
them to cuda:0, calls ``repdl_amd.backend.hip`` and brings the result back, so
that the golden-case runner can treat it like any other backend module."""
from __future__ import annotations

import torch

from repdl_amd.backend import hip


class _Adaptor:
    def __getattr__(self, name):
        fn = getattr(hip, name)

        def call(*args):
            moved = [a.cuda() if isinstance(a, torch.Tensor) else a for a in args]
            out = fn(*moved)
            torch.cuda.synchronize()
            return out.cpu()

        return call


backend = _Adaptor()
