"""repdl_amd -- RepDL's reproducible operators on AMD MI355X (gfx950).

The package mirrors the layout of RepDL's ``repdl`` package (``ops``, ``func``,
``nn``, ``optim``, ``utils``, ``from_torch_module``); every operator runs in
hand-written HIP kernels behind a C ABI (``include/repdl_hip.h``) and returns
results that are bit-identical to RepDL's CPU backend.
"""
from __future__ import annotations

from copy import copy

import torch

from . import func, nn, ops, optim, utils

__all__ = ["func", "nn", "ops", "optim", "utils", "from_torch_module", "init"]
__version__ = "0.1.0"


def init() -> None:
    """Runs the library's one-time device check (are the matrix instructions chains of single-rounding FMAs on
    this GPU?) for the current device now, instead of inside the first GEMM-shaped call.  Importing the package
    touches no device, so a launcher may still re-launch itself after the import; a program that captures graphs
    calls this before its first capture (the check cannot run under capture, and calls made before it has run
    take the slower ``v_fma_f32`` kernels -- same bits)."""
    from . import _lib

    _lib.init()


def _bn_args(m):
    return (m.num_features, m.eps, m.momentum, m.weight is not None, m.track_running_stats)


def from_torch_module(m: torch.nn.Module) -> torch.nn.Module:
    """Return a copy of ``m`` in which every ``torch.nn`` layer that has a
    reproducible counterpart is replaced by it, weights included.

    Same rules as RepDL's ``repdl/__init__.py:15-65``: the match is on the exact
    type (subclasses are left alone); ``Sequential`` is rebuilt; any other module
    is shallow-copied and its children converted recursively."""
    if not isinstance(m, torch.nn.Module):
        raise TypeError("from_torch_module expects a torch.nn.Module")
    kind = type(m)
    if kind is torch.nn.Sequential:
        return torch.nn.Sequential(*[from_torch_module(child) for child in m])
    if kind is torch.nn.CrossEntropyLoss:
        return nn.CrossEntropyLoss(m.weight, None, m.ignore_index, None, m.reduction, m.label_smoothing)
    if kind is torch.nn.Linear:
        new = nn.Linear(m.in_features, m.out_features, m.bias is not None)
    elif kind is torch.nn.Conv2d:
        new = nn.Conv2d(m.in_channels, m.out_channels, m.kernel_size, m.stride, m.padding, m.dilation, m.groups,
                        m.bias is not None, m.padding_mode)
    elif kind is torch.nn.BatchNorm1d:
        new = nn.BatchNorm1d(*_bn_args(m))
    elif kind is torch.nn.BatchNorm2d:
        new = nn.BatchNorm2d(*_bn_args(m))
    else:
        new = copy(m)
        for name, child in m.named_children():
            setattr(new, name, from_torch_module(child))
        return new
    new.load_state_dict(m.state_dict())
    return new
