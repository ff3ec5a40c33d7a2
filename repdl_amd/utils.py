"""Hash helpers with the convention of RepDL's ``repdl/utils.py:10-23``: SHA-256
of the raw little-endian bytes of a tensor, or of all parameters of a module in
``parameters()`` order (buffers excluded)."""
from __future__ import annotations

import hashlib
from typing import Union

import torch


def _raw(t: torch.Tensor) -> bytes:
    return t.detach().cpu().contiguous().numpy().tobytes()


def get_hash(x: Union[torch.Tensor, torch.nn.Module]) -> str:
    h = hashlib.sha256()
    if isinstance(x, torch.Tensor):
        h.update(_raw(x))
    elif isinstance(x, torch.nn.Module):
        for p in x.parameters():
            h.update(_raw(p))
    else:
        raise TypeError("get_hash takes a Tensor or a Module, got %s" % type(x).__name__)
    return h.hexdigest()


def print_hash(x: Union[torch.Tensor, torch.nn.Module]) -> None:
    print(get_hash(x))
