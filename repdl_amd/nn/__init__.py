"""Reproducible ``torch.nn`` layers (RepDL ``repdl/nn/__init__.py:4-8``)."""
from . import functional
from .modules import BatchNorm1d, BatchNorm2d, Conv2d, CrossEntropyLoss, Linear

__all__ = ["functional", "BatchNorm1d", "BatchNorm2d", "Conv2d", "CrossEntropyLoss", "Linear"]
