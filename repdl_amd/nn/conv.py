"""The names of RepDL's ``repdl/nn/conv.py`` (``Conv2dFunction`` :11-50, ``conv2d`` :53-76, ``Conv2d`` :105-107):
the implementations live in ``functional.py`` and ``modules.py``."""
from .functional import _Conv2d as Conv2dFunction, conv2d
from .modules import Conv2d

__all__ = ["Conv2dFunction", "conv2d", "Conv2d"]
