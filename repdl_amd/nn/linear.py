"""The names of RepDL's ``repdl/nn/linear.py`` (``LinearFunction`` :11-38, ``linear`` :41-49, ``Linear`` :52-54):
the implementations live in ``functional.py`` and ``modules.py``."""
from .functional import _Linear as LinearFunction, linear
from .modules import Linear

__all__ = ["LinearFunction", "linear", "Linear"]
