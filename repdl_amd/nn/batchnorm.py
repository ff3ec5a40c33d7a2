"""The names of RepDL's ``repdl/nn/batchnorm.py`` (``BatchNormFunction`` :12-66, ``batch_norm`` :67-97,
``BatchNorm1d`` / ``BatchNorm2d`` :127-133): the implementations live in ``functional.py`` and ``modules.py``."""
from .functional import _BatchNorm as BatchNormFunction, batch_norm
from .modules import BatchNorm1d, BatchNorm2d

__all__ = ["BatchNormFunction", "batch_norm", "BatchNorm1d", "BatchNorm2d"]
