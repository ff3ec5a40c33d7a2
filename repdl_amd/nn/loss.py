"""The names of RepDL's ``repdl/nn/loss.py`` (``CrossEntropyFunction`` :11-34, ``cross_entropy`` :37-58,
``CrossEntropyLoss`` :61-63): the implementations live in ``functional.py`` and ``modules.py``."""
from .functional import _CrossEntropy as CrossEntropyFunction, cross_entropy
from .modules import CrossEntropyLoss

__all__ = ["CrossEntropyFunction", "cross_entropy", "CrossEntropyLoss"]
