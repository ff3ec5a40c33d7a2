"""``repdl_amd.backend.hip`` -- the module that takes the place of RepDL's compiled
``repdl.backend.cuda`` (backend/cuda/bind.cpp:12-19): the same ten functions with the
same positional signatures, tensors in and a new tensor out, plus the elementwise
operators (``exp``, ``log``, ``sqrt``, ``div``, ``div_scalar``) and ``mm_bias`` /
``conv2d_bias`` (a layer's bias added in the kernel's epilogue) and the fused elementwise
passes of batch normalisation (``bn_apply``, ``bn_gvar_term``, ``bn_gweight_term``).

Two bindings of the one C-ABI library (include/repdl_hip.h) can serve it:

* ``ext``    -- ``_hip_ext``, the PyTorch C++ extension module built from csrc/bind.cpp
               (``python -m repdl_amd.build``), the form the reference's backends have;
* ``ctypes`` -- ``hip_ctypes``, the same functions in Python over ctypes.

The compiled binding is used when it is there.  Either way the kernels are those of
``librepdl_hip.so``; there is no other implementation behind this module.
"""
from __future__ import annotations

from . import hip_ctypes as _ctypes_binding

try:
    from . import _hip_ext as _ext_binding
except ImportError:  # not built
    _ext_binding = None

FUNCTIONS = ("mm", "conv2d", "conv2d_grad_input", "conv2d_grad_kernel", "sum1d", "sum2d_dim0", "sum2d_dim1",
             "sum4d_dim023", "softmax", "cross_entropy", "exp", "log", "sqrt", "div", "div_scalar", "mm_bias", "conv2d_bias",
             "bn_apply", "bn_gvar_term", "bn_gweight_term")
if _ext_binding is not None and not all(hasattr(_ext_binding, fn) for fn in FUNCTIONS):
    import warnings

    warnings.warn("repdl_amd.backend._hip_ext was built from an older csrc/bind.cpp and is ignored; "
                  "rebuild it with `python -m repdl_amd.build`")
    _ext_binding = None
BINDING = None


def use_binding(name: str) -> None:
    """Selects ``"ext"`` or ``"ctypes"`` for every function of this module."""
    global BINDING
    if name == "ext":
        if _ext_binding is None:
            raise RuntimeError("repdl_amd.backend._hip_ext has not been built (python -m repdl_amd.build)")
        src = _ext_binding
    elif name == "ctypes":
        src = _ctypes_binding
    else:
        raise ValueError("binding must be 'ext' or 'ctypes'")
    for fn in FUNCTIONS:
        globals()[fn] = getattr(src, fn)
    BINDING = name


use_binding("ext" if _ext_binding is not None else "ctypes")
