"""Reproducible operators -- the API of RepDL's ``repdl/ops.py:12-157`` served by
the MI355X backend.

Same names, argument order and meaning as the reference.  The reference picks
``backend.cuda`` or ``backend.cpu`` from ``tensor.is_cuda``; here every operator
goes to ``repdl_amd.backend.hip`` and a tensor that is not on the GPU is an
error -- there is no CPU implementation in this package.  ``div`` and ``sqrt``,
which the reference composes from PyTorch calls (``ops.py:98-103, 122-123``), are
HIP kernels with the same IEEE results.  ``exp``, ``log`` (the reference's
internal ``exp2d`` / ``log1d``, ``backend/cpu/math.cpp:14-47``) and ``sum`` are
added as public operators.
"""
from __future__ import annotations

from typing import Optional, Sequence, Union

import torch

from .backend import hip as _hip


def _backend(t: torch.Tensor):
    """The backend module that serves tensor ``t``."""
    if not t.is_cuda:
        raise RuntimeError(
            "repdl_amd.ops: tensor is on %s; this package only implements the GPU (HIP) backend" % t.device
        )
    return _hip


def mm(input: torch.Tensor, mat2: torch.Tensor, transA: bool = False, transB: bool = False) -> torch.Tensor:
    return _backend(input).mm(input, mat2, transA, transB)


def mm_bias(input: torch.Tensor, mat2: torch.Tensor, bias: Optional[torch.Tensor], transA: bool = False,
            transB: bool = False) -> torch.Tensor:
    """``mm(...)`` followed by ``+= bias`` over the rows (the reference's linear layer,
    nn/linear.py:21-22), the one rounded addition made where the chain ends instead of in a
    second pass.  Not in the reference's ``ops``."""
    return _backend(input).mm_bias(input, mat2, bias, transA, transB)


def conv2d(input: torch.Tensor, weight: torch.Tensor, stride: Sequence[int], padding: Sequence[int],
           groups: int) -> torch.Tensor:
    sh, sw = stride
    ph, pw = padding
    return _backend(input).conv2d(input, weight, sh, sw, ph, pw, groups)


def conv2d_bias(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], stride: Sequence[int],
                padding: Sequence[int], groups: int) -> torch.Tensor:
    """``conv2d(...)`` followed by ``+= bias`` per output channel (nn/conv.py:27-28), the
    addition made in the kernel's epilogue.  Not in the reference's ``ops``."""
    sh, sw = stride
    ph, pw = padding
    return _backend(input).conv2d_bias(input, weight, bias, sh, sw, ph, pw, groups)


def conv2d_grad_input(input_shape: Sequence[int], weight: torch.Tensor, grad_output: torch.Tensor,
                      stride: Sequence[int], padding: Sequence[int]) -> torch.Tensor:
    # the backend takes grad_output first and only H, W of the input shape
    # (reference ops.py:36-46)
    return _backend(grad_output).conv2d_grad_input(
        grad_output, weight, input_shape[2], input_shape[3], stride[0], stride[1], padding[0], padding[1])


def conv2d_grad_kernel(input: torch.Tensor, weight_shape: Sequence[int], grad_output: torch.Tensor,
                       stride: Sequence[int], padding: Sequence[int]) -> torch.Tensor:
    return _backend(input).conv2d_grad_kernel(
        grad_output, input, weight_shape[2], weight_shape[3], stride[0], stride[1], padding[0], padding[1])


def cross_entropy(input: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
    return _backend(input).cross_entropy(input, target)


def softmax(input: torch.Tensor) -> torch.Tensor:
    return _backend(input).softmax(input)


def div(input: torch.Tensor, other: Union[torch.Tensor, float]) -> torch.Tensor:
    """True IEEE division.  A Python number is rounded to float32 first, exactly
    as the reference's 0-dim float32 tensor is (ops.py:103)."""
    be = _backend(input)
    if isinstance(other, torch.Tensor):
        if other.dim() == 0:
            return be.div_scalar(input, float(other.to(torch.float32)))
        return be.div(input, other.to(input.device))
    return be.div_scalar(input, float(other))


def sqrt(input: torch.Tensor) -> torch.Tensor:
    return _backend(input).sqrt(input)


def exp(input: torch.Tensor) -> torch.Tensor:
    return _backend(input).exp(input)


def log(input: torch.Tensor) -> torch.Tensor:
    return _backend(input).log(input)


def sum1d(input: torch.Tensor, average: bool = False) -> torch.Tensor:
    return _backend(input).sum1d(input, average)


def sum2d_dim0(input: torch.Tensor, keepdim: bool = False, average: bool = False) -> torch.Tensor:
    return _backend(input).sum2d_dim0(input, keepdim, average)


def sum2d_dim1(input: torch.Tensor, keepdim: bool = False, average: bool = False) -> torch.Tensor:
    return _backend(input).sum2d_dim1(input, keepdim, average)


def sum4d_dim023(input: torch.Tensor, keepdim: bool = False, average: bool = False) -> torch.Tensor:
    return _backend(input).sum4d_dim023(input, keepdim, average)


def sum(input: torch.Tensor, dim=None, keepdim: bool = False, average: bool = False) -> torch.Tensor:
    """Sequential-order sum: picks the reference operator that matches the shape.

    1-D (dim None or 0) -> sum1d; 2-D with dim 0 / 1 (or -1) -> sum2d_dim0 / sum2d_dim1;
    4-D with dim (0, 2, 3) -> sum4d_dim023."""
    nd = input.dim()
    if nd == 1 and dim in (None, 0, -1, (0,)):
        return sum1d(input, average)
    if nd == 2 and dim in (0, -2, (0,)):
        return sum2d_dim0(input, keepdim, average)
    if nd == 2 and dim in (1, -1, (1,)):
        return sum2d_dim1(input, keepdim, average)
    if nd == 4 and dim is not None and tuple(dim) == (0, 2, 3):
        return sum4d_dim023(input, keepdim, average)
    raise NotImplementedError("sum over dim=%r of a %d-D tensor has no reproducible operator" % (dim, nd))


def bn_apply(input: torch.Tensor, mean: torch.Tensor, std: torch.Tensor, weight: torch.Tensor,
             bias: torch.Tensor) -> torch.Tensor:
    """``((input - mean) / std) * weight + bias`` with the per-channel vectors broadcast over a
    [N,C,H,W] or [B,F] input: the four rounded operations of the reference's forward
    (nn/batchnorm.py:25-32) in one pass.  Not in the reference's ``ops``."""
    return _backend(input).bn_apply(input, mean, std, weight, bias)


def bn_gvar_term(grad_output: torch.Tensor, input: torch.Tensor, mean: torch.Tensor, coef: torch.Tensor) -> torch.Tensor:
    """``(grad_output * (mean - input)) * coef``: the tensor that grad_var sums (nn/batchnorm.py:56-58)."""
    return _backend(input).bn_gvar_term(grad_output, input, mean, coef)


def bn_gweight_term(input: torch.Tensor, mean: torch.Tensor, std: torch.Tensor, grad_output: torch.Tensor) -> torch.Tensor:
    """``((input - mean) / std) * grad_output``: the tensor that grad_weight sums (nn/batchnorm.py:60-61)."""
    return _backend(input).bn_gweight_term(input, mean, std, grad_output)
