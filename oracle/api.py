"""ctypes front end of ``oracle/repdl_oracle.c`` (test infrastructure only).

Functions take and return torch CPU float32 tensors and use the signatures of
RepDL's backend module (``backend/cpu/bind.cpp:12-18`` and the ``m.def`` lists
in each source), including the output shapes: ``sum1d`` returns a 0-dim tensor,
the other sums return ``[1,N]`` / ``[M,1]`` / ``[1,C,1,1]`` and ``squeeze()``
them unless ``keepdim`` (``backend/cpu/summation.cpp:38, 57, 77``).
"""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None

_I64 = ctypes.c_int64
_P = ctypes.c_void_p


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            from . import build

            build.build_oracle()
        _lib = ctypes.CDLL(path)
        _lib.repdl_oracle_sum1d.restype = ctypes.c_float
        _lib.repdl_oracle_cross_entropy.restype = ctypes.c_float
        _lib.repdl_oracle_threads.restype = ctypes.c_int
        _lib.repdl_oracle_div_scalar.argtypes = [_P, ctypes.c_float, _P, _I64]
        _lib.repdl_oracle_adam_step.argtypes = [_P, _P, _P, _P, _P, _I64] + [ctypes.c_float] * 8
        _lib.repdl_oracle_sgd_step.argtypes = [_P, _P, _I64, ctypes.c_float]
    return _lib


def threads() -> int:
    return int(lib().repdl_oracle_threads())


def _f32(t: torch.Tensor) -> torch.Tensor:
    if t.device.type != "cpu" or t.dtype != torch.float32:
        raise TypeError("oracle takes float32 CPU tensors")
    return t.contiguous()


def _p(t: torch.Tensor) -> _P:
    return _P(t.data_ptr())


def mm(input: torch.Tensor, mat2: torch.Tensor, transA: bool = False, transB: bool = False) -> torch.Tensor:
    a, b = _f32(input), _f32(mat2)
    M, K = (a.shape[0], a.shape[1]) if not transA else (a.shape[1], a.shape[0])
    N = b.shape[1] if not transB else b.shape[0]
    out = torch.empty((M, N), dtype=torch.float32)
    lib().repdl_oracle_mm(_p(a), _p(b), _p(out), _I64(M), _I64(N), _I64(K), int(transA), int(transB))
    return out


def conv2d(input, kernel, sH, sW, pH, pW, groups) -> torch.Tensor:
    x, k = _f32(input), _f32(kernel)
    N, IC, H, W = x.shape
    OC, _, KH, KW = k.shape
    OH, OW = (H + 2 * pH - KH) // sH + 1, (W + 2 * pW - KW) // sW + 1
    out = torch.empty((N, OC, OH, OW), dtype=torch.float32)
    lib().repdl_oracle_conv2d(
        _p(x), _p(k), _p(out), _I64(N), _I64(IC), _I64(H), _I64(W), _I64(OC), _I64(KH), _I64(KW),
        _I64(sH), _I64(sW), _I64(pH), _I64(pW), _I64(groups))
    return out


def conv2d_grad_input(grad_output, kernel, H, W, sH, sW, pH, pW) -> torch.Tensor:
    go, k = _f32(grad_output), _f32(kernel)
    N, OC, OH, OW = go.shape
    _, IC, KH, KW = k.shape
    out = torch.empty((N, IC, H, W), dtype=torch.float32)
    lib().repdl_oracle_conv2d_grad_input(
        _p(go), _p(k), _p(out), _I64(N), _I64(OC), _I64(OH), _I64(OW), _I64(IC), _I64(KH), _I64(KW),
        _I64(H), _I64(W), _I64(sH), _I64(sW), _I64(pH), _I64(pW))
    return out


def conv2d_grad_kernel(grad_output, input, KH, KW, sH, sW, pH, pW) -> torch.Tensor:
    go, x = _f32(grad_output), _f32(input)
    N, IC, H, W = x.shape
    _, OC, OH, OW = go.shape
    out = torch.empty((OC, IC, KH, KW), dtype=torch.float32)
    lib().repdl_oracle_conv2d_grad_kernel(
        _p(go), _p(x), _p(out), _I64(N), _I64(IC), _I64(H), _I64(W), _I64(OC), _I64(OH), _I64(OW),
        _I64(KH), _I64(KW), _I64(sH), _I64(sW), _I64(pH), _I64(pW))
    return out


def sum1d(input, average: bool = False) -> torch.Tensor:
    x = _f32(input)
    return torch.tensor(lib().repdl_oracle_sum1d(_p(x), _I64(x.shape[0]), int(average)), dtype=torch.float32)


def sum2d_dim0(input, keepdim: bool = False, average: bool = False) -> torch.Tensor:
    x = _f32(input)
    M, N = x.shape
    out = torch.empty((1, N), dtype=torch.float32)
    lib().repdl_oracle_sum2d_dim0(_p(x), _p(out), _I64(M), _I64(N), int(average))
    return out if keepdim else out.squeeze()


def sum2d_dim1(input, keepdim: bool = False, average: bool = False) -> torch.Tensor:
    x = _f32(input)
    M, N = x.shape
    out = torch.empty((M, 1), dtype=torch.float32)
    lib().repdl_oracle_sum2d_dim1(_p(x), _p(out), _I64(M), _I64(N), int(average))
    return out if keepdim else out.squeeze()


def sum4d_dim023(input, keepdim: bool = False, average: bool = False) -> torch.Tensor:
    x = _f32(input)
    N, C, H, W = x.shape
    out = torch.empty((1, C, 1, 1), dtype=torch.float32)
    lib().repdl_oracle_sum4d_dim023(_p(x), _p(out), _I64(N), _I64(C), _I64(H), _I64(W), int(average))
    return out if keepdim else out.squeeze()


def _unary(name: str, input: torch.Tensor) -> torch.Tensor:
    x = _f32(input)
    out = torch.empty_like(x)
    getattr(lib(), name)(_p(x), _p(out), _I64(x.numel()))
    return out


def exp(input):
    return _unary("repdl_oracle_exp", input)


def log(input):
    return _unary("repdl_oracle_log", input)


def sqrt(input):
    return _unary("repdl_oracle_sqrt", input)


def div(input, other) -> torch.Tensor:
    x = _f32(input)
    out = torch.empty_like(x)
    if isinstance(other, torch.Tensor) and other.dim() > 0:
        y = _f32(other)
        if y.shape != x.shape:
            y = y.expand_as(x).contiguous()
        lib().repdl_oracle_div(_p(x), _p(y), _p(out), _I64(x.numel()))
    else:
        b = float(torch.tensor(float(other), dtype=torch.float32))
        lib().repdl_oracle_div_scalar(_p(x), ctypes.c_float(b), _p(out), _I64(x.numel()))
    return out


def softmax(input) -> torch.Tensor:
    x = _f32(input)
    out = torch.empty_like(x)
    lib().repdl_oracle_softmax(_p(x), _p(out), _I64(x.shape[0]), _I64(x.shape[1]))
    return out


def cross_entropy(input, target) -> torch.Tensor:
    x = _f32(input)
    t = target.to(torch.int64).contiguous()
    scratch = torch.empty(x.shape[0], dtype=torch.float32)
    v = lib().repdl_oracle_cross_entropy(_p(x), _p(t), _I64(x.shape[0]), _I64(x.shape[1]), _p(scratch))
    return torch.tensor(v, dtype=torch.float32)


def adam_step(param, grad, exp_avg, exp_avg_sq, max_exp_avg_sq, step, lr, betas, eps, weight_decay) -> None:
    """One Adam update of one tensor, in place (repdl/optim.py:56-83); ``step`` is the
    count after the increment; ``max_exp_avg_sq`` None = amsgrad off.  The scalars are
    computed in binary64 as the Python code does and rounded to binary32 once."""
    import math

    beta1, beta2 = betas
    for t in (param, exp_avg, exp_avg_sq, max_exp_avg_sq):
        if t is not None and (t.device.type != "cpu" or t.dtype != torch.float32 or not t.is_contiguous()):
            raise TypeError("oracle updates contiguous float32 CPU tensors in place")
    g = _f32(grad)
    bc1, bc2 = 1 - beta1 ** step, 1 - beta2 ** step
    lib().repdl_oracle_adam_step(
        _p(param), _p(g), _p(exp_avg), _p(exp_avg_sq), _p(max_exp_avg_sq) if max_exp_avg_sq is not None else None,
        _I64(param.numel()), beta1, 1 - beta1, beta2, 1 - beta2, eps, weight_decay, math.sqrt(bc2), -(lr / bc1))


def sgd_step(param, grad, lr) -> None:
    if param.device.type != "cpu" or param.dtype != torch.float32 or not param.is_contiguous():
        raise TypeError("oracle updates contiguous float32 CPU tensors in place")
    lib().repdl_oracle_sgd_step(_p(param), _p(_f32(grad)), _I64(param.numel()), lr)
