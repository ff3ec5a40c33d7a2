"""Optimizers whose update is a fixed sequence of individually rounded operations.

``Adam`` follows RepDL's ``repdl/optim.py:56-83``: PyTorch's Adam state and
hyper-parameters, with the denominator computed as
``ops.div(ops.sqrt(v), sqrt(bias_correction2)) + eps`` (reproducible square root
and true division) and the step written as separate multiply and add passes.

``SGD`` is plain stochastic gradient descent written as two rounded operations,
``p -= (lr * g)``: ``Tensor.add_(g, alpha=-lr)`` (what ``torch.optim.SGD`` calls) is
a fused multiply-add on some devices and not on others, which changes the bits.

Parameters on the GPU (float32, contiguous, dense gradients) are updated by the fused
kernels of the C ABI (``repdl_hip_adam_step`` / ``repdl_hip_sgd_step``): the same
operations with the same roundings, evaluated per element in one pass over all the
tensors of a parameter group instead of a dozen launches per parameter.  Any other
parameter goes through the operation sequence itself (``_adam_sequence``), which is
also what the fused kernels are tested against.
"""
from __future__ import annotations

import ctypes
import math

import torch

from . import _lib, ops


FUSED = True  # False: every parameter goes through the operation sequence (for comparisons)


def _fusable(*tensors: torch.Tensor) -> bool:
    dev = tensors[0].device
    return FUSED and all(t.is_cuda and t.device == dev and t.dtype == torch.float32 and t.is_contiguous() and not t.is_sparse
               for t in tensors)


def _by_device(entries):
    """entries: (device, descriptor, keep-alive) -> {device: [descriptor, ...]}"""
    out = {}
    for dev, desc, _ in entries:
        out.setdefault(dev, []).append(desc)
    return out


def _adam_sequence(p, g, m, v, vmax, t, lr, beta1, beta2, eps, wd):
    """repdl/optim.py:56-83 operation by operation."""
    if wd != 0:
        g = g.add(p, alpha=wd)
    m.mul_(beta1).add_(g, alpha=1 - beta1)
    v.mul_(beta2).add_(torch.mul(g, g).mul(1 - beta2))
    second = v
    if vmax is not None:
        torch.maximum(vmax, v, out=vmax)
        second = vmax
    bc1, bc2 = 1 - beta1 ** t, 1 - beta2 ** t
    denom = ops.div(ops.sqrt(second), math.sqrt(bc2)).add_(eps)
    p.add_(ops.div(m, denom).mul(-(lr / bc1)))


class Adam(torch.optim.Adam):
    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            beta1, beta2 = group["betas"]
            lr, eps, wd, amsgrad = group["lr"], group["eps"], group["weight_decay"], group["amsgrad"]
            fused = []
            for p in group["params"]:
                if p.grad is None:
                    continue
                if p.grad.is_sparse:
                    raise RuntimeError("Adam does not support sparse gradients, please consider SparseAdam instead")
                state = self.state[p]
                if len(state) == 0:
                    state["step"] = 0
                    state["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    state["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    if amsgrad:
                        state["max_exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                state["step"] += 1
                # an integer whatever holds the count: after load_state_dict PyTorch keeps it as a float32
                # tensor, and beta ** tensor would compute the bias corrections in binary32
                t = int(state["step"])
                g = p.grad
                m, v = state["exp_avg"], state["exp_avg_sq"]
                vmax = state["max_exp_avg_sq"] if amsgrad else None
                if p.is_cuda and not g.is_contiguous():
                    g = g.contiguous()
                if _fusable(*([p, g, m, v] + ([vmax] if amsgrad else []))):
                    bc1, bc2 = 1 - beta1 ** t, 1 - beta2 ** t
                    desc = _lib.AdamTensor(p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(),
                                           vmax.data_ptr() if amsgrad else None, p.numel(), math.sqrt(bc2),
                                           -(lr / bc1))
                    fused.append((p.device, desc, g))
                else:
                    _adam_sequence(p, g, m, v, vmax, t, lr, beta1, beta2, eps, wd)
            for dev, descs in _by_device(fused).items():
                arr = (_lib.AdamTensor * len(descs))(*descs)
                with torch.cuda.device(dev):
                    _lib.call("repdl_hip_adam_step", arr, len(descs), beta1, 1 - beta1, beta2, 1 - beta2, eps, wd,
                              ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
        return loss


class SGD(torch.optim.Optimizer):
    """p <- p - RN(lr * g): one rounded multiply, one rounded subtract."""

    def __init__(self, params, lr: float = 0.01):
        if lr < 0.0:
            raise ValueError("invalid learning rate: %r" % lr)
        super().__init__(params, dict(lr=lr))

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            lr = group["lr"]
            fused = []
            for p in group["params"]:
                if p.grad is None:
                    continue
                g = p.grad
                if p.is_cuda and not g.is_sparse and not g.is_contiguous():
                    g = g.contiguous()
                if _fusable(p, g):
                    fused.append((p.device, _lib.SgdTensor(p.data_ptr(), g.data_ptr(), p.numel()), g))
                else:
                    p.sub_(g.mul(lr))
            for dev, descs in _by_device(fused).items():
                arr = (_lib.SgdTensor * len(descs))(*descs)
                with torch.cuda.device(dev):
                    _lib.call("repdl_hip_sgd_step", arr, len(descs), lr,
                              ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
        return loss
