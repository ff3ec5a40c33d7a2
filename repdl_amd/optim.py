"""Optimizers whose update is a fixed sequence of individually rounded operations.

``Adam`` follows RepDL's ``repdl/optim.py:56-83``: PyTorch's Adam state and
hyper-parameters, with the denominator computed as
``ops.div(ops.sqrt(v), sqrt(bias_correction2)) + eps`` (reproducible square root
and true division) and the step written as separate multiply and add passes.

``SGD`` is plain stochastic gradient descent written as two rounded operations,
``p -= (lr * g)``: ``Tensor.add_(g, alpha=-lr)`` (what ``torch.optim.SGD`` calls) is
a fused multiply-add on some devices and not on others, which changes the bits.
"""
from __future__ import annotations

import math

import torch

from . import ops


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
                t = state["step"]
                g = p.grad
                if wd != 0:
                    g = g.add(p, alpha=wd)
                m, v = state["exp_avg"], state["exp_avg_sq"]
                m.mul_(beta1).add_(g, alpha=1 - beta1)
                v.mul_(beta2).add_(torch.mul(g, g).mul(1 - beta2))
                second = v
                if amsgrad:
                    torch.maximum(state["max_exp_avg_sq"], v, out=state["max_exp_avg_sq"])
                    second = state["max_exp_avg_sq"]
                bc1, bc2 = 1 - beta1 ** t, 1 - beta2 ** t
                denom = ops.div(ops.sqrt(second), math.sqrt(bc2)).add_(eps)
                p.add_(ops.div(m, denom).mul(-(lr / bc1)))
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
            for p in group["params"]:
                if p.grad is not None:
                    p.sub_(p.grad.mul(lr))
        return loss
