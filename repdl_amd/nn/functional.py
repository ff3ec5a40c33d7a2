"""Functional layer API with reproducible forward and backward passes -- the
counterpart of RepDL's ``repdl/nn/functional.py`` (``linear``, ``conv2d``,
``cross_entropy``, ``batch_norm``) and of the autograd Functions behind it
(``repdl/nn/linear.py:11-38``, ``conv.py:11-50``, ``loss.py:11-34``,
``batchnorm.py:12-66``).  Every tensor contraction, reduction, division and
square root goes through ``repdl_amd.ops``; which operator is called, in which
order, and which updates are in place follows the reference.
"""
from __future__ import annotations

from typing import Optional, Tuple, Union

import torch

from .. import func, ops

_Pair = Union[int, Tuple[int, int]]


class _Linear(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight)
        return ops.mm_bias(x, weight, bias, transB=True)  # x [B,in] . W[out,in]^T, then + bias

    @staticmethod
    def backward(ctx, gy):
        x, weight = ctx.saved_tensors
        need_x, need_w, need_b = ctx.needs_input_grad
        gx = ops.mm(gy, weight) if need_x else None
        gw = ops.mm(gy, x, transA=True) if need_w else None  # gy^T . x, the batch is K
        gb = ops.sum2d_dim0(gy) if need_b else None
        return gx, gw, gb


def linear(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    if input.dim() != 2:
        raise NotImplementedError("linear: only 2-D input is supported")
    assert weight.dim() == 2
    assert bias is None or bias.dim() == 1
    return _Linear.apply(input, weight, bias)


_SIDE_STREAMS = {}
_DEFER_STREAMS = {}
_DEFERRED = {}
_DEFER_POOL = 3  # side streams that deferred jobs rotate over (with the current stream: the four hardware queues of a process)
defer_parameter_gradients = True  # False: every job of _side_by_side is joined where it was started
deferred_stats = {"jobs": 0, "copies_rewritten": 0}  # (for tests: how often each path was taken)


def _deferrable(param: Optional[torch.Tensor]) -> bool:
    """Whether the gradient of `param` may still be in flight on a side stream when the backward
    function that made it returns.  It may if nothing reads it before the backward pass ends: the
    tensor is a leaf without hooks whose .grad is empty -- autograd then keeps the gradient tensor
    itself, or a copy that _join_deferred() makes again once the gradient is complete -- and no
    graph is being recorded through the backward pass.  Code that reads parameter gradients DURING
    the backward pass by other means (hooks on autograd nodes) sets defer_parameter_gradients = False."""
    return (defer_parameter_gradients and param is not None and param.is_leaf and param.grad is None
            and param.is_contiguous() and not torch.is_grad_enabled() and not param._backward_hooks
            and not getattr(param, "_post_accumulate_grad_hooks", None))


def _join_deferred(key: int) -> None:
    """End of a backward pass: the current stream waits for the deferred jobs, and a parameter whose
    .grad is not the job's own tensor (autograd copied it, possibly before it was complete) gets
    the finished values."""
    pending = _DEFERRED.pop(key, None)
    if pending is None:
        return
    cur = torch.cuda.current_stream(key)
    for st in pending["streams"]:
        cur.wait_stream(st)
    for param, grad in pending["grads"]:
        if param.grad is not None and param.grad.data_ptr() != grad.data_ptr():
            param.grad.copy_(grad)
            deferred_stats["copies_rewritten"] += 1


def _side_by_side(device: torch.device, jobs, defer=None, reads=(), params=None):
    """Runs independent jobs (callables returning a tensor, or None for "not needed") and
    returns their results in order.  On the GPU the first needed job runs on the current
    stream and the others on side streams of their own (default priority, made once per
    device), so that they overlap: the reductions and the grad-kernel of a backward pass are
    chains as long as the batch -- bound by the latency of one chain, busy on a fraction of
    the CUs -- and side by side they take the time of the longest instead of the sum.
    The results are what the jobs return one after the other: the jobs are independent.

    defer[i] (only inside a backward pass; job i makes the gradient of params[i], and the caller
    has asked _deferrable(params[i])): the result is not waited for here but when the backward
    pass ends (a callback queued with the autograd engine), so that the current stream goes on with
    the next layer's backward while a grad-kernel chain of this one is still running.  Such jobs
    take turns on a small pool of streams, and `reads` -- the tensors they read -- are kept from
    reuse until those streams are done with them."""
    todo = [i for i, j in enumerate(jobs) if j is not None]
    out = [None] * len(jobs)
    if device.type != "cuda" or len(todo) < 2:
        for i in todo:
            out[i] = jobs[i]()
        return out
    key = device.index if device.index is not None else torch.cuda.current_device()
    cur = torch.cuda.current_stream(key)
    late = [i for i in todo[1:] if defer is not None and defer[i]]
    side = [i for i in todo[1:] if i not in late]
    streams = _SIDE_STREAMS.setdefault(key, [])
    while len(streams) < len(side):
        streams.append(torch.cuda.Stream(device=key))
    for st, i in zip(streams, side):
        st.wait_stream(cur)  # the inputs are complete
        with torch.cuda.stream(st):
            out[i] = jobs[i]()
    if late:
        pool = _DEFER_STREAMS.setdefault(key, {"streams": [], "next": 0})
        while len(pool["streams"]) < _DEFER_POOL:
            pool["streams"].append(torch.cuda.Stream(device=key))
        pending = _DEFERRED.setdefault(key, {"streams": [], "grads": []})
        # (one callback per call: whichever runs first joins everything that is pending, the others find nothing)
        torch.autograd.Variable._execution_engine.queue_callback(lambda: _join_deferred(key))
        for i in late:
            st = pool["streams"][pool["next"] % _DEFER_POOL]
            pool["next"] += 1
            st.wait_stream(cur)
            with torch.cuda.stream(st):
                out[i] = jobs[i]()
            for t in reads:
                t.record_stream(st)
            out[i].record_stream(cur)
            if st not in pending["streams"]:
                pending["streams"].append(st)
            deferred_stats["jobs"] += 1
            pending["grads"].append((params[i], out[i].detach()))  # (an alias: the result itself stays autograd's alone)
    out[todo[0]] = jobs[todo[0]]()
    for st, i in zip(streams, side):
        cur.wait_stream(st)  # later work on the current stream sees the result, and the inputs are
        out[i].record_stream(cur)  # not reused before the side stream is done with them
    return out


class _Conv2d(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, stride, padding, groups):
        ctx.save_for_backward(x, weight)
        ctx.conf = (stride, padding, groups)
        ctx.params = (weight, bias)  # (the parameters themselves, for their .grad and hooks)
        return ops.conv2d_bias(x, weight, bias, stride=stride, padding=padding, groups=groups)

    @staticmethod
    def backward(ctx, gy):
        stride, padding, groups = ctx.conf
        if groups != 1:
            raise NotImplementedError("conv2d backward: groups != 1")
        x, weight = ctx.saved_tensors
        need_x, need_w, need_b = ctx.needs_input_grad[:3]
        # grad-input fills the chip; grad-kernel and the bias sum are latency-bound chains: side by side
        # (the chains of the parameters' gradients need not end before the next layer's backward starts)
        gx, gw, gb = _side_by_side(gy.device, [
            (lambda: ops.conv2d_grad_input(x.shape, weight, gy, stride, padding)) if need_x else None,
            (lambda: ops.conv2d_grad_kernel(x, weight.shape, gy, stride, padding)) if need_w else None,
            (lambda: ops.sum4d_dim023(gy)) if need_b else None],
            defer=(False, need_x and _deferrable(ctx.params[0]), need_x and _deferrable(ctx.params[1])), reads=(x, gy),
            params=(None,) + ctx.params)
        return gx, gw, gb, None, None, None


def conv2d(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, stride: _Pair = 1,
           padding: Union[str, _Pair] = 0, dilation: _Pair = 1, groups: int = 1) -> torch.Tensor:
    if isinstance(padding, str) or dilation not in (1, (1, 1)) or input.dim() != 4:
        raise NotImplementedError("conv2d: string padding, dilation != 1 and non-4-D input are not supported")
    assert weight.dim() == 4
    assert bias is None or bias.dim() == 1
    stride = (stride, stride) if isinstance(stride, int) else tuple(stride)
    padding = (padding, padding) if isinstance(padding, int) else tuple(padding)
    return _Conv2d.apply(input, weight, bias, stride, padding, groups)


class _CrossEntropy(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, target):
        ctx.save_for_backward(logits, target)
        return ops.cross_entropy(logits, target)

    @staticmethod
    def backward(ctx, g):
        logits, target = ctx.saved_tensors
        if not ctx.needs_input_grad[0]:
            return None, None
        rows, classes = logits.shape
        gl = ops.softmax(logits) - torch.nn.functional.one_hot(target, classes)
        gl *= 1.0 / rows  # first the mean factor, then the incoming gradient (loss.py:32-33)
        gl *= g
        return gl, None


def cross_entropy(input: torch.Tensor, target: torch.Tensor, weight: Optional[torch.Tensor] = None,
                  size_average: Optional[bool] = None, ignore_index: int = -100, reduce: Optional[bool] = None,
                  reduction: str = "mean", label_smoothing: float = 0.0) -> torch.Tensor:
    plain = (weight is None and size_average is None and ignore_index == -100 and reduce is None
             and reduction == "mean" and label_smoothing == 0.0)
    if not plain or input.dim() != 2 or target.dim() != 1:
        raise NotImplementedError("cross_entropy: only mean reduction of [B,C] logits and [B] class indices")
    return _CrossEntropy.apply(input, target)


def _per_channel(t: torch.Tensor, like: torch.Tensor) -> torch.Tensor:
    return t.unsqueeze(-1).unsqueeze(-1) if like.dim() == 4 else t


class _BatchNorm(torch.autograd.Function):
    """y = (x - mean) / std * weight + bias with std = sqrt(var + eps); mean and var are
    inputs with their own gradients (reference batchnorm.py:12-66).  Divisions and
    the square root go through ops so they are the IEEE results on the GPU as well."""

    @staticmethod
    def forward(ctx, x, mean, var, weight, bias, eps):
        std = ops.sqrt(var + eps)
        ctx.save_for_backward(x, mean, std, weight)
        return ops.bn_apply(x, mean, std, weight, bias)  # ((x - mean) / std) * weight + bias, four roundings

    @staticmethod
    def backward(ctx, gy):
        x, mean, std, weight = ctx.saved_tensors
        reduce = ops.sum4d_dim023 if gy.dim() == 4 else ops.sum2d_dim0
        need = ctx.needs_input_grad
        w_over_std = ops.div(weight, std)
        coef = ops.div(weight, 2 * std * std * std) if need[2] else None
        # one elementwise product and up to three reductions (grad_mean and grad_bias share theirs:
        # the same operator on the same tensor), all independent: side by side
        gx, rgy, gvar, gweight = _side_by_side(gy.device, [
            (lambda: _per_channel(w_over_std, gy) * gy) if need[0] else None,
            (lambda: reduce(gy)) if need[1] or need[4] else None,
            (lambda: reduce(ops.bn_gvar_term(gy, x, mean, coef))) if need[2] else None,      # gy * (mean - x) * coef
            (lambda: reduce(ops.bn_gweight_term(x, mean, std, gy))) if need[3] else None])  # (x - mean) / std * gy
        gmean = (-w_over_std) * rgy if need[1] else None
        gbias = rgy if need[4] else None
        return gx, gmean, gvar, gweight, gbias, None


# The reference evaluates the running-statistics updates in training (batchnorm.py:92-93) and drops
# the results, so its buffers keep their initial values.  False reproduces that; True stores the two
# expressions it evaluates (running mean as PyTorch's, running variance from the biased batch variance).
STORE_RUNNING_STATS = False


def batch_norm(input: torch.Tensor, running_mean: Optional[torch.Tensor], running_var: Optional[torch.Tensor],
               weight: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
               batch_statistics: bool = False, momentum: float = 0.1, eps: float = 1e-5) -> torch.Tensor:
    if weight is None or bias is None or input.dim() not in (2, 4):
        raise NotImplementedError("batch_norm: affine parameters and 2-D or 4-D input are required")
    assert weight.dim() == 1 and bias.dim() == 1
    if batch_statistics:
        if input.dim() == 4:
            mean = func.mean4d_dim023(input)
            centred = input - func.expand_as(mean.unsqueeze(-1).unsqueeze(-1), input)
            var = func.mean4d_dim023(centred * centred)
        else:
            mean = func.mean2d_dim0(input)
            centred = input - func.expand_as(mean, input)
            var = func.mean2d_dim0(centred * centred)
        if STORE_RUNNING_STATS and running_mean is not None and running_var is not None:
            with torch.no_grad():
                running_mean.copy_(momentum * mean.detach() + (1.0 - momentum) * running_mean)
                running_var.copy_(momentum * var.detach() + (1.0 - momentum) * running_var)
    else:
        mean, var = running_mean, running_var
    return _BatchNorm.apply(input, mean, var, weight, bias, eps)
