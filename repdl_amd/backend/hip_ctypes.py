"""``repdl_amd.backend.hip_ctypes`` -- the function set of RepDL's compiled
``repdl.backend.cuda`` (backend/cuda/bind.cpp:12-19) bound to the C ABI with ctypes:
the same ten functions with the same positional signatures, tensors in and a new
tensor out, plus the elementwise operators (``exp``, ``log``, ``sqrt``, ``div``,
``div_scalar``), ``mm_bias`` / ``conv2d_bias`` (the layer's bias added in the
kernel's epilogue) and the fused elementwise passes of batch normalisation.  ``repdl_amd.backend.hip`` serves these when the compiled binding
(csrc/bind.cpp) has not been built; both call the same library.

Each function validates its tensors (float32, on the GPU, made contiguous),
allocates the output with PyTorch on the input's device and hands raw pointers
and the current stream to the C ABI (include/repdl_hip.h).  Output shapes follow
the reference, including ``squeeze()`` of the sums when ``keepdim`` is false
(backend/cuda/summation.cu:41, 68, 103, 141) and the 0-dim results of ``sum1d``
and ``cross_entropy``.
"""
from __future__ import annotations

import ctypes

import torch

from .. import _lib

_P = ctypes.c_void_p


def _check(t: torch.Tensor, name: str, dim: int | None = None, dtype=torch.float32) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a torch.Tensor" % name)
    if not t.is_cuda:
        raise RuntimeError("%s must be on the GPU (this backend has no CPU path)" % name)
    if t.dtype != dtype:
        raise RuntimeError("%s must be %s, got %s" % (name, dtype, t.dtype))
    if dim is not None and t.dim() != dim:
        raise RuntimeError("%s must have %d dimensions, got %d" % (name, dim, t.dim()))
    return t.contiguous()


def _ptr(t: torch.Tensor) -> _P:
    return _P(t.data_ptr())


def _stream(t: torch.Tensor) -> _P:
    return _P(torch.cuda.current_stream(t.device).cuda_stream)


def _scratch(query: str, like: torch.Tensor, *args):
    """Scratch memory of a call from PyTorch's allocator, sized by the entry point's own query: (tensor or None,
    pointer, size).  The library then allocates, frees and keeps nothing, so the call can be captured into a graph."""
    nbytes = int(getattr(_lib.lib(), query)(*args))
    if nbytes == 0:
        return None, None, ctypes.c_size_t(0)
    work = torch.empty((nbytes,), dtype=torch.uint8, device=like.device)
    return work, _ptr(work), ctypes.c_size_t(nbytes)


def _same_device(a: torch.Tensor, b: torch.Tensor) -> None:
    if a.device != b.device:
        raise RuntimeError("tensors are on different devices: %s and %s" % (a.device, b.device))


def _bias(bias, like: torch.Tensor, channels: int):
    """The bias of a layer as a pointer: [channels] on the same device, or None."""
    if bias is None:
        return None, None
    b = _check(bias, "bias", 1)
    _same_device(b, like)
    if b.shape[0] != channels:
        raise RuntimeError("bias has %d elements for %d output channels" % (b.shape[0], channels))
    return b, _ptr(b)


def mm(input: torch.Tensor, mat2: torch.Tensor, transA: bool, transB: bool) -> torch.Tensor:
    return mm_bias(input, mat2, None, transA, transB)


def mm_bias(input: torch.Tensor, mat2: torch.Tensor, bias, transA: bool, transB: bool) -> torch.Tensor:
    """mm followed by ``+= bias`` (repdl/nn/linear.py:21-22), the addition made in the kernel's epilogue."""
    a, b = _check(input, "input", 2), _check(mat2, "mat2", 2)
    _same_device(a, b)
    M, K = (a.shape[0], a.shape[1]) if not transA else (a.shape[1], a.shape[0])
    N, Kb = (b.shape[1], b.shape[0]) if not transB else (b.shape[0], b.shape[1])
    if K != Kb:
        raise RuntimeError("mm: inner dimensions differ (%d vs %d)" % (K, Kb))
    hold, bp = _bias(bias, a, N)
    out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    with torch.cuda.device(a.device):
        _lib.call("repdl_hip_mm_bias", _ptr(a), _ptr(b), bp, _ptr(out), M, N, K, int(bool(transA)), int(bool(transB)),
                  _stream(a))
    return out


def conv2d(input, kernel, strideH, strideW, paddingH, paddingW, groups) -> torch.Tensor:
    return conv2d_bias(input, kernel, None, strideH, strideW, paddingH, paddingW, groups)


def conv2d_bias(input, kernel, bias, strideH, strideW, paddingH, paddingW, groups) -> torch.Tensor:
    """conv2d followed by ``+= bias`` per output channel (repdl/nn/conv.py:27-28), in the epilogue."""
    x, k = _check(input, "input", 4), _check(kernel, "kernel", 4)
    _same_device(x, k)
    N, IC, H, W = x.shape
    OC, ICg, KH, KW = k.shape
    if groups <= 0 or IC % groups or OC % groups or ICg != IC // groups:
        raise RuntimeError("conv2d: channels (%d in, %d out, kernel %d) do not match groups=%d" % (IC, OC, ICg, groups))
    if H + 2 * paddingH < KH or W + 2 * paddingW < KW:
        raise RuntimeError("conv2d: kernel larger than padded input")
    OH, OW = (H + 2 * paddingH - KH) // strideH + 1, (W + 2 * paddingW - KW) // strideW + 1
    hold, bp = _bias(bias, x, OC)
    out = torch.empty((N, OC, OH, OW), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        dims = (N, IC, H, W, OC, KH, KW, strideH, strideW, paddingH, paddingW, groups)
        work, wp, wn = _scratch("repdl_hip_conv2d_workspace_bytes", x, _ptr(x), _ptr(k), *dims)
        _lib.call("repdl_hip_conv2d_ws", _ptr(x), _ptr(k), bp, _ptr(out), *dims, wp, wn, _stream(x))
    return out


def conv2d_grad_input(grad_output, kernel, H, W, strideH, strideW, paddingH, paddingW) -> torch.Tensor:
    go, k = _check(grad_output, "grad_output", 4), _check(kernel, "kernel", 4)
    _same_device(go, k)
    N, OC, OH, OW = go.shape
    OCk, IC, KH, KW = k.shape
    if OCk != OC:
        raise RuntimeError("conv2d_grad_input: grad_output has %d channels, kernel has %d" % (OC, OCk))
    out = torch.empty((N, IC, H, W), dtype=torch.float32, device=go.device)
    with torch.cuda.device(go.device):
        dims = (N, OC, OH, OW, IC, KH, KW, H, W, strideH, strideW, paddingH, paddingW)
        work, wp, wn = _scratch("repdl_hip_conv2d_grad_input_workspace_bytes", go, _ptr(go), _ptr(k), *dims)
        _lib.call("repdl_hip_conv2d_grad_input_ws", _ptr(go), _ptr(k), _ptr(out), *dims, wp, wn, _stream(go))
    return out


def conv2d_grad_kernel(grad_output, input, KH, KW, strideH, strideW, paddingH, paddingW) -> torch.Tensor:
    go, x = _check(grad_output, "grad_output", 4), _check(input, "input", 4)
    _same_device(go, x)
    N, IC, H, W = x.shape
    Ng, OC, OH, OW = go.shape
    if Ng != N:
        raise RuntimeError("conv2d_grad_kernel: batch sizes differ (%d vs %d)" % (N, Ng))
    out = torch.empty((OC, IC, KH, KW), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        dims = (N, IC, H, W, OC, OH, OW, KH, KW, strideH, strideW, paddingH, paddingW)
        work, wp, wn = _scratch("repdl_hip_conv2d_grad_kernel_workspace_bytes", x, _ptr(go), _ptr(x), *dims)
        _lib.call("repdl_hip_conv2d_grad_kernel_ws", _ptr(go), _ptr(x), _ptr(out), *dims, wp, wn, _stream(x))
    return out


def sum1d(input, average: bool = False) -> torch.Tensor:
    x = _check(input, "input", 1)
    out = torch.empty((), dtype=torch.float32, device=x.device)
    n = x.shape[0]
    with torch.cuda.device(x.device):
        # scratch for the parallel evaluation of the sequential chain
        work, wp, wn = _scratch("repdl_hip_sum1d_workspace_bytes", x, n)
        _lib.call("repdl_hip_sum1d_ws", _ptr(x), _ptr(out), n, int(bool(average)), wp, wn, _stream(x))
    return out


def sum2d_dim0(input, keepdim: bool = False, average: bool = False) -> torch.Tensor:
    x = _check(input, "input", 2)
    M, N = x.shape
    out = torch.empty((1, N), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _lib.call("repdl_hip_sum2d_dim0", _ptr(x), _ptr(out), M, N, int(bool(average)), _stream(x))
    return out if keepdim else out.squeeze()


def sum2d_dim1(input, keepdim: bool = False, average: bool = False) -> torch.Tensor:
    x = _check(input, "input", 2)
    M, N = x.shape
    out = torch.empty((M, 1), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        work, wp, wn = _scratch("repdl_hip_sum2d_dim1_workspace_bytes", x, M, N)
        _lib.call("repdl_hip_sum2d_dim1_ws", _ptr(x), _ptr(out), M, N, int(bool(average)), wp, wn, _stream(x))
    return out if keepdim else out.squeeze()


def sum4d_dim023(input, keepdim: bool = False, average: bool = False) -> torch.Tensor:
    x = _check(input, "input", 4)
    N, C, H, W = x.shape
    out = torch.empty((1, C, 1, 1), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        work, wp, wn = _scratch("repdl_hip_sum4d_dim023_workspace_bytes", x, N, C, H, W)
        _lib.call("repdl_hip_sum4d_dim023_ws", _ptr(x), _ptr(out), N, C, H, W, int(bool(average)), wp, wn, _stream(x))
    return out if keepdim else out.squeeze()


def _unary(name: str, input: torch.Tensor) -> torch.Tensor:
    x = _check(input, "input")
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        _lib.call(name, _ptr(x), _ptr(out), x.numel(), _stream(x))
    return out


def exp(input: torch.Tensor) -> torch.Tensor:
    return _unary("repdl_hip_exp", input)


def log(input: torch.Tensor) -> torch.Tensor:
    return _unary("repdl_hip_log", input)


def sqrt(input: torch.Tensor) -> torch.Tensor:
    return _unary("repdl_hip_sqrt", input)


def div(input: torch.Tensor, other: torch.Tensor) -> torch.Tensor:
    """input / other elementwise; ``other`` is broadcast to ``input``'s shape.  A
    0-dim ``other`` goes through the scalar entry point."""
    x = _check(input, "input")
    if other.dim() == 0:
        return div_scalar(x, float(other))
    y = _check(other, "other")
    _same_device(x, y)
    shape = torch.broadcast_shapes(x.shape, y.shape)
    if tuple(shape) != tuple(x.shape):
        x = x.expand(shape).contiguous()
    if tuple(y.shape) != tuple(shape):
        y = y.expand(shape).contiguous()
    out = torch.empty(shape, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _lib.call("repdl_hip_div", _ptr(x), _ptr(y), _ptr(out), out.numel(), _stream(x))
    return out


def div_scalar(input: torch.Tensor, other: float) -> torch.Tensor:
    x = _check(input, "input")
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        _lib.call("repdl_hip_div_scalar", _ptr(x), ctypes.c_float(other), _ptr(out), x.numel(), _stream(x))
    return out


def softmax(input: torch.Tensor) -> torch.Tensor:
    x = _check(input, "input", 2)
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        _lib.call("repdl_hip_softmax", _ptr(x), _ptr(out), x.shape[0], x.shape[1], _stream(x))
    return out


def cross_entropy(input: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
    x = _check(input, "input", 2)
    t = _check(target, "target", 1, dtype=torch.int64)
    _same_device(x, t)
    if t.shape[0] != x.shape[0]:
        raise RuntimeError("cross_entropy: %d rows but %d targets" % (x.shape[0], t.shape[0]))
    out = torch.empty((), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        # the row losses and the scratch of their mean
        work, wp, wn = _scratch("repdl_hip_cross_entropy_workspace_bytes", x, x.shape[0], x.shape[1])
        _lib.call("repdl_hip_cross_entropy_ws", _ptr(x), _ptr(t), _ptr(out), x.shape[0], x.shape[1], wp, wn, _stream(x))
    return out


def _bn_geometry(x: torch.Tensor, *vectors: torch.Tensor):
    """[N,C,H,W] or [B,F] with per-channel vectors of C (F) elements -> (outer, channels, inner)."""
    if x.dim() == 4:
        outer, channels, inner = x.shape[0], x.shape[1], x.shape[2] * x.shape[3]
    elif x.dim() == 2:
        outer, channels, inner = x.shape[0], x.shape[1], 1
    else:
        raise RuntimeError("batch norm takes 2-D or 4-D tensors, got %d dimensions" % x.dim())
    for v in vectors:
        if v.numel() != channels:
            raise RuntimeError("a per-channel vector has %d elements for %d channels" % (v.numel(), channels))
        _same_device(v, x)
    return outer, channels, inner


def bn_apply(input, mean, std, weight, bias) -> torch.Tensor:
    """((input - mean) / std) * weight + bias per channel, every operation rounded (repdl/nn/batchnorm.py:25-32)."""
    x = _check(input, "input")
    m, s, w, b = (_check(t, n, 1) for t, n in ((mean, "mean"), (std, "std"), (weight, "weight"), (bias, "bias")))
    outer, channels, inner = _bn_geometry(x, m, s, w, b)
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        _lib.call("repdl_hip_bn_apply", _ptr(x), _ptr(m), _ptr(s), _ptr(w), _ptr(b), _ptr(out), outer, channels, inner,
                  _stream(x))
    return out


def bn_gvar_term(grad_output, input, mean, coef) -> torch.Tensor:
    """(grad_output * (mean - input)) * coef per channel: what grad_var sums (repdl/nn/batchnorm.py:56-58)."""
    g, x = _check(grad_output, "grad_output"), _check(input, "input")
    m, c = _check(mean, "mean", 1), _check(coef, "coef", 1)
    if g.shape != x.shape:
        raise RuntimeError("grad_output and input differ in shape")
    _same_device(g, x)
    outer, channels, inner = _bn_geometry(x, m, c)
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        _lib.call("repdl_hip_bn_gvar_term", _ptr(g), _ptr(x), _ptr(m), _ptr(c), _ptr(out), outer, channels, inner, _stream(x))
    return out


def bn_gweight_term(input, mean, std, grad_output) -> torch.Tensor:
    """((input - mean) / std) * grad_output per channel: what grad_weight sums (repdl/nn/batchnorm.py:60-61)."""
    x, g = _check(input, "input"), _check(grad_output, "grad_output")
    m, s = _check(mean, "mean", 1), _check(std, "std", 1)
    if g.shape != x.shape:
        raise RuntimeError("grad_output and input differ in shape")
    _same_device(g, x)
    outer, channels, inner = _bn_geometry(x, m, s)
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        _lib.call("repdl_hip_bn_gweight_term", _ptr(x), _ptr(m), _ptr(s), _ptr(g), _ptr(out), outer, channels, inner,
                  _stream(x))
    return out
