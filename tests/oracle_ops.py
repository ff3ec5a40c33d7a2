"""Test helper: lets the package's Python glue (repdl_amd.nn / func / optim) run on
CPU tensors by pointing ``repdl_amd.ops._backend`` at the C oracle for them.  GPU
tensors keep going to the HIP backend.  The product has no such path: this is a
monkeypatch made by tests only, so the same glue can be run on both sides of a
parity check."""
from __future__ import annotations

import contextlib

import torch

import repdl_amd
from oracle import api as oracle


class _OracleBackend:
    """The function set of repdl_amd.backend.hip, served by the oracle."""

    mm = staticmethod(oracle.mm)
    conv2d = staticmethod(oracle.conv2d)
    conv2d_grad_input = staticmethod(oracle.conv2d_grad_input)
    conv2d_grad_kernel = staticmethod(oracle.conv2d_grad_kernel)
    cross_entropy = staticmethod(oracle.cross_entropy)
    softmax = staticmethod(oracle.softmax)
    sum1d = staticmethod(oracle.sum1d)
    sum2d_dim0 = staticmethod(oracle.sum2d_dim0)
    sum2d_dim1 = staticmethod(oracle.sum2d_dim1)
    sum4d_dim023 = staticmethod(oracle.sum4d_dim023)
    exp = staticmethod(oracle.exp)
    log = staticmethod(oracle.log)
    sqrt = staticmethod(oracle.sqrt)

    @staticmethod
    def mm_bias(input, mat2, bias, transA, transB):
        y = oracle.mm(input, mat2, transA, transB)  # repdl/nn/linear.py:21-22
        if bias is not None:
            y += bias
        return y

    @staticmethod
    def conv2d_bias(input, kernel, bias, sH, sW, pH, pW, groups):
        y = oracle.conv2d(input, kernel, sH, sW, pH, pW, groups)  # repdl/nn/conv.py:27-28
        if bias is not None:
            y += bias.unsqueeze(-1).unsqueeze(-1)
        return y

    # the reference's own compositions (repdl/nn/batchnorm.py:25-32, 56-58, 60-61); its divisions go through
    # the oracle's div, which is PyTorch's CPU division
    @staticmethod
    def _bc(v, like):
        return v.unsqueeze(-1).unsqueeze(-1) if like.dim() == 4 else v

    @staticmethod
    def bn_apply(x, mean, std, weight, bias):
        bc = _OracleBackend._bc
        y = _OracleBackend.div(x - bc(mean, x), bc(std, x))
        y *= bc(weight, x)
        y += bc(bias, x)
        return y

    @staticmethod
    def bn_gvar_term(gy, x, mean, coef):
        bc = _OracleBackend._bc
        return gy * (bc(mean, x) - x) * bc(coef, x)

    @staticmethod
    def bn_gweight_term(x, mean, std, gy):
        bc = _OracleBackend._bc
        return _OracleBackend.div(x - bc(mean, x), bc(std, x)) * gy

    @staticmethod
    def div(a, b):
        shape = torch.broadcast_shapes(a.shape, b.shape)
        return oracle.div(a.expand(shape).contiguous(), b.expand(shape).contiguous())

    @staticmethod
    def div_scalar(a, b):
        return oracle.div(a, float(b))


@contextlib.contextmanager
def oracle_for_cpu_tensors():
    original = repdl_amd.ops._backend

    def pick(t):
        return _OracleBackend if not t.is_cuda else original(t)

    repdl_amd.ops._backend = pick
    try:
        yield
    finally:
        repdl_amd.ops._backend = original
