"""The fused elementwise passes of batch normalisation (repdl_hip_bn_apply, _bn_gvar_term,
_bn_gweight_term) against the reference's own compositions of PyTorch CPU operations
(repdl/nn/batchnorm.py:25-32, 56-58, 60-61), bit for bit: rows long enough for the
row kernel and rows that take the flat kernel, row lengths that are no multiple of 4, a base
pointer that is not 16-byte aligned, [B,F] inputs, and data with zeros of both signs,
subnormals and infinities (NaN results compare as NaN)."""
import numpy as np
import pytest
import torch

import gen
from oracle_ops import _OracleBackend as cpu

pytestmark = pytest.mark.gpu

SHAPES = [(4, 8, 32, 32), (3, 5, 33, 35), (2, 3, 64, 66), (70, 16, 7, 7), (2, 6, 1, 1), (5, 3, 17, 241), (64, 10), (1000, 7),
          (1, 1, 1, 5000)]


def bits(t):
    a = t.detach().cpu().contiguous().numpy()
    b = a.view(np.uint32).copy()
    b[np.isnan(a)] = 0x7FC00000
    return b


def _data(shape, seed, special):
    C = shape[1]
    x, gy = gen.normal_like(seed, *shape) * 3, gen.scaled_normal(seed + 1, *shape, lo=-12, hi=4)
    mean, std = gen.normal_like(seed + 2, C), gen.uniform_pm1(seed + 3, C).abs() + 0.01
    weight, bias, coef = gen.normal_like(seed + 4, C), gen.normal_like(seed + 5, C), gen.scaled_normal(seed + 6, C, lo=-8, hi=8)
    if special:
        n = x.numel()
        x.view(-1)[::7] = gen.elementwise_mix(seed + 7, n)[::7]
        gy.view(-1)[3::11] = gen.elementwise_mix(seed + 8, n)[3::11]
        x.view(-1)[1::13] = mean[0]          # exact cancellation against channel 0's mean
        std[0], bias[0] = 1e-30, -0.0
        weight[-1] = 0.0
    return x, gy, mean, std, weight, bias, coef


@pytest.mark.parametrize("special", [False, True], ids=["plain", "special"])
@pytest.mark.parametrize("shape", SHAPES, ids=str)
def test_fused_passes_equal_the_compositions(shape, special):
    from repdl_amd import ops

    x, gy, mean, std, weight, bias, coef = _data(shape, 700 + len(shape) + shape[1], special)
    d = lambda t: t.cuda()
    assert np.array_equal(bits(ops.bn_apply(d(x), d(mean), d(std), d(weight), d(bias))), bits(cpu.bn_apply(x, mean, std, weight, bias)))
    assert np.array_equal(bits(ops.bn_gvar_term(d(gy), d(x), d(mean), d(coef))), bits(cpu.bn_gvar_term(gy, x, mean, coef)))
    assert np.array_equal(bits(ops.bn_gweight_term(d(x), d(mean), d(std), d(gy))), bits(cpu.bn_gweight_term(x, mean, std, gy)))


def test_unaligned_base_pointer():
    from repdl_amd import ops

    shape = (3, 4, 40, 40)
    x, gy, mean, std, weight, bias, coef = _data(shape, 750, False)
    off = lambda t: torch.cat([torch.zeros(1), t.view(-1)]).cuda()[1:].view(*t.shape)
    xd, gd = off(x), off(gy)
    assert xd.data_ptr() % 16 != 0
    assert np.array_equal(bits(ops.bn_apply(xd, mean.cuda(), std.cuda(), weight.cuda(), bias.cuda())), bits(cpu.bn_apply(x, mean, std, weight, bias)))
    assert np.array_equal(bits(ops.bn_gvar_term(gd, xd, mean.cuda(), coef.cuda())), bits(cpu.bn_gvar_term(gy, x, mean, coef)))
    assert np.array_equal(bits(ops.bn_gweight_term(xd, mean.cuda(), std.cuda(), gd)), bits(cpu.bn_gweight_term(x, mean, std, gy)))


def test_shape_errors():
    from repdl_amd import ops

    x = torch.zeros(2, 3, 4, 4, device="cuda")
    v3, v4 = torch.ones(3, device="cuda"), torch.ones(4, device="cuda")
    with pytest.raises(RuntimeError):
        ops.bn_apply(x, v3, v3, v4, v3)
    with pytest.raises(RuntimeError):
        ops.bn_gvar_term(x[:1], x, v3, v3)
    with pytest.raises(RuntimeError):
        ops.bn_apply(torch.zeros(2, 3, 4, device="cuda"), v3, v3, v3, v3)
