"""Seeded random shapes through mm and the three convolutions on the GPU, each output
compared bit for bit with the oracle: a sweep over the kernel-selection logic (tile sizes,
whole-tile and general kernels, padded-workspace and general gathers, piece lengths of the
grad-kernel, fallbacks) rather than over data."""
import numpy as np
import pytest
import torch

import gen
from oracle import api as oracle

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("matrix_path")]


def _mm_shapes():
    r = np.random.default_rng(20240607)
    shapes = []
    for _ in range(14):  # whole tiles of one of the three tile sizes, K a multiple of 16
        t = int(r.choice([64, 128, 256]))
        shapes.append((t * int(r.integers(1, 5)), t * int(r.integers(1, 5)), 16 * int(r.integers(1, 40))))
    for _ in range(14):  # anything
        shapes.append((int(r.integers(1, 700)), int(r.integers(1, 700)), int(r.integers(1, 600))))
    shapes += [(2560, 2304, 48), (4096, 2048, 32)]  # enough 256-tiles for the largest configuration
    return [(m, n, k, int(r.integers(0, 2)), int(r.integers(0, 2))) for (m, n, k) in shapes]


@pytest.mark.parametrize("shape", _mm_shapes(), ids=str)
def test_mm(shape):
    from repdl_amd import ops

    M, N, K, tA, tB = shape
    a = gen.normal_like(M + 3 * K, *((K, M) if tA else (M, K)))
    b = gen.scaled_normal(N + 5 * K, *((N, K) if tB else (K, N)), lo=-4, hi=4)
    got = ops.mm(a.cuda(), b.cuda(), bool(tA), bool(tB)).cpu()
    assert torch.equal(got.view(torch.int32), oracle.mm(a, b, bool(tA), bool(tB)).view(torch.int32))


def _conv_shapes():
    r = np.random.default_rng(77)
    out = []
    while len(out) < 28:
        g = int(r.choice([1, 1, 1, 2]))
        icg = int(r.choice([1, 3, 8, 16, 32]))
        ocg = int(r.choice([4, 16, 64, 128]))
        kh, kw = int(r.integers(1, 5)), int(r.integers(1, 5))
        sh, sw = int(r.integers(1, 3)), int(r.integers(1, 3))
        ph, pw = int(r.integers(0, 3)), int(r.integers(0, 3))
        h, w = int(r.integers(4, 40)), int(r.choice([8, 12, 16, 28, 30, 33, 56, 64]))
        if h + 2 * ph < kh or w + 2 * pw < kw:
            continue
        out.append((int(r.integers(1, 4)), icg * g, h, w, ocg * g, kh, kw, sh, sw, ph, pw, g))
    return out


@pytest.mark.parametrize("shape", _conv_shapes(), ids=str)
def test_conv(shape):
    from repdl_amd import ops

    N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, g = shape
    OH, OW = (H + 2 * pH - KH) // sH + 1, (W + 2 * pW - KW) // sW + 1
    x = gen.relu_like(H * W + IC, N, IC, H, W)
    w = gen.normal_like(OC + KH, OC, IC // g, KH, KW)
    go = gen.normal_like(OH + OW, N, OC, OH, OW)
    xd, wd, god = x.cuda(), w.cuda(), go.cuda()
    y = ops.conv2d(xd, wd, (sH, sW), (pH, pW), g).cpu()
    assert torch.equal(y.view(torch.int32), oracle.conv2d(x, w, sH, sW, pH, pW, g).view(torch.int32))
    if g == 1:
        gi = ops.conv2d_grad_input((N, IC, H, W), wd, god, (sH, sW), (pH, pW)).cpu()
        assert torch.equal(gi.view(torch.int32), oracle.conv2d_grad_input(go, w, H, W, sH, sW, pH, pW).view(torch.int32))
        gk = ops.conv2d_grad_kernel(xd, (OC, IC, KH, KW), god, (sH, sW), (pH, pW)).cpu()
        assert torch.equal(gk.view(torch.int32), oracle.conv2d_grad_kernel(go, x, KH, KW, sH, sW, pH, pW).view(torch.int32))
