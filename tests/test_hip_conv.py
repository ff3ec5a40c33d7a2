"""GPU parity of the three convolutions against the oracle beyond the golden cases: shapes
that take the matrix-instruction kernels' fast paths (whole channel tiles, K a multiple of
16, padded-workspace gather; grad-kernel with every piece length, with widths that are
not multiples of 4 and with strides) and shapes that fall back, strides, paddings larger
and smaller than the kernel reach, groups, pixels that do not fill the last tile, and three
kinds of data: plain (ReLU zeros: zero results that the padded chains already get right),
"special" (signed zeros and infinities: NaN results are recomputed with the literal chain)
and "tiny" (products that underflow to -0.0f: the guard of the zero results must send them
through the literal chain, while whole dead channels stay exact zeros)."""
import pytest
import torch

import gen
from oracle import api as oracle

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("matrix_path")]

# (N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, groups)
FWD = [
    (2, 32, 20, 24, 64, 3, 3, 1, 1, 1, 1, 1),    # fast path, 480 pixels (3.75 tiles)
    (3, 16, 17, 13, 64, 1, 1, 1, 1, 0, 0, 1),    # fast path, no padding workspace
    (2, 64, 19, 19, 128, 3, 3, 2, 2, 1, 1, 2),   # fast path, groups, stride 2
    (1, 16, 12, 40, 128, 5, 5, 1, 2, 1, 3, 1),   # fast path, BM = 128, asymmetric stride / padding
    (2, 16, 9, 9, 64, 1, 1, 1, 1, 1, 1, 1),      # padding beyond the kernel reach
    (2, 8, 14, 14, 24, 3, 3, 1, 1, 1, 1, 1),     # K = 72, few and ragged k-steps: gather kernel
    (1, 12, 10, 11, 70, 3, 2, 2, 1, 0, 1, 1),    # ragged everything
    (2, 32, 12, 13, 96, 3, 3, 1, 1, 1, 1, 1),    # fast path, 96 rows in a 128-row tile
    (2, 30, 12, 13, 40, 3, 3, 1, 1, 1, 1, 1),    # fast path, K = 270 rounded up to 272, 40 rows in a 64-row tile
    (2, 60, 10, 10, 80, 3, 3, 1, 1, 1, 1, 2),    # the same per group
    (1, 20, 9, 9, 200, 4, 4, 1, 1, 2, 2, 1),     # 200 rows: 64-row tiles (192 + 8)
    # small images, many channels: one matrix product over an im2col workspace (forward and grad-input)
    (32, 64, 8, 8, 128, 3, 3, 1, 1, 1, 1, 1),
    (24, 128, 9, 10, 64, 3, 3, 1, 1, 1, 1, 1),
    (40, 128, 15, 15, 128, 3, 3, 2, 2, 1, 1, 1),   # (forward only: its 15x15 input is too large for grad-input to take this route)
    (32, 128, 9, 9, 128, 5, 3, 2, 1, 2, 1, 1),     # strides in grad-input: input 9x9, output 5x9
    (32, 512, 8, 8, 128, 1, 1, 1, 1, 0, 0, 1),
    # 3x3 at stride 1 on images 32 to 62 wide, channels in fours, rows in 64s: the input-patch kernel
    (2, 64, 20, 40, 64, 3, 3, 1, 1, 1, 1, 1),      # 800 pixels: 6.25 tiles, tiles that start mid-row
    (1, 8, 9, 33, 128, 3, 3, 1, 1, 0, 2, 1),       # two row tiles, no padding above / two columns left, 7x35 output
    (3, 64, 35, 32, 64, 3, 3, 1, 1, 2, 0, 1),      # narrowest image: a tile spans five rows; output 37x30 (below 32: falls back)
    (2, 12, 5, 62, 64, 3, 3, 1, 1, 1, 1, 1),       # widest image, three chunks of four channels, few rows
    (1, 64, 34, 34, 64, 3, 3, 1, 1, 0, 0, 1),      # forward skips no tap (32x32 output), grad-input does
    # 1x1 at stride 1 without padding on images of 1024 pixels and more: the kernel that streams both operands
    (2, 32, 33, 40, 64, 1, 1, 1, 1, 0, 0, 1),      # 1320 pixels: 10.3 tiles
    (1, 16, 32, 32, 128, 1, 1, 1, 1, 0, 0, 1),     # two row tiles forward, 16 channels: one step of the stream
    (3, 64, 30, 45, 64, 1, 1, 1, 1, 0, 0, 1),      # 1350 pixels, the last tile half full
    # 3x3 at stride 1, source width in fours, channels in fours: both operands straight into LDS
    (2, 32, 20, 24, 64, 3, 3, 1, 1, 1, 1, 1),      # (also above) 480 pixels: 7.5 tiles of 64
    (3, 8, 12, 28, 40, 3, 3, 1, 1, 1, 1, 1),       # 40 rows of a 64-row tile forward, 8 in grad-input
    (2, 16, 9, 112, 72, 3, 3, 1, 1, 0, 2, 1),      # wide rows (a tile inside one row), no padding above, two columns left
    (1, 4, 8, 8, 4, 3, 3, 1, 1, 2, 2, 1),          # one chunk, padding 2, eight patch rows for a tile
    (2, 132, 10, 12, 68, 3, 3, 1, 1, 1, 0, 1),     # 33 chunks (three buffers: 11 turns), ragged rows both ways
    # the same with 4 bytes per DMA lane: any width
    (3, 64, 14, 14, 64, 3, 3, 1, 1, 1, 1, 1),
    (2, 16, 11, 30, 24, 3, 3, 1, 1, 2, 1, 1),      # rows of 30, padding 2 above and below, 24 rows
    (5, 128, 7, 7, 128, 3, 3, 1, 1, 1, 1, 1),      # an image smaller than a tile
    (2, 8, 6, 61, 20, 3, 3, 1, 1, 0, 0, 1),        # no padding: 4x59 output, nothing skipped forward
    # 1x1 at stride 1 without padding, pixels in fours, channels in fours: a batch of matrix products per image
    (2, 96, 20, 20, 72, 1, 1, 1, 1, 0, 0, 1),      # 400 pixels, 72 rows forward (96 in grad-input): tile edges both ways
    (3, 128, 33, 40, 192, 1, 1, 1, 1, 0, 0, 1),    # chains of 128 (forward) and 192 (grad-input) terms
    # 1x1 at a stride without padding: grad-input is the stride-1 layer's, scattered (forward: the implicit product)
    (2, 64, 56, 56, 128, 1, 1, 2, 2, 0, 0, 1),     # 28x28 output: a batch of matrix products per image
    (3, 16, 33, 41, 64, 1, 1, 2, 3, 0, 0, 1),      # different strides, 17x14 output, rows and columns past the last tap
    (2, 8, 10, 9, 24, 1, 1, 4, 4, 0, 0, 1),        # 3x3 output, stride wider than half the image
    (2, 8, 9, 20, 16, 1, 1, 1, 2, 0, 0, 1),        # a stride along the rows only
    (2, 8, 20, 9, 16, 1, 1, 3, 1, 0, 0, 1),        # ... down the columns only
    (1, 68, 6, 6, 20, 1, 1, 1, 1, 0, 0, 1),        # one small image: a k-tile tail of one quad, 20 rows
    (5, 24, 8, 12, 36, 1, 1, 1, 1, 0, 0, 1),       # chains shorter than a k-tile
]


def _data(shape, seed, special):
    N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, g = shape
    x = gen.relu_like(seed, N, IC, H, W)
    w = gen.normal_like(seed + 1, OC, IC // g, KH, KW)
    if special == "tiny":
        x, w = _tiny(x, 0), _tiny(w, 0)
    elif special:
        x.view(-1)[::97] = float("inf")
        x.view(-1)[5::211] = -0.0
        w.view(-1)[::53] = 0.0
        w.view(-1)[7::59] = -0.0
    return x, w


def _tiny(t, dim):
    """The slices of even index along `dim` scaled to about 1e-25 with mixed signs: where two
    such slices meet in a chain every product underflows to +-0 and the result is a zero
    whose sign depends on the taps that were skipped."""
    t = t.clone()
    flat = t.view(-1)
    scale = torch.full_like(flat, 1e-25)
    scale[::3] = -1e-25
    keep = torch.zeros(t.shape[dim], dtype=torch.bool)
    keep[1::2] = True
    shape = [1] * t.dim()
    shape[dim] = -1
    scale = torch.where(keep.view(shape).expand_as(t), torch.ones_like(t), scale.view_as(t))
    return t * scale


KINDS = [False, True, "tiny"]
KIND_IDS = ["plain", "special", "tiny"]


def _same(got, want):
    nan = torch.isnan(want)
    return torch.equal(torch.isnan(got), nan) and torch.equal(got.view(torch.int32)[~nan], want.view(torch.int32)[~nan])


@pytest.mark.parametrize("special", KINDS, ids=KIND_IDS)
@pytest.mark.parametrize("shape", FWD, ids=[str(s) for s in FWD])
def test_forward(shape, special):
    from repdl_amd import ops

    N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, g = shape
    x, w = _data(shape, 100, special)
    got = ops.conv2d(x.cuda(), w.cuda(), (sH, sW), (pH, pW), g).cpu()
    assert _same(got, oracle.conv2d(x, w, sH, sW, pH, pW, g))


@pytest.mark.parametrize("special", KINDS, ids=KIND_IDS)
@pytest.mark.parametrize("shape", FWD, ids=[str(s) for s in FWD])
def test_forward_with_bias(shape, special):
    """conv2d_bias = conv2d followed by one rounded `+= bias` per channel (repdl/nn/conv.py:27-28)
    on every forward kernel; zero results that are recomputed with the literal chain get their
    bias after the recomputation (the sign of a zero sum decides -0 + -0 against +0 + -0)."""
    from repdl_amd import ops

    N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, g = shape
    x, w = _data(shape, 150, special)
    bias = gen.scaled_normal(151, OC, lo=-20, hi=10)
    bias[::4] = -0.0
    bias[1::9] = 0.0
    want = oracle.conv2d(x, w, sH, sW, pH, pW, g)
    want += bias.unsqueeze(-1).unsqueeze(-1)
    got = ops.conv2d_bias(x.cuda(), w.cuda(), bias.cuda(), (sH, sW), (pH, pW), g).cpu()
    assert _same(got, want)


# grad-input with strides on the matrix path (IC a multiple of 64, OC*KH*KW of 16): grad_output is
# dilated into the workspace; input rows and columns that no output reaches (remainders of the stride)
DGRAD = [s for s in FWD if s[-1] == 1] + [
    (2, 64, 19, 19, 128, 3, 3, 2, 2, 1, 1, 1),
    (1, 64, 17, 23, 64, 1, 1, 2, 2, 0, 0, 1),
    (1, 128, 11, 13, 32, 3, 3, 3, 2, 0, 2, 1),
    (2, 64, 20, 22, 16, 5, 5, 4, 4, 2, 2, 1),
    (1, 64, 9, 9, 16, 2, 2, 1, 1, 3, 3, 1),      # padding beyond the kernel reach, stride 1
    # strides with enough work (3 GFLOP of products that count) for the route that takes the residues of the stride
    # one by one: stride-1 layers with the taps of a residue, their results interleaved
    (64, 64, 56, 56, 128, 3, 3, 2, 2, 1, 1, 1),   # 3x3 at stride 2: kernels of 2x2, 2x1, 1x2 and 1x1 taps
    (72, 64, 31, 29, 160, 5, 3, 2, 3, 2, 0, 1),   # 5x3 at stride (2, 3): a residue with a single column of taps, ragged extents
    (64, 192, 30, 30, 320, 2, 2, 3, 3, 0, 0, 1),  # stride wider than the kernel: residues without any tap (+0)
    (48, 64, 33, 34, 128, 3, 3, 1, 2, 1, 1, 1),   # a stride along the rows only
    # residues whose positions outnumber the rows / columns of grad_output (their trailing positions have no tap, +0):
    # the single-tap residues are 1x1 layers whose input and output planes differ
    (44, 64, 32, 32, 256, 3, 3, 2, 2, 0, 0, 1),   # 15x15 outputs, residue 1 has 16x16 positions: products per image
    (32, 128, 31, 31, 384, 2, 2, 2, 2, 0, 0, 1),  # every residue a single tap, 16 against 15 positions
    (32, 128, 29, 29, 448, 3, 3, 3, 3, 0, 0, 1),  # stride 3: 10 against 9
    (40, 64, 66, 66, 64, 3, 3, 2, 2, 0, 0, 1),    # 33x33 positions against 32x32 outputs, chains of 64: the streaming 1x1 kernel's shape
]


@pytest.mark.parametrize("special", KINDS, ids=KIND_IDS)
@pytest.mark.parametrize("shape", DGRAD, ids=[str(s) for s in DGRAD])
def test_grad_input(shape, special):
    from repdl_amd import ops

    N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, g = shape
    OH, OW = (H + 2 * pH - KH) // sH + 1, (W + 2 * pW - KW) // sW + 1
    go = gen.normal_like(7, N, OC, OH, OW) * gen.relu_like(8, N, OC, OH, OW).sign()
    w = gen.normal_like(9, OC, IC, KH, KW)
    if special == "tiny":
        go, w = _tiny(go, 0), _tiny(w, 1)
        go[:, 0] = 0.0
    elif special:
        go.view(-1)[::101] = float("-inf")
        w.view(-1)[3::41] = -0.0
    got = ops.conv2d_grad_input((N, IC, H, W), w.cuda(), go.cuda(), (sH, sW), (pH, pW)).cpu()
    assert _same(got, oracle.conv2d_grad_input(go, w, H, W, sH, sW, pH, pW))


WGRAD = [
    (3, 20, 18, 16, 40, 3, 3, 1, 1, 1, 1),   # OW = 16: one piece of 4 instructions
    (2, 8, 30, 28, 70, 3, 3, 1, 1, 1, 1),    # OW = 28: pieces of 7, OH = 30 -> chunks of several rows
    (2, 16, 16, 64, 16, 1, 1, 1, 1, 0, 0),   # OW = 64: pieces of 16, 1x1
    (2, 6, 33, 65, 33, 3, 3, 2, 2, 1, 1),    # stride 2, OW = 33 and W = 65: both operands through padded copies
    (2, 5, 11, 12, 9, 2, 3, 1, 1, 0, 1),     # ragged
    (4, 8, 14, 14, 16, 3, 3, 1, 1, 1, 1),    # OW = W = 14: rows rounded up to 16, pieces of 4
    (2, 3, 9, 7, 5, 3, 3, 1, 1, 1, 1),       # OW = 7: pieces of 2
    (2, 3, 5, 3, 4, 1, 1, 1, 1, 0, 0),       # OW = 3: pieces of 1
    (2, 4, 12, 40, 6, 3, 5, 1, 3, 1, 2),     # stride 3 along the row
    (1, 2, 8, 70, 3, 1, 3, 1, 17, 0, 1),     # stride 17: v_fma_f32 kernel
    (4, 64, 7, 7, 512, 3, 3, 1, 1, 1, 1),    # many short chains: one matrix product over an im2col workspace
    (2, 128, 7, 7, 2048, 1, 1, 1, 1, 0, 0),  # the same, 1x1 without padding (nothing to fix up)
    (3, 64, 15, 15, 512, 3, 3, 2, 2, 1, 1),  # the same with strides
    (3, 16, 30, 28, 32, 1, 1, 2, 2, 0, 0),   # 1x1 at stride 2: the input gathered, then the stride-1 layer (chain kernel)
    (2, 8, 17, 23, 12, 1, 1, 3, 2, 0, 0),    # the same with different strides and ragged extents
    (2, 8, 9, 20, 16, 1, 1, 1, 2, 0, 0),     # a stride along the rows only
    (2, 8, 20, 9, 16, 1, 1, 3, 1, 0, 0),     # ... down the columns only
    (4, 128, 14, 14, 512, 1, 1, 2, 2, 0, 0), # the same, many short chains: gathered, then one matrix product
    (2, 24, 28, 28, 96, 3, 3, 2, 2, 1, 1),   # 3x3 at stride 2, enough chains for several rounds of the chain kernel
]


@pytest.mark.parametrize("special", KINDS, ids=KIND_IDS)
@pytest.mark.parametrize("shape", WGRAD, ids=[str(s) for s in WGRAD])
def test_grad_kernel(shape, special):
    from repdl_amd import ops

    N, IC, H, W, OC, KH, KW, sH, sW, pH, pW = shape
    OH, OW = (H + 2 * pH - KH) // sH + 1, (W + 2 * pW - KW) // sW + 1
    x = gen.relu_like(21, N, IC, H, W)
    go = gen.normal_like(22, N, OC, OH, OW)
    if special == "tiny":
        x, go = _tiny(x, 1), _tiny(go, 1)
    elif special:
        x.view(-1)[::89] = float("inf")
        go.view(-1)[::61] = 0.0
    if special or N > 2:
        go[:, 0] = 0.0  # a whole output channel of zero gradients: results are exact zeros
    got = ops.conv2d_grad_kernel(x.cuda(), (OC, IC, KH, KW), go.cuda(), (sH, sW), (pH, pW)).cpu()
    assert _same(got, oracle.conv2d_grad_kernel(go, x, KH, KW, sH, sW, pH, pW))


def test_large_launch():
    """Launches of 4096 workgroups of 128 pixels: the size from which the two-wave kernel
    keeps its 128-pixel tiles (smaller launches, all the shapes above, take 64-pixel tiles)."""
    from repdl_amd import ops

    x = gen.relu_like(31, 64, 16, 64, 128)
    w = gen.normal_like(32, 64, 16, 3, 3)
    got = ops.conv2d(x.cuda(), w.cuda(), (1, 1), (1, 1), 1)
    assert gen.sha256(got) == gen.sha256(oracle.conv2d(x, w, 1, 1, 1, 1, 1))
    go = gen.normal_like(33, 64, 16, 64, 128)
    w2 = gen.normal_like(34, 16, 64, 3, 3)
    got = ops.conv2d_grad_input((64, 64, 64, 128), w2.cuda(), go.cuda(), (1, 1), (1, 1))
    assert gen.sha256(got) == gen.sha256(oracle.conv2d_grad_input(go, w2, 64, 128, 1, 1, 1, 1))


@pytest.mark.parametrize("layer", [(64, 64, 56, 56, 64, 3, 1, 1), (64, 256, 56, 56, 64, 1, 1, 0)], ids=["3x3_64_64", "1x1_256_64"])
def test_benchmark_layers_full_size(layer, matrix_path):
    """The two convolution layers of the benchmark configuration at full size (batch 64, 56x56),
    all three operators, every output bit against the oracle."""
    from repdl_amd import ops

    N, IC, H, W, OC, Kk, st, pd = layer
    g = torch.Generator().manual_seed(5)
    x = torch.randn(N, IC, H, W, generator=g).clamp_(min=0)
    w = torch.randn(OC, IC, Kk, Kk, generator=g) * (2.0 / (IC * Kk * Kk)) ** 0.5
    OH = (H + 2 * pd - Kk) // st + 1
    go = torch.randn(N, OC, OH, OH, generator=g)
    xd, wd, god = x.cuda(), w.cuda(), go.cuda()
    assert gen.sha256(ops.conv2d(xd, wd, (st, st), (pd, pd), 1)) == gen.sha256(oracle.conv2d(x, w, st, st, pd, pd, 1))
    assert gen.sha256(ops.conv2d_grad_input(x.shape, wd, god, (st, st), (pd, pd))) == gen.sha256(
        oracle.conv2d_grad_input(go, w, H, W, st, st, pd, pd))
    if matrix_path == "matrix":  # the v_fma_f32 grad-kernel needs seconds at this size; the golden cases cover it
        assert gen.sha256(ops.conv2d_grad_kernel(xd, w.shape, god, (st, st), (pd, pd))) == gen.sha256(
            oracle.conv2d_grad_kernel(go, x, Kk, Kk, st, st, pd, pd))
