"""GPU parity of mm against the oracle beyond the golden cases: all four layouts on
tile-edge shapes, K tails, unaligned pointers, and the larger Linear shapes."""
import pytest
import torch

import gen
from oracle import api as oracle

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("matrix_path")]

SHAPES = [(128, 128, 16), (127, 129, 15), (257, 130, 1000), (1, 513, 77), (640, 1, 3), (384, 256, 2049), (2, 2, 2)]


@pytest.mark.parametrize("tA,tB", [(0, 0), (1, 0), (0, 1), (1, 1)])
@pytest.mark.parametrize("shape", SHAPES, ids=[str(s) for s in SHAPES])
def test_layouts_and_edges(shape, tA, tB):
    from repdl_amd import ops

    M, N, K = shape
    a = gen.scaled_normal(M * 7 + K, *((K, M) if tA else (M, K)), lo=-6, hi=6)
    b = gen.normal_like(N * 3 + K, *((N, K) if tB else (K, N)))
    got = ops.mm(a.cuda(), b.cuda(), bool(tA), bool(tB)).cpu()
    assert torch.equal(got, oracle.mm(a, b, bool(tA), bool(tB)))


# Operands whose rows start on 16-byte boundaries take the kernel that moves them from global memory
# straight into LDS.  Whole-tile shapes for each of its tile configurations (128x128; 64x64 with the
# shallow and the deep k-tile; 32x32; 64x32), then shapes that hang over the tile edges, K that
# leaves a tail behind the last whole k-tile, K shorter than one k-tile, and the smallest extents.
WHOLE_TILE_SHAPES = [(4096, 4096, 48), (2048, 2048, 80), (512, 512, 96), (512, 512, 48), (64, 1024, 128), (48, 1024, 192),
                     (256, 192, 128), (128, 128, 2048),
                     (260, 132, 1000), (100, 36, 52), (4, 4, 4), (68, 20, 24), (1028, 2052, 36), (2500, 1300, 76), (8, 4100, 12),
                     (132, 260, 1001), (64, 64, 71), (512, 512, 2), (128, 4096, 72), (132, 4100, 40),
                     (768, 772, 1102), (772, 768, 100), (1100, 1092, 52),
                     (770, 771, 1101), (1029, 2051, 37), (2501, 1299, 75), (4097, 4099, 21)]

@pytest.mark.parametrize("tA,tB", [(0, 0), (1, 0), (0, 1), (1, 1)])
@pytest.mark.parametrize("shape", WHOLE_TILE_SHAPES, ids=str)
def test_whole_tile_shapes(shape, tA, tB):
    """Operands with zeros of both signs, subnormals, huge and tiny magnitudes and infinities
    (NaN results only have to be NaN), then well-scaled operands with a bias."""
    from repdl_amd import ops

    M, N, K = shape
    a = gen.elementwise_mix(M + 3 * K, M * K).view((K, M) if tA else (M, K))
    b = gen.elementwise_mix(N + 5 * K, N * K).view((N, K) if tB else (K, N))
    a = torch.where(torch.isnan(a), torch.zeros_like(a), a)
    b = torch.where(torch.isnan(b), torch.full_like(b, -0.0), b)
    got = ops.mm(a.cuda(), b.cuda(), bool(tA), bool(tB)).cpu()
    assert _same_bits_or_both_nan(got, oracle.mm(a, b, bool(tA), bool(tB)))
    a = gen.scaled_normal(M * 7 + K, *((K, M) if tA else (M, K)), lo=-6, hi=6)
    b = gen.normal_like(N * 3 + K, *((N, K) if tB else (K, N)))
    bias = gen.scaled_normal(N + 1, N, lo=-30, hi=30)
    bias[::5] = 0.0
    bias[1::7] = -0.0
    want = oracle.mm(a, b, bool(tA), bool(tB))
    got = ops.mm(a.cuda(), b.cuda(), bool(tA), bool(tB)).cpu()
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    want += bias
    got = ops.mm_bias(a.cuda(), b.cuda(), bias.cuda(), bool(tA), bool(tB)).cpu()
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))


def test_edge_of_the_largest_tile():
    """Enough tiles that the 128x128 configuration is chosen, with a last tile-row of four rows."""
    from repdl_amd import ops

    M, N, K = 8196, 8192, 20
    a = gen.scaled_normal(5, M, K, lo=-6, hi=6)
    b = gen.normal_like(6, K, N)
    got = ops.mm(a.cuda(), b.cuda()).cpu()
    assert torch.equal(got.view(torch.int32), oracle.mm(a, b).view(torch.int32))


@pytest.mark.parametrize("tA,tB", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("shape", SHAPES + [(512, 768, 256), (300, 1000, 64)], ids=str)
def test_bias_in_the_epilogue(shape, tA, tB):
    """mm_bias = mm followed by one rounded `+= bias` (repdl/nn/linear.py:21-22), on every kernel
    variant: whole tiles, edge tiles, the general kernel; bias values that cancel, dwarf and vanish
    against the products, and signed zeros (-0 + +0 = +0, -0 + -0 = -0)."""
    from repdl_amd import ops

    M, N, K = shape
    a = gen.scaled_normal(M * 5 + K, *((K, M) if tA else (M, K)), lo=-6, hi=6)
    b = gen.normal_like(N * 11 + K, *((N, K) if tB else (K, N)))
    bias = gen.scaled_normal(N + 1, N, lo=-30, hi=30)
    bias[::5] = 0.0
    bias[1::7] = -0.0
    a[0] = 0.0  # a row of zero chains: the result is the bias with the zero's sign rules
    want = oracle.mm(a, b, bool(tA), bool(tB))
    want += bias
    got = ops.mm_bias(a.cuda(), b.cuda(), bias.cuda(), bool(tA), bool(tB)).cpu()
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    none = ops.mm_bias(a.cuda(), b.cuda(), None, bool(tA), bool(tB)).cpu()
    assert torch.equal(none.view(torch.int32), oracle.mm(a, b, bool(tA), bool(tB)).view(torch.int32))


def test_rows_longer_than_32_bit_tile_offsets():
    """Rows of 2^25 + 4 elements: a 32-row operand tile spans more than 2^32 bytes, which the kernel that
    moves tiles global->LDS with 32-bit lane offsets declines; the product must come out right anyway."""
    from repdl_amd import ops

    M, N, K = 4, 4, (1 << 25) + 4
    rng = torch.Generator().manual_seed(11)
    a = torch.randint(-3, 4, (M, K), generator=rng).float()
    b = torch.randint(-3, 4, (N, K), generator=rng).float()
    a[:, ::3] *= 0.37  # products and partial sums round
    got = ops.mm(a.cuda(), b.cuda(), False, True).cpu()
    want = oracle.mm(a, b, False, True)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    # the same with the long rows in an operand whose k runs down the columns
    a2 = torch.randint(-3, 4, (2, 6), generator=rng).float() * 0.37
    b2 = torch.randint(-3, 4, (6, K), generator=rng).float()
    got = ops.mm(a2.cuda(), b2.cuda()).cpu()
    assert torch.equal(got.view(torch.int32), oracle.mm(a2, b2).view(torch.int32))


def test_unaligned_operands():
    from repdl_amd import ops

    M, N, K = 100, 96, 64
    buf_a = gen.normal_like(1, M * K + 3).cuda()
    buf_b = gen.normal_like(2, K * N + 3).cuda()
    a = buf_a[1:1 + M * K].view(M, K)
    b = buf_b[3:3 + K * N].view(K, N)
    assert a.data_ptr() % 16 and b.data_ptr() % 16 and a.is_contiguous()
    assert torch.equal(ops.mm(a, b).cpu(), oracle.mm(a.cpu(), b.cpu()))
    # non-contiguous views are made contiguous by the host layer
    at = gen.normal_like(3, K, M).cuda().t()
    assert torch.equal(ops.mm(at, b).cpu(), oracle.mm(at.cpu().contiguous(), b.cpu()))


@pytest.mark.parametrize("shape", [(2048, 2048, 2048, 0, 1), (1024, 1024, 8192, 0, 0), (1024, 1024, 16384, 1, 0)])
def test_linear_shapes(shape):
    """Scaled-down versions of the BASELINE config-4 Linear shapes (forward NT, the
    long-K NN / TN weight-gradient form), full output compared."""
    from repdl_amd import ops

    M, N, K, tA, tB = shape
    g = torch.Generator().manual_seed(M + K)
    a = torch.randn((K, M) if tA else (M, K), generator=g)
    b = torch.randn((N, K) if tB else (K, N), generator=g)
    got = ops.mm(a.cuda(), b.cuda(), bool(tA), bool(tB)).cpu()
    assert gen.sha256(got) == gen.sha256(oracle.mm(a, b, bool(tA), bool(tB)))


def test_determinism():
    from repdl_amd import ops

    a, b = gen.normal_like(5, 700, 900).cuda(), gen.normal_like(6, 900, 500).cuda()
    h = {gen.sha256(ops.mm(a, b)) for _ in range(5)}
    assert len(h) == 1


def _same_bits_or_both_nan(got, want):
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan)
    return torch.equal(got.view(torch.int32)[~nan], want.view(torch.int32)[~nan])


@pytest.mark.parametrize("tA,tB", [(0, 1), (1, 0)])
def test_special_values(tA, tB):
    """Zeros of both signs, subnormals, products that underflow or overflow, infinities:
    the chains must still agree bit for bit (NaN results only have to be NaN)."""
    from repdl_amd import ops

    M, N, K = 200, 136, 333
    a = gen.elementwise_mix(11, M * K).view((K, M) if tA else (M, K))
    b = gen.elementwise_mix(12, N * K).view((N, K) if tB else (K, N))
    a = torch.where(torch.isnan(a), torch.zeros_like(a), a)
    b = torch.where(torch.isnan(b), torch.full_like(b, -0.0), b)
    got = ops.mm(a.cuda(), b.cuda(), bool(tA), bool(tB)).cpu()
    assert _same_bits_or_both_nan(got, oracle.mm(a, b, bool(tA), bool(tB)))
    # tiny magnitudes: every product is subnormal or underflows, sums of signed zeros
    a = gen.scaled_normal(13, M, K, lo=-90, hi=-70)
    b = gen.scaled_normal(14, K, N, lo=-80, hi=-60) * gen.relu_like(15, K, N).sign()
    got = ops.mm(a.cuda(), b.cuda()).cpu()
    want = oracle.mm(a, b)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    assert (want.abs() < 2.0 ** -126).all() and (want != 0).any()


@pytest.mark.parametrize("K", [1, 2, 3, 15, 16, 17, 31, 33])
def test_k_tails_keep_negative_zero(K):
    """A K that does not fill the last tile must not disturb an accumulator that is -0."""
    from repdl_amd import ops

    a = torch.full((70, K), -1e-30)
    b = torch.full((K, 40), 1e-30)  # every product rounds to -0, so every result is -0
    got = ops.mm(a.cuda(), b.cuda()).cpu()
    want = oracle.mm(a, b)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    assert (want.view(torch.int32) == -(2 ** 31)).all()


@pytest.mark.parametrize("shape", [(8192, 8192, 8192, 0, 1), (4096, 4096, 32768, 0, 0), (4096, 4096, 32768, 0, 1),
                                   (4096, 4096, 65536, 1, 0)], ids=str)
def test_full_size_shapes(shape):
    """The Linear shapes at their full sizes (forward NT, the long-K products, the weight
    gradient with the batch as K).  The CPU oracle needs minutes for one of these, so the whole
    output is checked through a property -- the matrix-instruction kernel and the v_fma_f32 kernel,
    two independent evaluations of the same chains, must agree in every bit -- and a slab of
    rows is checked against the oracle itself."""
    from repdl_amd import _lib, ops

    M, N, K, tA, tB = shape
    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    a = torch.randn((K, M) if tA else (M, K), generator=g, device="cuda")
    b = torch.randn((N, K) if tB else (K, N), generator=g, device="cuda")
    got = ops.mm(a, b, bool(tA), bool(tB))
    mode = _lib.lib().repdl_hip_matrix_path()
    _lib.call("repdl_hip_set_matrix_path", 0 if mode == 1 else -1)
    other = ops.mm(a, b, bool(tA), bool(tB))
    _lib.call("repdl_hip_set_matrix_path", 0 if mode == 0 else -1)
    assert torch.equal(got.view(torch.int32), other.view(torch.int32))
    del other
    rows = 16
    a_slab = (a[:, :rows] if tA else a[:rows]).contiguous().cpu()
    want = oracle.mm(a_slab, b.cpu(), bool(tA), bool(tB))
    assert torch.equal(got[:rows].cpu().view(torch.int32), want.view(torch.int32))
