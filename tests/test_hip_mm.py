"""GPU parity of mm against the oracle beyond the golden cases: all four layouts on
tile-edge shapes, K tails, unaligned pointers, and the larger Linear shapes."""
import pytest
import torch

import gen
from oracle import api as oracle

pytestmark = pytest.mark.gpu

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
