"""softmax and cross_entropy on the GPU against the oracle for shapes on both sides of the row
count (4096) and the row length (4096) at which the library changes from a wave per row to
workgroups that hold 4 to 64 rows on chip: row lengths around every change of rows per
workgroup (64, 128, 256, 512, 1024, 2048), lengths that are no multiple of 4 (scalar loads), a
base pointer that is not 16-byte aligned, row counts that do not fill the last workgroup,
logits of very different magnitude and -inf entries (exp gives exact zeros inside the serial
sums)."""
import pytest
import torch

import gen
from oracle import api as oracle

pytestmark = pytest.mark.gpu

SHAPES = [(4095, 10), (4096, 10), (4097, 1), (4100, 63), (4160, 64), (4099, 65), (5000, 130), (4096, 1000), (8192, 257),
          (70000, 12), (4200, 4), (4101, 128), (4098, 256), (4097, 258), (4100, 512), (4099, 515), (4096, 1024), (4097, 1028),
          (4098, 2048), (4097, 2050), (4099, 4096), (4097, 4097), (4096, 3001),
          (1024, 2048), (1023, 2050), (1500, 1399), (2047, 1024), (2049, 1023)]


def _logits(seed, M, N):
    x = gen.normal_like(seed, M, N) * 6
    x.view(-1)[::37] *= 20          # rows with one dominant logit
    x.view(-1)[5::101] = -float("inf")
    x[3] = 1.25                     # a constant row
    if N > 1:
        x[7, 1:] = -float("inf")    # a row that is one value and zeros after exp
    return x


@pytest.mark.parametrize("shape", SHAPES, ids=str)
def test_softmax_many_rows(shape):
    from repdl_amd import ops

    M, N = shape
    x = _logits(300 + N, M, N)
    want = oracle.softmax(x)
    got = ops.softmax(x.cuda()).cpu()
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))


@pytest.mark.parametrize("shape", SHAPES, ids=str)
def test_cross_entropy_many_rows(shape):
    from repdl_amd import ops

    M, N = shape
    x = _logits(400 + N, M, N)
    x[7] = gen.normal_like(1, N)    # keep every target's logit finite: -inf - max is fine, but the loss must stay finite
    x.view(-1)[5::101] = -50.0
    t = gen.labels(401 + N, M, N)
    want = oracle.cross_entropy(x, t)
    got = ops.cross_entropy(x.cuda(), t.cuda()).cpu()
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))


def test_unaligned_base_pointer():
    from repdl_amd import ops

    M, N = 4500, 68
    x = _logits(500, M, N)
    flat = torch.cat([torch.zeros(1), x.view(-1)]).cuda()
    xd = flat[1:].view(M, N)
    assert xd.data_ptr() % 16 != 0
    assert torch.equal(ops.softmax(xd).cpu().view(torch.int32), oracle.softmax(x).view(torch.int32))
    t = gen.labels(501, M, N)
    x2 = x.clamp(min=-80.0)
    xd2 = torch.cat([torch.zeros(1), x2.view(-1)]).cuda()[1:].view(M, N)
    assert torch.equal(ops.cross_entropy(xd2, t.cuda()).cpu().view(torch.int32), oracle.cross_entropy(x2, t).view(torch.int32))
