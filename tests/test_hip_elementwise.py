"""GPU parity of the elementwise operators against the CPU oracle (which calls the
host's glibc / IEEE hardware exactly as the reference does): the config-3 value
mix, every pair of special values, odd lengths and unaligned pointers, and a
sweep over ALL 2^32 binary32 bit patterns for exp, log, sqrt and x/10."""
import numpy as np
import pytest
import torch

import gen
from oracle import api as oracle

pytestmark = pytest.mark.gpu


def _ops():
    from repdl_amd import ops

    return ops


def _same_bits(a: torch.Tensor, b: torch.Tensor) -> bool:
    return torch.equal(a.cpu().view(torch.int32), b.cpu().view(torch.int32))


@pytest.mark.parametrize("name", ["exp", "log", "sqrt"])
@pytest.mark.parametrize("n", [1, 3, 4, 5, 1023, 16384 * 4 + 7, 1 << 22])
def test_unary_mix(name, n):
    x = gen.elementwise_mix(100 + n % 97, n)
    got = getattr(_ops(), name)(x.cuda())
    assert _same_bits(got, getattr(oracle, name)(x)), name


@pytest.mark.parametrize("name", ["exp", "log", "sqrt"])
def test_unary_unaligned_and_shaped(name):
    ops = _ops()
    buf = gen.elementwise_mix(7, 5000).cuda()
    x = buf[1:4098]  # data pointer is 4 bytes off a 16-byte boundary
    assert x.data_ptr() % 16 != 0
    assert _same_bits(getattr(ops, name)(x), getattr(oracle, name)(x.cpu()))
    y = gen.elementwise_mix(8, 6 * 35).reshape(6, 35).cuda()
    out = getattr(ops, name)(y)
    assert out.shape == y.shape and _same_bits(out, getattr(oracle, name)(y.cpu()))
    t = y.t()  # non-contiguous input
    assert _same_bits(getattr(ops, name)(t), getattr(oracle, name)(t.cpu().contiguous()))


def test_div_mix_and_specials():
    ops = _ops()
    a, b = gen.elementwise_mix(11, 1 << 22), gen.elementwise_mix(12, 1 << 22)
    assert _same_bits(ops.div(a.cuda(), b.cuda()), oracle.div(a, b))
    sp = torch.from_numpy(gen.SPECIAL_BITS.view(np.float32).copy())
    A, B = sp.repeat_interleave(len(sp)), sp.repeat(len(sp))
    assert _same_bits(ops.div(A.cuda(), B.cuda()), oracle.div(A, B))
    assert _same_bits(ops.div(A.cuda(), B.cuda()), A.div(B))  # PyTorch CPU is what RepDL's div calls
    for d in (10.0, 3.0, -0.1, 1e-40, 3e38, 0.0, float("inf"), float("nan")):
        assert _same_bits(ops.div(a.cuda(), d), oracle.div(a, d)), d
        assert _same_bits(ops.div(a.cuda(), d), a.div(torch.tensor(d))), d
    # a 0-dim tensor divisor and broadcasting
    assert _same_bits(ops.div(a.cuda(), torch.tensor(10.0).cuda()), oracle.div(a, 10.0))
    m, col = gen.normal_like(13, 33, 17), gen.normal_like(14, 33, 1)
    assert _same_bits(ops.div(m.cuda(), col.cuda()), m.div(col))
    assert _same_bits(ops.div(a[1:1001].cuda(), b[3:1003].cuda()), oracle.div(a[1:1001], b[3:1003]))


def test_div_tensor_by_tensor_at_full_size():
    """The 2^28-element launch of the elementwise configuration (x / y, both from the value mix), every
    output against the oracle and against PyTorch CPU's x.div(y), which is what RepDL's div is
    (repdl/ops.py:98-103)."""
    n = 1 << 28
    a, b = gen.elementwise_mix(3, n), gen.elementwise_mix(4, n)
    got = _ops().div(a.cuda(), b.cuda()).cpu()
    assert _same_bits(got, oracle.div(a, b))
    assert _same_bits(got, a.div(b))


def test_sqrt_matches_torch_cpu_convention():
    ops = _ops()
    x = gen.elementwise_mix(15, 1 << 20)
    assert _same_bits(ops.sqrt(x.cuda()), x.to(torch.float64).sqrt().to(torch.float32))


@pytest.mark.parametrize("name", ["exp", "log", "sqrt", "div10"])
def test_all_bit_patterns(name):
    """2^32 inputs in 64 chunks of 2^26; the host side runs the oracle in parallel."""
    ops = _ops()
    chunk = 1 << 26
    base = torch.arange(chunk, dtype=torch.int64, device="cuda")
    for c in range((1 << 32) // chunk):
        bits = (base + c * chunk).to(torch.int32) if c < 32 else (base + (c * chunk - (1 << 32))).to(torch.int32)
        x = bits.view(torch.float32)
        if name == "div10":
            got, want = ops.div(x, 10.0), oracle.div(x.cpu(), 10.0)
        else:
            got, want = getattr(ops, name)(x), getattr(oracle, name)(x.cpu())
        same = _same_bits(got, want)
        if not same:
            g, w = got.cpu().view(torch.int32), want.view(torch.int32)
            idx = (g != w).nonzero().flatten()[:8]
            bad = [(hex(int(bits[i]) & 0xFFFFFFFF), hex(int(g[i]) & 0xFFFFFFFF), hex(int(w[i]) & 0xFFFFFFFF)) for i in idx]
            raise AssertionError("%s chunk %d: %s" % (name, c, bad))
        if c % 8 == 7:
            print(name, "chunk", c, "ok", flush=True)
