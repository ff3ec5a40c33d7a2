"""repdl_hip_sum1d_static -- the sum1d entry point that allocates nothing (its scratch is a
fixed array inside the library) -- against repdl_hip_sum1d, bit for bit, through the C ABI:
two calls in a row on one device, the second on a smaller input (the array still holds the
first call's contents), then the serial range, the capacity limit and a third call."""
import ctypes

import pytest
import torch

import gen

pytestmark = pytest.mark.gpu


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(x, average):
    from repdl_amd import _lib

    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    want = torch.full((1,), 7.0, device="cuda")
    got = torch.full((1,), 9.0, device="cuda")
    _lib.call("repdl_hip_sum1d", _p(x), _p(want), x.numel(), average, stream)
    _lib.call("repdl_hip_sum1d_static", _p(x), _p(got), x.numel(), average, stream)
    torch.cuda.synchronize()
    return got.cpu().view(torch.int32).item(), want.cpu().view(torch.int32).item()


def test_static_scratch_matches_allocating_entry_point():
    from repdl_amd import _lib

    lib = _lib.lib()
    cap = lib.repdl_hip_sum1d_static_max_n()
    assert 1 << 22 <= cap <= 1 << 26
    big = gen.uniform_pm1(21, 3_000_000).cuda()
    small = (gen.uniform_pm1(22, 200_003) * 3 + 0.25).cuda()
    for x, avg in ((big, 0), (small, 1), (big[: 1 << 20], 0), (small[:1000], 0), (big, 1)):
        got, want = _both(x.contiguous(), avg)
        assert got == want, (x.numel(), avg)
    # beyond the capacity: refused with its own code, nothing launched, nothing allocated
    out = torch.zeros(1, device="cuda")
    rc = lib.repdl_hip_sum1d_static(_p(big), _p(out), cap + 1, 0, None)
    assert rc == -4
    assert b"capacity" in lib.repdl_hip_error_string(rc)
    # the largest admissible length (only the library reads that far: the buffer is that long)
    full = gen.uniform_pm1(23, cap).cuda()
    got, want = _both(full, 0)
    assert got == want
