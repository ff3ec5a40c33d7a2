"""Every kernel family of the library is reached and gives the reference's bits.

mm picks a tile by a cost model, the convolutions a route by shape, alignment and the matrix
path, the sums by the number and length of their chains.  A retuned constant can leave a family
without any shape that reaches it, and the other tests would go on passing.  Here every family
the library names (repdl_hip_route_name) has a case that must take it -- the library reports
which families launched (repdl_hip_routes_taken) -- and whose result is held against the oracle
(whole, or the rows / images the oracle finishes in seconds) and, for the matrix kernels, against
the v_fma_f32 kernels' result on every bit.  A family without a case fails the last test."""
import ctypes

import pytest
import torch

import gen
from oracle import api as oracle

pytestmark = pytest.mark.gpu

P = ctypes.c_void_p


def _lib():
    from repdl_amd import _lib

    return _lib


def _names():
    lib, out, i = _lib().lib(), [], 0
    while lib.repdl_hip_route_name(i) is not None:
        out.append(lib.repdl_hip_route_name(i).decode())
        i += 1
    return out


def _taken():
    mask = _lib().lib().repdl_hip_routes_taken(1)
    return {n for i, n in enumerate(_names()) if mask >> i & 1}


def _bits(t):
    return t.cpu().view(torch.int32)


def _same(got, want):
    got, want = got.cpu(), want.cpu()
    nan = torch.isnan(want)
    return torch.equal(torch.isnan(got), nan) and torch.equal(_bits(got)[~nan], _bits(want)[~nan])


def _matrix(on):
    lib = _lib()
    lib.call("repdl_hip_set_matrix_path", -1 if on else 0)
    assert lib.lib().repdl_hip_matrix_path() == (1 if on else 0)


@pytest.fixture(autouse=True)
def _restore_matrix_path():
    yield
    _lib().call("repdl_hip_set_matrix_path", -1)


# route -> (M, N, K, transA, transB)
MM = {
    "mm_128": (2048, 4096, 64, 0, 0),
    "mm_128_tall": (256, 512, 2048, 1, 0),       # chains four times as long as C is wide, both operands row-contiguous... see below
    "mm_64_four_buffers": (1024, 2048, 2048, 0, 1),
    "mm_64_deep": (1024, 1024, 2048, 0, 1),
    "mm_64_wide_k": (1024, 1024, 1000, 1, 0),
    "mm_64_three_buffers": (1024, 2048, 512, 0, 0),
    "mm_64_movers": (1024, 1024, 512, 1, 1),
    "mm_64_quad": (2048, 2048, 64, 0, 1),
    "mm_32": (256, 256, 300, 0, 0),
    "mm_64x32": (128, 4096, 256, 0, 1),
    "mm_unaligned_128": (2048, 4096, 65, 0, 0),
    "mm_unaligned_64_movers": (1024, 1024, 513, 0, 1),
    "mm_unaligned_64": (1024, 2048, 513, 0, 1),
    "mm_unaligned_quad": (2048, 2048, 65, 0, 1),
    "mm_unaligned_32": (256, 256, 301, 0, 0),
}
# the tall form needs the 128x128 tile to win the cost model: two rounds of 128x128 tiles, TN, K >= 4 max(M, N)
MM["mm_128_tall"] = (2048, 4096, 16384, 1, 0)
COVERED = set()


@pytest.mark.parametrize("route", sorted(MM))
def test_mm_tiles(route):
    from repdl_amd import ops

    M, N, K, tA, tB = MM[route]
    a = gen.normal_like(1, *((K, M) if tA else (M, K)))
    b = gen.normal_like(2, *((N, K) if tB else (K, N)))
    ad, bd = a.cuda(), b.cuda()
    _matrix(True)
    _taken()
    got = ops.mm(ad, bd, bool(tA), bool(tB))
    torch.cuda.synchronize()
    assert _taken() == {route}
    rows = 16  # the oracle on a slab of output rows; every bit against the v_fma_f32 kernels
    slab = a[:, :rows].contiguous() if tA else a[:rows]
    assert torch.equal(_bits(got[:rows]), _bits(oracle.mm(slab, b, bool(tA), bool(tB))))
    _matrix(False)
    ref = ops.mm(ad, bd, bool(tA), bool(tB))
    torch.cuda.synchronize()
    assert _taken() == {"mm_fma"}
    assert torch.equal(_bits(got), _bits(ref))
    COVERED.update({route, "mm_fma"})


# route -> (which, (N, IC, H, W, OC, KH, KW, sH, sW, pH, pW), matrix path, images the oracle checks)
CONV = {
    "conv_patch_16": ("fwd", (64, 128, 28, 28, 128, 3, 3, 1, 1, 1, 1), True, 1),  # (a large launch whose wide tiles would waste more)
    "conv_patch_4": ("dgrad", (3, 64, 7, 7, 64, 3, 3, 1, 1, 1, 1), True, 3),        # (an image of one narrow tile)
    "conv_patch_16_wide": ("fwd", (2, 32, 20, 24, 64, 3, 3, 1, 1, 1, 1), True, 2),
    "conv_patch_4_wide": ("dgrad", (3, 64, 14, 14, 64, 3, 3, 1, 1, 1, 1), True, 3),
    "conv_point": ("fwd", (2, 32, 33, 40, 64, 1, 1, 1, 1, 0, 0), True, 2),
    "conv_point_mm": ("dgrad", (3, 128, 33, 40, 192, 1, 1, 1, 1, 0, 0), True, 3),
    "conv_padded_64_half": ("fwd", (2, 32, 19, 19, 64, 3, 3, 2, 2, 1, 1), True, 2),
    "conv_padded_64": ("fwd", (128, 16, 64, 64, 64, 5, 5, 1, 1, 2, 2), True, 1),
    "conv_padded_128": ("fwd", (1, 16, 12, 40, 128, 5, 5, 1, 2, 1, 3), True, 1),
    "conv_gather_64": ("fwd", (2, 8, 14, 14, 24, 3, 3, 1, 1, 1, 1), False, 2),
    "conv_gather_128": ("dgrad", (2, 96, 20, 20, 72, 1, 1, 1, 1, 0, 0), False, 2),
    "conv_im2col": ("dgrad", (32, 128, 9, 9, 128, 5, 3, 2, 1, 2, 1), True, 4),
    "dgrad_point_scatter": ("dgrad", (2, 64, 56, 56, 128, 1, 1, 2, 2, 0, 0), True, 2),
    "dgrad_residues": ("dgrad", (64, 64, 56, 56, 128, 3, 3, 2, 2, 1, 1), True, 2),
    "wgrad_point_gather": ("wgrad", (3, 16, 30, 28, 32, 1, 1, 2, 2, 0, 0), True, 3),
    "wgrad_product": ("wgrad", (4, 64, 7, 7, 512, 3, 3, 1, 1, 1, 1), True, 4),
    "wgrad_chain": ("wgrad", (3, 20, 18, 16, 40, 3, 3, 1, 1, 1, 1), True, 3),
    "wgrad_fma": ("wgrad", (1, 2, 8, 70, 3, 1, 3, 1, 17, 0, 1), True, 1),
}


def _conv(which, x, w, go, dims):
    from repdl_amd import ops

    N, IC, H, W, OC, KH, KW, sH, sW, pH, pW = dims
    if which == "fwd":
        return ops.conv2d(x, w, (sH, sW), (pH, pW), 1)
    if which == "dgrad":
        return ops.conv2d_grad_input((x.shape[0], IC, H, W), w, go, (sH, sW), (pH, pW))
    return ops.conv2d_grad_kernel(x, (OC, IC, KH, KW), go, (sH, sW), (pH, pW))


@pytest.mark.parametrize("route", sorted(CONV))
def test_convolution_routes(route):
    which, dims, matrix, nimg = CONV[route]
    N, IC, H, W, OC, KH, KW, sH, sW, pH, pW = dims
    OH, OW = (H + 2 * pH - KH) // sH + 1, (W + 2 * pW - KW) // sW + 1
    x, w, go = gen.relu_like(3, N, IC, H, W), gen.normal_like(4, OC, IC, KH, KW), gen.normal_like(5, N, OC, OH, OW)
    xd, wd, god = x.cuda(), w.cuda(), go.cuda()
    _matrix(matrix)
    _taken()
    got = _conv(which, xd, wd, god, dims)
    torch.cuda.synchronize()
    taken = _taken()
    assert route in taken, (route, taken)
    if which == "wgrad":  # every image is part of every chain
        assert nimg == N
        want = oracle.conv2d_grad_kernel(go, x, KH, KW, sH, sW, pH, pW)
        assert _same(got, want)
    elif which == "fwd":
        assert _same(got[:nimg], oracle.conv2d(x[:nimg], w, sH, sW, pH, pW, 1))
    else:
        assert _same(got[:nimg], oracle.conv2d_grad_input(go[:nimg].contiguous(), w, H, W, sH, sW, pH, pW))
    _matrix(not matrix)  # the other implementation of the same chains, every bit
    other = _conv(which, xd, wd, god, dims)
    torch.cuda.synchronize()
    assert _same(got, other)
    COVERED.update(taken | _taken())


def test_sum_and_loss_routes():
    from repdl_amd import ops

    cases = {
        "sum_row_walk": lambda: (ops.sum2d_dim1, oracle.sum2d_dim1, gen.normal_like(6, 100, 333)),
        "sum_chains": lambda: (ops.sum4d_dim023, oracle.sum4d_dim023, gen.normal_like(7, 16, 24, 56, 56)),
        "sum_chains_rounds": lambda: (ops.sum1d, oracle.sum1d, gen.uniform_pm1(8, 1 << 22)),
        "sum_column_walk": lambda: (ops.sum2d_dim0, oracle.sum2d_dim0, gen.normal_like(9, 333, 100)),
        "sum_serial": lambda: (ops.sum1d, oracle.sum1d, gen.uniform_pm1(10, 1000)),
        "loss_onchip": lambda: (ops.softmax, oracle.softmax, gen.normal_like(11, 4096, 100)),
        "loss_row_per_wave": lambda: (ops.softmax, oracle.softmax, gen.normal_like(12, 64, 10)),
    }
    for route, make in cases.items():
        fn, ofn, x = make()
        _taken()
        got = fn(x.cuda())
        torch.cuda.synchronize()
        taken = _taken()
        assert route in taken, (route, taken)
        assert torch.equal(_bits(got), _bits(ofn(x))), route
        COVERED.update(taken)


def test_every_family_has_a_case():
    """(runs after the tests above in this file; alone it has nothing to count and is skipped)"""
    if not COVERED:
        pytest.skip("the cases of this file have not run in this process")
    assert set(MM) | set(CONV) <= set(_names())
    assert set(_names()) - COVERED == set()
