"""The two sources of scratch memory, through the C ABI:

* every entry point that takes scratch gives the same bits with the caller's workspace
  (`*_ws`, sized by `*_workspace_bytes`, here off every alignment and with canaries either side)
  as with the library's cache, on layers that take each of the convolution routes, on both
  settings of the matrix path; a workspace that is too small is refused;
* the cache while a stream is captured into a graph: a request it cannot serve from a buffer it
  already holds fails (nothing is allocated under capture), one it can serve pins that buffer --
  a larger eager call afterwards must not move it, and the graph still replays to the eager bits;
* repdl_hip_scratch_trim gives the cache's memory back.
"""
import ctypes

import pytest
import torch

import gen

pytestmark = pytest.mark.gpu

P = ctypes.c_void_p


def _p(t):
    return P(t.data_ptr())


def _stream():
    return P(torch.cuda.current_stream().cuda_stream)


def _bits(t):
    return t.cpu().view(torch.int32)


class _Workspace:
    """nbytes of device memory starting `shift` bytes off a 512-byte boundary, canaries before and after."""

    PAD = 4096

    def __init__(self, nbytes, shift):
        self.nbytes, self.shift = nbytes, shift
        self.buf = torch.full((nbytes + 2 * self.PAD,), 0xA5, dtype=torch.uint8, device="cuda")

    @property
    def ptr(self):
        return P(self.buf.data_ptr() + self.PAD + self.shift) if self.nbytes else None

    def intact(self):
        head = self.buf[: self.PAD + self.shift]
        tail = self.buf[self.PAD + self.shift + self.nbytes:]
        return bool((head == 0xA5).all()) and bool((tail == 0xA5).all())


# (N, IC, H, W, OC, KH, KW, sH, sW, pH, pW): one layer per route of the convolutions
LAYERS = [
    (4, 64, 28, 28, 64, 3, 3, 1, 1, 1, 1),      # input-patch kernel (forward, grad-input), chain kernel (grad-kernel)
    (3, 64, 33, 40, 64, 1, 1, 1, 1, 0, 0),      # 1x1: products per image / the streaming kernel
    (2, 64, 19, 19, 128, 3, 3, 2, 2, 1, 1),     # strides: padded copy of the gathered operand
    (32, 128, 9, 9, 128, 5, 3, 2, 1, 2, 1),     # small images: im2col and one product
    (64, 64, 56, 56, 128, 3, 3, 2, 2, 1, 1),    # grad-input residue by residue (nested calls, each with its own piece)
    (3, 16, 30, 28, 32, 1, 1, 2, 2, 0, 0),      # 1x1 at a stride: gathered, then the stride-1 layer (nested)
    (4, 64, 7, 7, 512, 3, 3, 1, 1, 1, 1),       # grad-kernel as one product over an im2col
    (2, 6, 33, 65, 33, 3, 3, 2, 2, 1, 1),       # grad-kernel with both operands through padded copies
    (2, 5, 11, 12, 9, 2, 3, 1, 1, 0, 1),        # ragged: gather kernels
]


def _conv_calls(layer):
    """(name, query args, call args before the workspace, output shape) for the three convolutions of a layer."""
    N, IC, H, W, OC, KH, KW, sH, sW, pH, pW = layer
    OH, OW = (H + 2 * pH - KH) // sH + 1, (W + 2 * pW - KW) // sW + 1
    x = gen.relu_like(3, N, IC, H, W).cuda()
    w = gen.normal_like(4, OC, IC, KH, KW).cuda()
    go = gen.normal_like(5, N, OC, OH, OW).cuda()
    bias = gen.normal_like(6, OC).cuda()
    return [
        ("conv2d", (x, w), (bias,), (N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, 1), (N, OC, OH, OW)),
        ("conv2d_grad_input", (go, w), (), (N, OC, OH, OW, IC, KH, KW, H, W, sH, sW, pH, pW), (N, IC, H, W)),
        ("conv2d_grad_kernel", (go, x), (), (N, IC, H, W, OC, OH, OW, KH, KW, sH, sW, pH, pW), (OC, IC, KH, KW)),
    ]


@pytest.mark.usefixtures("matrix_path")
@pytest.mark.parametrize("layer", LAYERS, ids=[str(l) for l in LAYERS])
def test_convolutions_with_the_callers_workspace(layer):
    from repdl_amd import _lib

    lib = _lib.lib()
    for i, (name, operands, extra, dims, oshape) in enumerate(_conv_calls(layer)):
        a, b = operands
        want = torch.full(oshape, 3.0, device="cuda")
        plain = "repdl_hip_conv2d_bias" if name == "conv2d" else "repdl_hip_" + name
        _lib.call(plain, _p(a), _p(b), *[_p(e) for e in extra], _p(want), *dims, _stream())
        nbytes = getattr(lib, "repdl_hip_%s_workspace_bytes" % name)(_p(a), _p(b), *dims)
        assert nbytes <= getattr(lib, "repdl_hip_%s_workspace_bytes" % name)(None, None, *dims)
        for shift in (0, 4, 252):
            ws = _Workspace(nbytes, shift)
            got = torch.full(oshape, 5.0, device="cuda")
            _lib.call("repdl_hip_%s_ws" % name, _p(a), _p(b), *[_p(e) for e in extra], _p(got), *dims, ws.ptr,
                      ctypes.c_size_t(nbytes), _stream())
            torch.cuda.synchronize()
            assert torch.equal(_bits(got), _bits(want)), (name, shift)
            assert ws.intact(), (name, shift)
        if nbytes > 0:
            ws = _Workspace(nbytes, 0)
            got = torch.full(oshape, 5.0, device="cuda")
            rc = getattr(lib, "repdl_hip_%s_ws" % name)(_p(a), _p(b), *[_p(e) for e in extra], _p(got), *dims, ws.ptr,
                                                       ctypes.c_size_t(255), _stream())
            torch.cuda.synchronize()
            # refused -- unless this setting of the matrix path needs no scratch at all (the query bounds both)
            assert rc == -3 or (rc == 0 and torch.equal(_bits(got), _bits(want))), (name, rc)
            assert ws.intact()


def test_sums_and_loss_with_the_callers_workspace():
    from repdl_amd import _lib

    lib = _lib.lib()
    rows = gen.uniform_pm1(7, 12 * 70_000).reshape(12, 70_000).cuda()
    chans = gen.normal_like(8, 16, 24, 56, 56).cuda()
    logits = (gen.normal_like(9, 40_000, 37) * 4).cuda()
    target = gen.labels(10, 40_000, 37).cuda()
    cases = [
        ("sum2d_dim1", (rows,), (12, 70_000, 1), (12, 70_000), (12,)),
        ("sum4d_dim023", (chans,), (16, 24, 56, 56, 0), (16, 24, 56, 56), (24,)),
    ]
    for name, ins, dims, qdims, oshape in cases:
        want, got = torch.full(oshape, 3.0, device="cuda"), torch.full(oshape, 5.0, device="cuda")
        _lib.call("repdl_hip_" + name, *[_p(t) for t in ins], _p(want), *dims, _stream())
        nbytes = getattr(lib, "repdl_hip_%s_workspace_bytes" % name)(*qdims)
        assert nbytes > 0
        for shift in (0, 12):
            ws = _Workspace(nbytes, shift)
            _lib.call("repdl_hip_%s_ws" % name, *[_p(t) for t in ins], _p(got), *dims, ws.ptr, ctypes.c_size_t(nbytes), _stream())
            torch.cuda.synchronize()
            assert torch.equal(_bits(got), _bits(want)) and ws.intact(), (name, shift)
        assert getattr(lib, "repdl_hip_%s_ws" % name)(*[_p(t) for t in ins], _p(got), *dims, None, ctypes.c_size_t(0), _stream()) == -3
    # cross_entropy: the row losses and the scratch of their mean (40000 rows: the parallel evaluation) in one workspace
    want, got = torch.zeros(1, device="cuda"), torch.ones(1, device="cuda")
    rowloss = torch.empty(40_000, device="cuda")
    _lib.call("repdl_hip_cross_entropy", _p(logits), _p(target), _p(want), 40_000, 37, _p(rowloss), _stream())
    nbytes = lib.repdl_hip_cross_entropy_workspace_bytes(40_000, 37)
    ws = _Workspace(nbytes, 8)
    _lib.call("repdl_hip_cross_entropy_ws", _p(logits), _p(target), _p(got), 40_000, 37, ws.ptr, ctypes.c_size_t(nbytes), _stream())
    torch.cuda.synchronize()
    assert torch.equal(_bits(got), _bits(want)) and ws.intact()


def test_cache_under_stream_capture_and_trim():
    from repdl_amd import _lib

    lib = _lib.lib()
    _lib.init()
    N, IC, H, W, OC = 4, 64, 19, 19, 128
    dims = (N, IC, H, W, OC, 3, 3, 2, 2, 1, 1, 1)  # stride 2: a padded copy of the input in scratch
    x = gen.relu_like(11, N, IC, H, W).cuda()
    w = gen.normal_like(12, OC, IC, 3, 3).cuda()
    y = torch.zeros(N, OC, 10, 10, device="cuda")
    big_dims = (4 * N, IC, H, W, OC, 3, 3, 2, 2, 1, 1, 1)
    xb = gen.relu_like(13, 4 * N, IC, H, W).cuda()
    yb = torch.zeros(4 * N, OC, 10, 10, device="cuda")

    def conv(dst, src, d):
        return lib.repdl_hip_conv2d(_p(src), _p(w), _p(dst), *d, _stream())

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    torch.cuda.synchronize()
    assert lib.repdl_hip_scratch_trim() == 0
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        # nothing on this stream yet: the cache has no buffer and may not allocate one under capture
        with torch.cuda.graph(graph, stream=side):
            rc_cold = conv(y, x, dims)
            y.add_(0.0)  # (so that the graph is not empty)
        assert rc_cold == 900, rc_cold
        assert conv(y, x, dims) == 0  # eager: the cache allocates
        torch.cuda.synchronize()
        want = y.clone()
        held = lib.repdl_hip_scratch_bytes()
        assert held > 0
        graph2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph2, stream=side):
            rc_warm = conv(y, x, dims)
        assert rc_warm == 0
        for rep in range(3):
            y.zero_()
            graph2.replay()
            torch.cuda.synchronize()
            assert torch.equal(_bits(y), _bits(want)), rep
            # a larger eager call on the same stream: the cache grows, but not by moving the graph's buffer
            assert conv(yb, xb, big_dims) == 0
            torch.cuda.synchronize()
        assert lib.repdl_hip_scratch_bytes() > held
        # trimming frees what no graph holds
        assert lib.repdl_hip_scratch_trim() == 0
        assert 0 < lib.repdl_hip_scratch_bytes() <= held
        y.zero_()
        graph2.replay()
        torch.cuda.synchronize()
        assert torch.equal(_bits(y), _bits(want))
    torch.cuda.current_stream().wait_stream(side)
