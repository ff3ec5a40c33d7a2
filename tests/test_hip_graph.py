"""The operators that allocate nothing can be captured into a HIP graph and replayed:
a Linear forward (mm with the bias in its epilogue), exp, a division, row sums and the
sum1d entry point with the fixed scratch array, replayed several times with new inputs and
eager work in between, every replay held against the eager result on the same bytes."""
import ctypes

import pytest
import torch

import gen

pytestmark = pytest.mark.gpu


def test_graph_replays_match_eager():
    from repdl_amd import ops

    dev = torch.device("cuda:0")
    M, N, K = 256, 384, 512
    x = gen.normal_like(1, M, K).to(dev)
    w = gen.normal_like(2, N, K).to(dev)
    bias = gen.normal_like(3, N).to(dev)

    from repdl_amd import _lib

    flat = gen.uniform_pm1(4, 600_000).to(dev)  # long enough for the parallel evaluation and its scratch

    def step():
        y = ops.mm_bias(x, w, bias, False, True)
        e = ops.exp(ops.div(y, 64.0))
        total = torch.empty(1, device=dev)
        _lib.call("repdl_hip_sum1d_static", ctypes.c_void_p(flat.data_ptr()), ctypes.c_void_p(total.data_ptr()), flat.numel(), 0,
                  ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        return y, e, ops.sum2d_dim1(e), total

    # the library's one-time device check and torch's lazy initialisations happen outside the capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for rep in range(4):
        x.copy_(gen.normal_like(10 + rep, M, K).to(dev))
        flat.copy_(gen.uniform_pm1(20 + rep, 600_000).to(dev))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = step()  # eager work between the replays
        torch.cuda.synchronize()
        for g, wnt in zip(got, want):
            assert torch.equal(g.view(torch.int32), wnt.view(torch.int32)), rep
