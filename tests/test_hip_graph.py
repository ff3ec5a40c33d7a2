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


_FRESH_CAPTURE = r"""
import sys, torch
sys.path.insert(0, {root!r}); sys.path.insert(0, {root!r} + "/tests")
import gen
import repdl_amd
from repdl_amd import ops
from repdl_amd.backend import hip

dev = torch.device("cuda:0")
repdl_amd.init()                        # the device check cannot run under capture; nothing else has run
N, IC, H, W, OC = 8, 64, 28, 28, 128
x = torch.relu(gen.normal_like(1, N, IC, H, W)).to(dev)
w3 = gen.normal_like(2, OC, IC, 3, 3).to(dev)       # 3x3 at stride 2: a padded copy, residues, padded rows in scratch
go3 = gen.normal_like(3, N, OC, 14, 14).to(dev)
w1 = gen.normal_like(4, IC, IC, 3, 3).to(dev)       # 3x3 at stride 1: guard words, the transposed kernel
go1 = gen.normal_like(5, N, IC, H, W).to(dev)
bias = gen.normal_like(6, OC).to(dev)

def step():
    return (ops.conv2d_bias(x, w3, bias, (2, 2), (1, 1), 1),
            ops.conv2d_grad_input((N, IC, H, W), w3, go3, (2, 2), (1, 1)),
            ops.conv2d_grad_kernel(x, (OC, IC, 3, 3), go3, (2, 2), (1, 1)),
            ops.conv2d(x, w1, (1, 1), (1, 1), 1),
            ops.conv2d_grad_input((N, IC, H, W), w1, go1, (1, 1), (1, 1)),
            ops.conv2d_grad_kernel(x, (IC, IC, 3, 3), go1, (1, 1), (1, 1)),
            ops.sum4d_dim023(go1.expand(N, IC, H, W).repeat(8, 1, 2, 1)))   # chains of 100352: the parallel evaluation

graph = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph):           # the first call of every operator in this process
    captured = step()
for rep in range(3):
    x.copy_(torch.relu(gen.normal_like(10 + rep, N, IC, H, W)).to(dev))
    go1.copy_(gen.normal_like(20 + rep, N, IC, H, W).to(dev))
    graph.replay()
    torch.cuda.synchronize()
    got = [t.clone() for t in captured]
    want = step()                       # eager work between the replays
    torch.cuda.synchronize()
    for i, (g, wnt) in enumerate(zip(got, want)):
        assert torch.equal(g.view(torch.int32), wnt.view(torch.int32)), (rep, i)
from repdl_amd import _lib
assert _lib.lib().repdl_hip_scratch_bytes() == 0    # the bindings bring their own scratch: the cache was never used
print("fresh-capture ok", hip.BINDING)
"""


def test_convolutions_captured_in_a_fresh_process():
    """Forward, grad-input and grad-kernel of two layers and a channel sum, captured into a graph as the first
    calls of a new process -- no warm-up, so nothing the operators need may be allocated, freed or kept by the
    library: their scratch comes from PyTorch's allocator through the *_ws entry points -- and replayed to the
    eager bits."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-c", _FRESH_CAPTURE.format(root=root)], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "fresh-capture ok" in proc.stdout


def test_training_step_captured():
    """A whole training step of the 2-conv + 2-FC CNN -- forward, loss, backward with its side streams, the fused
    SGD update -- captured into one graph (the operators bring their scratch from PyTorch's allocator, so nothing in
    it allocates behind PyTorch's back) and replayed: three eager steps, the capture, three replays give the weights
    of six eager steps, bit for bit."""
    import models
    import repdl_amd

    dev = torch.device("cuda:0")
    repdl_amd.init()
    x, y = models.images(21, 64).to(dev), gen.labels(22, 64, 10).to(dev)
    lossf = repdl_amd.nn.CrossEntropyLoss()

    def make():
        m = repdl_amd.from_torch_module(models.cnn(0)).to(dev)
        return m, repdl_amd.optim.SGD(m.parameters(), 0.01)

    def step(m, opt):
        opt.zero_grad(set_to_none=True)
        lossf(m(x), y).backward()
        opt.step()

    m, opt = make()
    for _ in range(6):
        step(m, opt)
    want = repdl_amd.utils.get_hash(m)

    m2, opt2 = make()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step(m2, opt2)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    opt2.zero_grad(set_to_none=True)
    with torch.cuda.graph(graph):
        lossf(m2(x), y).backward()
        opt2.step()
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    assert repdl_amd.utils.get_hash(m2) == want
