"""Operators that need a workspace, run on two streams at once and with sizes that grow and shrink
from call to call, give the results they give one by one on one stream: through the bindings
(scratch from PyTorch's allocator, which hands memory on within a stream only) and through the
plain C entry points (the library's scratch cache, csrc/workspace.hip: a buffer is reused on its
own stream only, and a call that nests another -- the gathered route of a strided 1x1
grad-kernel -- gets two buffers)."""
import ctypes

import pytest
import torch

import gen

pytestmark = pytest.mark.gpu


class _PlainOps:
    """The operators of _jobs through the plain C entry points: scratch from the library's cache."""

    @staticmethod
    def _run(name, out, *args):
        from repdl_amd import _lib

        _lib.call(name, *args, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        return out

    def sum4d_dim023(self, t):
        out = torch.empty(t.shape[1], device=t.device)
        return self._run("repdl_hip_sum4d_dim023", out, ctypes.c_void_p(t.data_ptr()), ctypes.c_void_p(out.data_ptr()), *t.shape, 0)

    def sum1d(self, t):
        out = torch.empty((), device=t.device)
        return self._run("repdl_hip_sum1d", out, ctypes.c_void_p(t.data_ptr()), ctypes.c_void_p(out.data_ptr()), t.numel(), 0)

    def conv2d_grad_kernel(self, x, kshape, go, stride, padding):
        out = torch.empty(kshape, device=x.device)
        N, IC, H, W = x.shape
        return self._run("repdl_hip_conv2d_grad_kernel", out, ctypes.c_void_p(go.data_ptr()), ctypes.c_void_p(x.data_ptr()),
                         ctypes.c_void_p(out.data_ptr()), N, IC, H, W, go.shape[1], go.shape[2], go.shape[3], kshape[2], kshape[3],
                         *stride, *padding)


def _jobs(dev, ops=None):
    if ops is None:
        from repdl_amd import ops

    chans = [gen.normal_like(31 + i, 16, c, 56, 56).to(dev) for i, c in enumerate((8, 24, 4, 16))]  # 50176-element chains: the parallel evaluation
    flat = [gen.uniform_pm1(41 + i, n).to(dev) for i, n in enumerate((300_000, 70_000, 1_200_000))]
    x = torch.relu(gen.normal_like(51, 4, 24, 17, 23)).to(dev)
    go = gen.normal_like(52, 4, 40, 6, 12).to(dev)  # 1x1 at stride (3, 2): gathered input, then the chain kernel with padded rows
    xs = torch.relu(gen.normal_like(53, 8, 64, 7, 7)).to(dev)
    gos = gen.normal_like(54, 8, 512, 7, 7).to(dev)  # many short chains: transposed grad_output and im2col
    jobs = [lambda t=t: ops.sum4d_dim023(t) for t in chans]
    jobs += [lambda t=t: ops.sum1d(t) for t in flat]
    jobs.append(lambda: ops.conv2d_grad_kernel(x, (40, 24, 1, 1), go, (3, 2), (0, 0)))
    jobs.append(lambda: ops.conv2d_grad_kernel(xs, (512, 64, 3, 3), gos, (1, 1), (1, 1)))
    return jobs


@pytest.mark.parametrize("source", ["bindings", "cache"])
def test_two_streams_and_changing_sizes(source):
    dev = torch.device("cuda:0")
    jobs = _jobs(dev, _PlainOps() if source == "cache" else None)
    want = [j().clone() for j in jobs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev)]
    for st in streams:
        st.wait_stream(torch.cuda.current_stream(dev))
    got = [[], []]
    for rep in range(3):
        for k, st in enumerate(streams):
            order = range(len(jobs)) if (rep + k) % 2 == 0 else reversed(range(len(jobs)))  # sizes up on one stream, down on the other
            with torch.cuda.stream(st):
                for i in order:
                    got[k].append((i, jobs[i]()))
    torch.cuda.synchronize()
    for k in range(2):
        for i, r in got[k]:
            assert torch.equal(r.view(torch.int32), want[i].view(torch.int32)), (k, i)
