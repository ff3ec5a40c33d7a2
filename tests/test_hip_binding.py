"""The two bindings of the C-ABI library -- the compiled PyTorch extension built from
csrc/bind.cpp and the ctypes module -- must give the same tensors: same bits, same
shapes (0-dim sums and losses, squeezed or kept dimensions), same errors for bad input."""
import pytest
import torch

import cases
import gen

pytestmark = pytest.mark.gpu


def test_compiled_binding_is_the_one_in_use():
    from repdl_amd.backend import hip

    assert hip.BINDING == "ext"


@pytest.mark.parametrize("case", cases.CASES, ids=[c["name"] for c in cases.CASES])
def test_bindings_agree_with_the_reference_digest(case, golden):
    from hipbackend import ctypes_backend, ext_backend

    g = golden[case["name"]]
    if "error" in g:
        pytest.skip("the reference rejects this input (%s)" % g["error"])
    a, b = cases.run(case, ext_backend), cases.run(case, ctypes_backend)
    assert a.shape == b.shape and list(a.shape) == g["shape"]
    assert gen.sha256(a) == g["sha256"] and gen.sha256(b) == g["sha256"]


def test_shapes_and_elementwise():
    from repdl_amd.backend import _hip_ext as ext
    from repdl_amd.backend import hip_ctypes as ct

    x = gen.elementwise_mix(3, 5000).cuda()
    y = gen.elementwise_mix(4, 5000).cuda()
    m = gen.normal_like(5, 33, 47).cuda()
    t4 = gen.normal_like(6, 3, 5, 7, 9).cuda()
    for name, args in [("exp", (x,)), ("log", (x,)), ("sqrt", (x,)), ("div", (x, y)), ("div_scalar", (x, 10.0)),
                       ("div", (m, m[:1])), ("div", (m, torch.tensor(3.0, device="cuda"))),
                       ("sum1d", (x[:777], True)), ("sum2d_dim0", (m, False, True)), ("sum2d_dim0", (m, True, False)),
                       ("sum2d_dim1", (m, False, False)), ("sum2d_dim1", (m[:1], False, False)),
                       ("sum4d_dim023", (t4, True, True)), ("sum4d_dim023", (t4, False, False)), ("softmax", (m,)),
                       ("cross_entropy", (m, gen.labels(7, 33, 47).cuda())),
                       ("mm_bias", (m, gen.normal_like(8, 21, 47).cuda(), gen.normal_like(9, 21).cuda(), False, True)),
                       ("mm_bias", (m, gen.normal_like(8, 21, 47).cuda(), None, False, True)),
                       ("conv2d_bias", (t4, gen.normal_like(10, 4, 5, 3, 3).cuda(), gen.normal_like(11, 4).cuda(), 1, 2, 1, 0, 1)),
                       ("conv2d_bias", (t4, gen.normal_like(10, 4, 5, 3, 3).cuda(), None, 1, 2, 1, 0, 1))]:
        a, b = getattr(ext, name)(*args), getattr(ct, name)(*args)
        assert a.shape == b.shape, name
        assert torch.equal(a.view(torch.int32), b.view(torch.int32)), name


def test_errors():
    from repdl_amd.backend import _hip_ext as ext

    x = torch.ones(4, 4)
    with pytest.raises(RuntimeError):
        ext.mm(x, x, False, False)  # not on the GPU
    with pytest.raises(RuntimeError):
        ext.mm(x.cuda().double(), x.cuda().double(), False, False)
    with pytest.raises(RuntimeError):
        ext.mm(x.cuda(), torch.ones(5, 4).cuda(), False, False)  # inner dimensions differ
    with pytest.raises(RuntimeError):
        ext.conv2d(torch.ones(1, 3, 8, 8).cuda(), torch.ones(4, 2, 3, 3).cuda(), 1, 1, 1, 1, 2)
    from repdl_amd.backend import hip_ctypes as ct

    for mod in (ext, ct):
        with pytest.raises(RuntimeError):
            mod.mm_bias(x.cuda(), x.cuda(), torch.ones(5).cuda(), False, False)  # bias length
        with pytest.raises(RuntimeError):
            mod.conv2d_bias(torch.ones(1, 3, 8, 8).cuda(), torch.ones(4, 3, 3, 3).cuda(), torch.ones(4), 1, 1, 1, 1, 1)  # bias on the CPU
