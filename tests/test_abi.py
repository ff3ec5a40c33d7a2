"""Host-side checks that need no GPU: the C-ABI library loads, exports every
symbol that include/repdl_hip.h declares, rejects bad arguments before touching
the device, and the Python operator layer refuses CPU tensors (no fallback)."""
import os
import re

import pytest
import torch

import repdl_amd
from repdl_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "repdl_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(repdl_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.lib()
    names = declared_symbols()
    assert len(names) >= 17
    for n in names:
        assert hasattr(lib, n), n
    other = {"repdl_hip_error_string", "repdl_hip_abi_version", "repdl_hip_matrix_path", "repdl_hip_init",
             "repdl_hip_sum1d_static_max_n", "repdl_hip_routes_taken", "repdl_hip_route_name"}
    assert set(_lib.SIGNATURES) | set(_lib.SIZE_QUERIES) | other == set(names)


def test_abi_version_and_error_strings():
    lib = _lib.lib()
    assert lib.repdl_hip_abi_version() == 1
    assert lib.repdl_hip_error_string(0) == b"success"
    assert b"invalid argument" in lib.repdl_hip_error_string(-1)
    assert b"workspace" in lib.repdl_hip_error_string(-3)
    assert b"capacity" in lib.repdl_hip_error_string(-4)


def test_bad_arguments_are_rejected_on_the_host():
    lib = _lib.lib()
    assert lib.repdl_hip_mm(None, None, None, 4, 4, 4, 0, 0, None) == -1
    assert lib.repdl_hip_mm(None, None, None, -1, 4, 4, 0, 0, None) == -1
    assert lib.repdl_hip_sum1d(None, None, 8, 0, None) == -1
    assert lib.repdl_hip_exp(None, None, 8, None) == -1
    assert lib.repdl_hip_exp(None, None, -8, None) == -1
    assert lib.repdl_hip_div(None, None, None, 8, None) == -1
    # groups must divide the channel counts; stride must be positive
    assert lib.repdl_hip_conv2d(None, None, None, 1, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1, 2, None) == -1
    assert lib.repdl_hip_conv2d(None, None, None, 1, 4, 8, 8, 4, 3, 3, 0, 1, 1, 1, 1, None) == -1
    # empty problems succeed without any pointer
    assert lib.repdl_hip_mm(None, None, None, 0, 4, 4, 0, 0, None) == 0
    assert lib.repdl_hip_exp(None, None, 0, None) == 0
    with pytest.raises(_lib.RepdlHipError):
        _lib.check(-1, "x")


def test_cpu_tensors_are_refused():
    x = torch.ones(4, 4)
    for call in (
        lambda: repdl_amd.ops.mm(x, x),
        lambda: repdl_amd.ops.sqrt(x),
        lambda: repdl_amd.ops.div(x, 10.0),
        lambda: repdl_amd.ops.sum2d_dim1(x),
        lambda: repdl_amd.ops.exp(x),
    ):
        with pytest.raises(RuntimeError):
            call()


def test_from_torch_module_type_mapping():
    m = torch.nn.Sequential(
        torch.nn.Conv2d(1, 2, 3, padding=1, bias=False), torch.nn.BatchNorm2d(2), torch.nn.ReLU(),
        torch.nn.Flatten(), torch.nn.Linear(8, 3), torch.nn.BatchNorm1d(3))

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.body = m
            self.loss = torch.nn.CrossEntropyLoss()

    r = repdl_amd.from_torch_module(Net())
    assert type(r.body[0]) is repdl_amd.nn.Conv2d and r.body[0].bias is None
    assert type(r.body[1]) is repdl_amd.nn.BatchNorm2d
    assert type(r.body[2]) is torch.nn.ReLU
    assert type(r.body[4]) is repdl_amd.nn.Linear
    assert type(r.body[5]) is repdl_amd.nn.BatchNorm1d
    assert type(r.loss) is repdl_amd.nn.CrossEntropyLoss
    assert torch.equal(r.body[4].weight, m[4].weight) and r.body[4].weight is not m[4].weight
    assert repdl_amd.utils.get_hash(r.body) == repdl_amd.utils.get_hash(m)
    with pytest.raises(TypeError):
        repdl_amd.from_torch_module(3)


def test_get_hash_convention():
    import hashlib

    t = torch.arange(12, dtype=torch.float32).reshape(3, 4)
    assert repdl_amd.utils.get_hash(t) == hashlib.sha256(t.numpy().tobytes()).hexdigest()
    lin = torch.nn.Linear(3, 2)
    h = hashlib.sha256()
    h.update(lin.weight.detach().numpy().tobytes())
    h.update(lin.bias.detach().numpy().tobytes())
    assert repdl_amd.utils.get_hash(lin) == h.hexdigest()


def test_compiled_binding_loads_when_built():
    """If csrc/bind.cpp has been built, repdl_amd.backend.hip must serve it (an extension that
    is there but does not import would otherwise go unnoticed behind the ctypes binding)."""
    from repdl_amd import build
    from repdl_amd.backend import hip

    if os.path.exists(build.ext_path()):
        assert hip.BINDING == "ext"
        for fn in hip.FUNCTIONS:
            assert callable(getattr(hip, fn))
    else:
        assert hip.BINDING == "ctypes"


def test_header_is_plain_c_and_struct_layouts_match(tmp_path):
    """include/repdl_hip.h compiles as C99 on its own, and the ctypes mirrors of its descriptor
    structs have the C compiler's sizes and field offsets."""
    import ctypes
    import subprocess

    src = tmp_path / "layout.c"
    src.write_text(
        '#include <stddef.h>\n#include <stdio.h>\n#include "repdl_hip.h"\n'
        "int main(void) {\n"
        '  printf("%zu %zu %zu %zu %zu\\n", sizeof(repdl_adam_tensor), offsetof(repdl_adam_tensor, max_exp_avg_sq),\n'
        "         offsetof(repdl_adam_tensor, n), offsetof(repdl_adam_tensor, sqrt_bias_correction2),\n"
        "         offsetof(repdl_adam_tensor, step_scale));\n"
        '  printf("%zu %zu %zu\\n", sizeof(repdl_sgd_tensor), offsetof(repdl_sgd_tensor, grad), offsetof(repdl_sgd_tensor, n));\n'
        "  return 0;\n}\n")
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
                    str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, stdout=subprocess.PIPE, text=True).stdout.split("\n")
    a, s = _lib.AdamTensor, _lib.SgdTensor
    assert [int(v) for v in out[0].split()] == [ctypes.sizeof(a), a.max_exp_avg_sq.offset, a.n.offset,
                                                 a.sqrt_bias_correction2.offset, a.step_scale.offset]
    assert [int(v) for v in out[1].split()] == [ctypes.sizeof(s), s.grad.offset, s.n.offset]
