"""The fused optimizer steps of the C ABI (repdl_hip_adam_step, repdl_hip_sgd_step) against
the oracle's restatement of RepDL's operation sequence (repdl/optim.py:56-83), bit for bit
over several steps, and the optimizer classes with the fused kernels against the same
classes running the operation sequence itself.  NaN results compare as NaN (the header
leaves their payload open)."""
import ctypes
import math

import numpy as np
import pytest
import torch

import gen
import models
import repdl_amd
from oracle import api as oracle
from repdl_amd import _lib
from test_optim_oracle import CONFIGS, bits, data

pytestmark = pytest.mark.gpu


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return t.data_ptr() if t is not None else None


def hip_adam(tensors, steps, lr, betas, eps, wd):
    """tensors: list of (p, g, m, v, vmax|None) GPU tensors; steps: the step count of each."""
    beta1, beta2 = betas
    descs = []
    for (p, g, m, v, x), t in zip(tensors, steps):
        bc1, bc2 = 1 - beta1 ** t, 1 - beta2 ** t
        descs.append(_lib.AdamTensor(_ptr(p), _ptr(g), _ptr(m), _ptr(v), _ptr(x), p.numel(), math.sqrt(bc2), -(lr / bc1)))
    arr = (_lib.AdamTensor * len(descs))(*descs)
    _lib.call("repdl_hip_adam_step", arr, len(descs), beta1, 1 - beta1, beta2, 1 - beta2, eps, wd, _stream())


def hip_sgd(pairs, lr):
    descs = [_lib.SgdTensor(_ptr(p), _ptr(g), p.numel()) for p, g in pairs]
    arr = (_lib.SgdTensor * len(descs))(*descs)
    _lib.call("repdl_hip_sgd_step", arr, len(descs), lr, _stream())


@pytest.mark.parametrize("kind", ["training", "special", "tiny"])
@pytest.mark.parametrize("cfg", range(len(CONFIGS)))
@pytest.mark.parametrize("n", [1, 3, 2047, 2048, 2049, 8195, (1 << 20) + 5])
def test_adam_steps_equal_oracle(kind, cfg, n):
    c = CONFIGS[cfg]
    p, g0 = data(kind, 1200 + cfg, n)
    grads = [g0] + [data(kind, 1210 + 3 * s + cfg, n)[1] for s in range(3)]
    ams = c["amsgrad"]
    # CPU side
    pc, mc, vc = p.clone(), torch.zeros_like(p), torch.zeros_like(p)
    xc = torch.zeros_like(p) if ams else None
    # GPU side
    pg, mg, vg = p.cuda(), torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    xg = torch.zeros(n, device="cuda") if ams else None
    for step, grad in enumerate(grads, 1):
        oracle.adam_step(pc, grad, mc, vc, xc, step, c["lr"], c["betas"], c["eps"], c["wd"])
        hip_adam([(pg, grad.cuda(), mg, vg, xg)], [step], c["lr"], c["betas"], c["eps"], c["wd"])
        for want, got, name in ((pc, pg, "param"), (mc, mg, "exp_avg"), (vc, vg, "exp_avg_sq"), (xc, xg, "max")):
            if want is not None:
                assert np.array_equal(bits(want), bits(got)), (name, step)


@pytest.mark.parametrize("n", [0, 1, 5, 2048, 4099, (1 << 21) + 3])
def test_sgd_step_equals_oracle(n):
    p, g = data("special" if n % 2 else "training", 1300, n)
    want = p.clone()
    oracle.sgd_step(want, g, 0.01)
    got = p.cuda()
    hip_sgd([(got, g.cuda())], 0.01)
    assert np.array_equal(bits(want), bits(got))


def test_many_tensors_one_call():
    """70 tensors (three launches of at most 32), sizes from empty to several workgroups,
    a step count of its own for each, amsgrad on every other one, some of them slices that
    are not 16-byte aligned."""
    c = CONFIGS[1]
    rng = np.random.default_rng(5)
    sizes = [0, 1, 2, 3, 2047, 2048, 2049, 4096, 10000] + [int(s) for s in rng.integers(1, 30000, size=61)]
    cpu, gpu, steps = [], [], []
    for i, n in enumerate(sizes):
        off = i % 3  # element offset inside a larger buffer: 0 keeps the alignment
        p, g = data("training", 1400 + 2 * i, n + off)
        m, v, x = gen.normal_like(1600 + i, n + off) * 0.01, gen.uniform_pm1(1700 + i, n + off) ** 2, gen.uniform_pm1(1800 + i, n + off) ** 2
        ams = i % 2 == 0
        host = [t.clone()[off:] for t in (p, g, m, v)] + [x.clone()[off:] if ams else None]
        dev = [t.cuda()[off:] for t in (p, g, m, v)] + [x.cuda()[off:] if ams else None]
        cpu.append(host)
        gpu.append(dev)
        steps.append(1 + i % 9)
    for (p, g, m, v, x), t in zip(cpu, steps):
        p_c, m_c, v_c = p.contiguous(), m.contiguous(), v.contiguous()
        x_c = x.contiguous() if x is not None else None
        oracle.adam_step(p_c, g, m_c, v_c, x_c, t, c["lr"], c["betas"], c["eps"], c["wd"])
        p.copy_(p_c), m.copy_(m_c), v.copy_(v_c)
        if x is not None:
            x.copy_(x_c)
    hip_adam(gpu, steps, c["lr"], c["betas"], c["eps"], c["wd"])
    for i, (host, dev) in enumerate(zip(cpu, gpu)):
        for want, got in zip(host, dev):
            if want is not None:
                assert np.array_equal(bits(want), bits(got)), (i, sizes[i])
    # SGD over the same list
    pairs_c = [(h[0].contiguous(), h[1]) for h in cpu]
    for p, g in pairs_c:
        oracle.sgd_step(p, g, 0.05)
    hip_sgd([(d[0], d[1]) for d in gpu], 0.05)
    for i, ((want, _), dev) in enumerate(zip(pairs_c, gpu)):
        assert np.array_equal(bits(want), bits(dev[0])), (i, sizes[i])


def test_bad_arguments_are_refused():
    p = torch.zeros(8, device="cuda")
    bad = (_lib.AdamTensor * 1)(_lib.AdamTensor(_ptr(p), None, _ptr(p), _ptr(p), None, 8, 1.0, -1.0))
    assert _lib.lib().repdl_hip_adam_step(bad, 1, 0.9, 0.1, 0.999, 0.001, 1e-8, 0.0, _stream()) == -1
    neg = (_lib.SgdTensor * 1)(_lib.SgdTensor(_ptr(p), _ptr(p), -1))
    assert _lib.lib().repdl_hip_sgd_step(neg, 1, 0.1, _stream()) == -1
    assert _lib.lib().repdl_hip_sgd_step(None, 0, 0.1, _stream()) == 0
    assert _lib.lib().repdl_hip_sgd_step(None, 1, 0.1, _stream()) == -1


@pytest.mark.parametrize("optim", ["sgd", "adam", "adam_amsgrad_decay"])
def test_optimizer_classes_fused_equals_sequence(optim):
    """Five training steps of the small CNN on the GPU: the classes with the fused kernels
    and the classes running the operation sequence leave the same weights."""
    x, y = models.images(31, 32).cuda(), gen.labels(32, 32, 10).cuda()

    def run(fused):
        repdl_amd.optim.FUSED = fused
        try:
            m = repdl_amd.from_torch_module(models.cnn(0)).cuda()
            if optim == "sgd":
                opt = repdl_amd.optim.SGD(m.parameters(), 0.01)
            elif optim == "adam":
                opt = repdl_amd.optim.Adam(m.parameters(), 0.01)
            else:
                opt = repdl_amd.optim.Adam(m.parameters(), 0.003, betas=(0.8, 0.99), weight_decay=0.05, amsgrad=True)
            models.train_steps(m, repdl_amd.nn.CrossEntropyLoss(), opt, x, y, 5)
            return repdl_amd.utils.get_hash(m), [gen.sha256(s[k]) for s in opt.state.values() for k in sorted(s) if torch.is_tensor(s[k])]
        finally:
            repdl_amd.optim.FUSED = True

    assert run(True) == run(False)


def test_adam_resumes_from_a_state_dict_with_the_same_bits():
    """Four steps in a row == two steps, state_dict() -> load_state_dict() into a fresh optimizer, two
    more, with the fused kernels (load_state_dict leaves the step count as a float32 tensor)."""
    x, y = models.images(41, 16).cuda(), gen.labels(42, 16, 10).cuda()
    make = lambda m: repdl_amd.optim.Adam(m.parameters(), 0.01, weight_decay=0.01, amsgrad=True)
    m1 = repdl_amd.from_torch_module(models.cnn(3)).cuda()
    models.train_steps(m1, repdl_amd.nn.CrossEntropyLoss(), make(m1), x, y, 4)
    m2 = repdl_amd.from_torch_module(models.cnn(3)).cuda()
    o2 = make(m2)
    models.train_steps(m2, repdl_amd.nn.CrossEntropyLoss(), o2, x, y, 2)
    o3 = make(m2)
    o3.load_state_dict(o2.state_dict())
    models.train_steps(m2, repdl_amd.nn.CrossEntropyLoss(), o3, x, y, 2)
    assert repdl_amd.utils.get_hash(m1) == repdl_amd.utils.get_hash(m2)
