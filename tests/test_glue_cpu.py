"""The Python glue (autograd Functions, modules, from_torch_module, optimizers) run
on CPU tensors with the oracle behind repdl_amd.ops (a test-only monkeypatch):
gradients must equal PyTorch autograd exactly on integer-valued data and within
float tolerance on random data; which operator is called in which order follows
the reference (repdl/nn/linear.py:11-38, conv.py:11-50, loss.py:11-34)."""
import numpy as np
import pytest
import torch

import gen
import models
import repdl_amd
from oracle_ops import oracle_for_cpu_tensors


def test_linear_matches_autograd():
    with oracle_for_cpu_tensors():
        lin_t = torch.nn.Linear(7, 5)
        with torch.no_grad():
            lin_t.weight.copy_(gen.small_ints(1, 5, 7))
            lin_t.bias.copy_(gen.small_ints(2, 5))
        lin_r = repdl_amd.from_torch_module(lin_t)
        x1 = gen.small_ints(3, 9, 7).requires_grad_(True)
        x2 = x1.detach().clone().requires_grad_(True)
        go = gen.small_ints(4, 9, 5)
        lin_t(x1).backward(go)
        y = lin_r(x2)
        y.backward(go)
        assert torch.equal(y, lin_t(x1))
        assert torch.equal(x2.grad, x1.grad)
        assert torch.equal(lin_r.weight.grad, lin_t.weight.grad)
        assert torch.equal(lin_r.bias.grad, lin_t.bias.grad)
        with pytest.raises(NotImplementedError):
            lin_r(torch.zeros(2, 3, 7))


@pytest.mark.parametrize("stride,padding", [(1, 1), (2, 0), ((2, 1), (0, 2))])
def test_conv2d_matches_autograd(stride, padding):
    with oracle_for_cpu_tensors():
        c_t = torch.nn.Conv2d(3, 4, 3, stride=stride, padding=padding)
        with torch.no_grad():
            c_t.weight.copy_(gen.small_ints(11, 4, 3, 3, 3, lo=-3, hi=3))
            c_t.bias.copy_(gen.small_ints(12, 4))
        c_r = repdl_amd.from_torch_module(c_t)
        x1 = gen.small_ints(13, 2, 3, 9, 8, lo=-3, hi=3).requires_grad_(True)
        x2 = x1.detach().clone().requires_grad_(True)
        y_t = c_t(x1)
        go = gen.small_ints(14, *y_t.shape, lo=-3, hi=3)
        y_t.backward(go)
        y_r = c_r(x2)
        y_r.backward(go)
        assert torch.equal(y_r, y_t)
        assert torch.equal(x2.grad, x1.grad)
        assert torch.equal(c_r.weight.grad, c_t.weight.grad)
        assert torch.equal(c_r.bias.grad, c_t.bias.grad)


def test_conv2d_rejections():
    with oracle_for_cpu_tensors():
        F = repdl_amd.nn.functional
        x, w = torch.zeros(1, 2, 5, 5), torch.zeros(2, 2, 3, 3)
        with pytest.raises(NotImplementedError):
            F.conv2d(x, w, padding="same")
        with pytest.raises(NotImplementedError):
            F.conv2d(x, w, dilation=2)
        y = F.conv2d(x.requires_grad_(True), torch.zeros(2, 1, 3, 3).requires_grad_(True), groups=2)
        with pytest.raises(NotImplementedError):
            y.sum().backward()


def test_cross_entropy_matches_torch():
    with oracle_for_cpu_tensors():
        x1 = (gen.normal_like(21, 12, 10) * 3).requires_grad_(True)
        x2 = x1.detach().clone().requires_grad_(True)
        t = gen.labels(22, 12, 10)
        l_t = torch.nn.functional.cross_entropy(x1, t)
        l_r = repdl_amd.nn.functional.cross_entropy(x2, t)
        assert l_r.shape == l_t.shape and abs(float(l_r) - float(l_t)) < 1e-6
        (l_t * 3).backward()
        (l_r * 3).backward()
        assert torch.allclose(x2.grad, x1.grad, atol=1e-6)
        loss = repdl_amd.from_torch_module(torch.nn.CrossEntropyLoss())
        assert float(loss(x2.detach(), t)) == float(l_r)
        with pytest.raises(NotImplementedError):
            repdl_amd.nn.functional.cross_entropy(x2, t, reduction="sum")


def test_batchnorm_close_to_torch(monkeypatch):
    with oracle_for_cpu_tensors():
        for bn_t, x in ((torch.nn.BatchNorm2d(5), gen.normal_like(31, 4, 5, 6, 7)),
                        (torch.nn.BatchNorm1d(6), gen.normal_like(32, 9, 6))):
            with torch.no_grad():
                bn_t.weight.copy_(gen.normal_like(33, bn_t.num_features))
                bn_t.bias.copy_(gen.normal_like(34, bn_t.num_features))
            bn_r = repdl_amd.from_torch_module(bn_t)
            x1, x2 = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
            # as the reference (batchnorm.py:92-93): the updates are evaluated and dropped
            before = bn_r.running_mean.clone(), bn_r.running_var.clone()
            bn_r(x.clone())
            assert torch.equal(bn_r.running_mean, before[0]) and torch.equal(bn_r.running_var, before[1])
            monkeypatch.setattr(repdl_amd.nn.functional, "STORE_RUNNING_STATS", True)
            y_t, y_r = bn_t(x1), bn_r(x2)
            monkeypatch.setattr(repdl_amd.nn.functional, "STORE_RUNNING_STATS", False)
            assert torch.allclose(y_r, y_t, atol=2e-5)
            go = gen.normal_like(35, *x.shape)
            y_t.backward(go)
            y_r.backward(go)
            assert torch.allclose(x2.grad, x1.grad, atol=2e-4)
            assert torch.allclose(bn_r.weight.grad, bn_t.weight.grad, atol=2e-4)
            assert torch.allclose(bn_r.bias.grad, bn_t.bias.grad, atol=2e-4)
            # running mean follows PyTorch; the running variance uses the biased batch
            # variance, as the reference's expression does (batchnorm.py:93)
            assert torch.allclose(bn_r.running_mean, bn_t.running_mean, atol=1e-6)
            bn_r.eval()
            assert torch.isfinite(bn_r(x)).all()


def test_func_means():
    with oracle_for_cpu_tensors():
        f = repdl_amd.func
        v = gen.normal_like(41, 37).requires_grad_(True)
        m = f.mean1d(v)
        assert float(m) == float(repdl_amd.ops.sum1d(v.detach(), True))
        m.backward()
        assert torch.equal(v.grad, torch.full((37,), 1 / 37))
        a = gen.normal_like(42, 6, 4).requires_grad_(True)
        f.mean2d_dim0(a).sum().backward()
        assert torch.equal(a.grad, torch.full((6, 4), 1 / 6))
        b = gen.normal_like(43, 2, 3, 4, 5).requires_grad_(True)
        f.mean4d_dim023(b).sum().backward()
        assert torch.equal(b.grad, torch.full((2, 3, 4, 5), 1 / 40))
        with pytest.raises(NotImplementedError):
            f.expand_as(torch.zeros(3), torch.zeros(2, 4))


def test_cnn_training_step_tracks_torch():
    """End to end through from_torch_module: losses stay close to PyTorch's own
    (not bit-equal: PyTorch sums in another order), and the run is deterministic."""
    x, y = models.images(51, 16), gen.labels(52, 16, 10)
    with oracle_for_cpu_tensors():
        outs = []
        for _ in range(2):
            m = repdl_amd.from_torch_module(models.cnn(0))
            logits, losses = models.train_steps(m, repdl_amd.nn.CrossEntropyLoss(), repdl_amd.optim.SGD(m.parameters(), 0.01), x, y, 3)
            outs.append((repdl_amd.utils.get_hash(m), repdl_amd.utils.get_hash(logits), losses))
        assert outs[0][:2] == outs[1][:2]
    mt = models.cnn(0)
    _, losses_t = models.train_steps(mt, torch.nn.CrossEntropyLoss(), torch.optim.SGD(mt.parameters(), 0.01), x, y, 3)
    for a, b in zip(outs[0][2], losses_t):
        assert abs(float(a) - float(b)) < 1e-4


def test_adam_matches_formula():
    with oracle_for_cpu_tensors():
        p = torch.nn.Parameter(gen.normal_like(61, 50))
        g = gen.normal_like(62, 50)
        opt = repdl_amd.optim.Adam([p], lr=0.01)
        p0 = p.detach().clone()
        p.grad = g.clone()
        opt.step()
        m = g * np.float32(1 - 0.9)
        v = (g * g) * np.float32(1 - 0.999)
        denom = repdl_amd.ops.div(repdl_amd.ops.sqrt(v), (1 - 0.999) ** 0.5) + 1e-8
        want = p0 + repdl_amd.ops.div(m, denom) * (-(0.01 / (1 - 0.9)))
        assert torch.equal(p.detach(), want)
        pt = torch.nn.Parameter(p0.clone())
        pt.grad = g.clone()
        torch.optim.Adam([pt], lr=0.01).step()
        assert torch.allclose(p.detach(), pt.detach(), atol=1e-6)


@pytest.mark.parametrize("amsgrad", [False, True])
def test_adam_resumes_from_a_state_dict_with_the_same_bits(amsgrad):
    """Four steps in a row == two steps, state_dict() -> load_state_dict() into a fresh optimizer,
    two more.  (load_state_dict turns the step count into a float32 tensor; the bias corrections
    must still be the binary64 values of an integer count.)"""
    x, y = models.images(71, 16), gen.labels(72, 16, 10)
    make = lambda m: repdl_amd.optim.Adam(m.parameters(), 0.01, weight_decay=0.01, amsgrad=amsgrad)
    with oracle_for_cpu_tensors():
        m1 = repdl_amd.from_torch_module(models.cnn(3))
        models.train_steps(m1, repdl_amd.nn.CrossEntropyLoss(), make(m1), x, y, 4)
        m2 = repdl_amd.from_torch_module(models.cnn(3))
        o2 = make(m2)
        models.train_steps(m2, repdl_amd.nn.CrossEntropyLoss(), o2, x, y, 2)
        o3 = make(m2)
        o3.load_state_dict(o2.state_dict())
        models.train_steps(m2, repdl_amd.nn.CrossEntropyLoss(), o3, x, y, 2)
    assert repdl_amd.utils.get_hash(m1) == repdl_amd.utils.get_hash(m2)


def test_readme_initial_model_hash():
    """The one known answer the reference holds for the glue: README.md:36, the SHA-256 of the
    LeNet-5 of examples/mnist_trainig.py:12-33 built under torch.manual_seed(0) (:106-108),
    converted by from_torch_module and hashed by utils.get_hash (parameters in order)."""

    class TorchModel(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.net = torch.nn.Sequential(
                torch.nn.Conv2d(1, 6, kernel_size=5, padding=2), torch.nn.ReLU(), torch.nn.MaxPool2d(kernel_size=2, stride=2),
                torch.nn.Conv2d(6, 16, kernel_size=5), torch.nn.ReLU(), torch.nn.MaxPool2d(kernel_size=2, stride=2),
                torch.nn.Flatten(), torch.nn.Linear(16 * 5 * 5, 120), torch.nn.ReLU(), torch.nn.Linear(120, 84),
                torch.nn.ReLU(), torch.nn.Linear(84, 10))

        def forward(self, x):
            return self.net(x)

    torch.manual_seed(0)
    model = repdl_amd.from_torch_module(TorchModel())
    assert repdl_amd.utils.get_hash(model) == "2a2d133895b1684e55d0f152ead2914b55adc551d9790a4b4585309b79c60362"
    kinds = [type(m).__name__ for m in model.net]
    assert kinds.count("Conv2d") == 2 and kinds.count("Linear") == 3
    assert all(type(m).__module__.startswith("repdl_amd") for m in model.net if type(m).__name__ in ("Conv2d", "Linear"))


def test_reference_names_resolve():
    """Every public name of the reference's Python packages resolves under the same path here
    (repdl/__init__.py:8-15, func.py, ops.py, optim.py, utils.py, nn/__init__.py:4-8, nn/functional.py:4-7,
    nn/linear.py, nn/conv.py, nn/loss.py, nn/batchnorm.py)."""
    import importlib

    names = {
        "repdl_amd": ["func", "nn", "ops", "optim", "utils", "from_torch_module"],
        "repdl_amd.ops": ["conv2d", "conv2d_grad_input", "conv2d_grad_kernel", "cross_entropy", "div", "mm", "softmax", "sqrt",
                          "sum1d", "sum2d_dim0", "sum2d_dim1", "sum4d_dim023"],
        "repdl_amd.func": ["ExpandFunction", "expand_as", "Mean1dFunction", "mean1d", "Mean2dDim0Function", "mean2d_dim0",
                           "Mean4dDim023Function", "mean4d_dim023"],
        "repdl_amd.optim": ["Adam"],
        "repdl_amd.utils": ["get_hash", "print_hash"],
        "repdl_amd.nn": ["functional", "BatchNorm1d", "BatchNorm2d", "Conv2d", "Linear", "CrossEntropyLoss"],
        "repdl_amd.nn.functional": ["batch_norm", "conv2d", "linear", "cross_entropy"],
        "repdl_amd.nn.linear": ["LinearFunction", "linear", "Linear"],
        "repdl_amd.nn.conv": ["Conv2dFunction", "conv2d", "Conv2d"],
        "repdl_amd.nn.loss": ["CrossEntropyFunction", "cross_entropy", "CrossEntropyLoss"],
        "repdl_amd.nn.batchnorm": ["BatchNormFunction", "batch_norm", "BatchNorm1d", "BatchNorm2d"],
    }
    for mod, attrs in names.items():
        m = importlib.import_module(mod)
        for a in attrs:
            assert hasattr(m, a), (mod, a)
    from repdl_amd.nn.linear import LinearFunction

    assert issubclass(LinearFunction, torch.autograd.Function)
    assert issubclass(repdl_amd.func.Mean1dFunction, torch.autograd.Function)
