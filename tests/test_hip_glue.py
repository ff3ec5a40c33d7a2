"""GPU parity through the Python glue: the same repdl_amd modules run once on CPU
tensors (oracle behind repdl_amd.ops, a test-only monkeypatch) and once on GPU
tensors (HIP backend); outputs, gradients and trained weights must hash equal."""
import pytest
import torch

import gen
import models
import repdl_amd
from oracle_ops import oracle_for_cpu_tensors

pytestmark = pytest.mark.gpu


def _both(build, run):
    """run(module, device) on cpu (oracle) and cuda (hip); returns the two results."""
    with oracle_for_cpu_tensors():
        res = []
        for dev in ("cpu", "cuda"):
            m = build().to(dev)
            res.append(run(m, dev))
    return res


def test_linear_forward_backward_bits():
    def build():
        torch.manual_seed(3)
        return repdl_amd.from_torch_module(torch.nn.Linear(300, 130))

    def run(m, dev):
        x = gen.normal_like(1, 77, 300).to(dev).requires_grad_(True)
        y = m(x)
        y.backward(gen.normal_like(2, 77, 130).to(dev))
        return [gen.sha256(t) for t in (y, x.grad, m.weight.grad, m.bias.grad)]

    a, b = _both(build, run)
    assert a == b


@pytest.mark.parametrize("cfg", [(3, 8, 3, 1, 1), (8, 16, 3, 2, 1), (16, 8, 1, 1, 0), (4, 6, 5, 1, 2)])
def test_conv2d_forward_backward_bits(cfg):
    ic, oc, k, s, p = cfg

    def build():
        torch.manual_seed(4)
        return repdl_amd.from_torch_module(torch.nn.Conv2d(ic, oc, k, stride=s, padding=p))

    def run(m, dev):
        x = gen.relu_like(5, 6, ic, 20, 17).to(dev).requires_grad_(True)
        y = m(x)
        y.backward(gen.normal_like(6, *y.shape).to(dev))
        return [gen.sha256(t) for t in (y, x.grad, m.weight.grad, m.bias.grad)]

    a, b = _both(build, run)
    assert a == b


def test_cross_entropy_and_softmax_bits():
    def build():
        return repdl_amd.nn.CrossEntropyLoss()

    def run(m, dev):
        x = (gen.normal_like(7, 64, 10) * 4).to(dev).requires_grad_(True)
        t = gen.labels(8, 64, 10).to(dev)
        loss = m(x, t)
        loss.backward()
        return [gen.sha256(loss), gen.sha256(x.grad)]

    a, b = _both(build, run)
    assert a == b


def test_batchnorm_bits():
    def build():
        torch.manual_seed(9)
        return repdl_amd.from_torch_module(torch.nn.Sequential(torch.nn.Conv2d(3, 8, 3, padding=1), torch.nn.BatchNorm2d(8)))

    def run(m, dev):
        x = gen.normal_like(10, 4, 3, 12, 12).to(dev).requires_grad_(True)
        y = m(x)
        y.backward(gen.normal_like(11, *y.shape).to(dev))
        return [gen.sha256(t) for t in (y, x.grad, m[1].weight.grad, m[1].bias.grad, m[0].weight.grad)]

    a, b = _both(build, run)
    assert a == b


@pytest.mark.parametrize("optim", ["sgd", "adam"])
def test_cnn_training_bits(optim):
    """BASELINE config 5, end to end: 2-conv + 2-FC CNN from from_torch_module, batch
    64 of synthetic 1x28x28 images, 10 random classes, SGD lr 0.01 (explicit
    two-rounding update) -- hashes of the final weights and logits, CPU vs GPU."""
    x, y = models.images(21, 64), gen.labels(22, 64, 10)

    def build():
        return repdl_amd.from_torch_module(models.cnn(0))

    def run(m, dev):
        opt = repdl_amd.optim.SGD(m.parameters(), 0.01) if optim == "sgd" else repdl_amd.optim.Adam(m.parameters(), 0.01)
        logits, losses = models.train_steps(m, repdl_amd.nn.CrossEntropyLoss(), opt, x.to(dev), y.to(dev), 3)
        return [repdl_amd.utils.get_hash(m), repdl_amd.utils.get_hash(logits)] + [gen.sha256(l) for l in losses]

    a, b = _both(build, run)
    print(optim, "weights", b[0], "logits", b[1], flush=True)
    assert a == b


def test_backward_streams_repeated():
    """The backward passes of conv2d and batch_norm run their independent gradients on side
    streams.  Many passes in a row with fresh tensors each time (so that the allocator reuses
    blocks across the streams) must give, every time, the bits of the operators called one
    after the other on the current stream."""
    from repdl_amd import ops
    from repdl_amd.nn import functional as F

    for it in range(12):
        N, IC, H, W, OC = 8, 16 + 8 * (it % 3), 20, 20, 32
        x = gen.relu_like(300 + it, N, IC, H, W).cuda().requires_grad_(True)
        w = (gen.normal_like(400 + it, OC, IC, 3, 3) * 0.1).cuda().requires_grad_(True)
        b = gen.normal_like(500 + it, OC).cuda().requires_grad_(True)
        go = gen.normal_like(600 + it, N, OC, H, W).cuda()
        F.conv2d(x, w, b, 1, 1).backward(go)
        torch.cuda.synchronize()
        assert torch.equal(x.grad, ops.conv2d_grad_input(x.shape, w.detach(), go, (1, 1), (1, 1))), it
        assert torch.equal(w.grad, ops.conv2d_grad_kernel(x.detach(), w.shape, go, (1, 1), (1, 1))), it
        assert torch.equal(b.grad, ops.sum4d_dim023(go)), it

        mean = gen.normal_like(700 + it, OC).cuda().requires_grad_(True)
        var = (gen.relu_like(800 + it, OC) + 0.5).cuda().requires_grad_(True)
        gamma = gen.normal_like(900 + it, OC).cuda().requires_grad_(True)
        beta = gen.normal_like(1000 + it, OC).cuda().requires_grad_(True)
        y = gen.normal_like(1100 + it, N, OC, H, W).cuda().requires_grad_(True)
        from repdl_amd.nn.functional import _BatchNorm
        _BatchNorm.apply(y, mean, var, gamma, beta, 1e-5).backward(go)
        torch.cuda.synchronize()
        std = ops.sqrt(var.detach() + 1e-5)
        pc = lambda t: t.view(1, -1, 1, 1)
        assert torch.equal(beta.grad, ops.sum4d_dim023(go)), it
        assert torch.equal(mean.grad, (-ops.div(gamma.detach(), std)) * ops.sum4d_dim023(go)), it
        assert torch.equal(gamma.grad, ops.sum4d_dim023(ops.div(y.detach() - pc(mean.detach()), pc(std).expand_as(y)) * go)), it
        coef = ops.div(gamma.detach(), 2 * std * std * std)
        assert torch.equal(var.grad, ops.sum4d_dim023(go * (pc(mean.detach()) - y.detach()) * pc(coef))), it


def _two_conv_grads(defer, accumulate=False, hook=False, keep=None):
    """Gradients of a two-layer convolution stack (the first layer's parameter gradients can be
    deferred: its input needs a gradient too) after one or two backward passes."""
    from repdl_amd.nn import functional as F

    old = F.defer_parameter_gradients
    F.defer_parameter_gradients = defer
    try:
        x = gen.relu_like(41, 8, 3, 24, 24).cuda().requires_grad_(True)
        w1 = (gen.normal_like(42, 16, 3, 3, 3) * 0.2).cuda().requires_grad_(True)
        b1 = gen.normal_like(43, 16).cuda().requires_grad_(True)
        w2 = (gen.normal_like(44, 8, 16, 3, 3) * 0.1).cuda().requires_grad_(True)
        b2 = gen.normal_like(45, 8).cuda().requires_grad_(True)
        seen = []
        if hook:
            w1.register_hook(lambda g: seen.append(g.clone()))
        go = gen.normal_like(46, 8, 8, 24, 24).cuda()
        for _ in range(2 if accumulate else 1):
            y = F.conv2d(torch.relu(F.conv2d(x, w1, b1, 1, 1)), w2, b2, 1, 1)
            y.backward(go)
        torch.cuda.synchronize()
        out = [t.grad.clone() for t in (x, w1, b1, w2, b2)] + seen
        if keep is not None:
            keep.append(w1.grad)
        return out
    finally:
        F.defer_parameter_gradients = old


@pytest.mark.parametrize("accumulate,hook", [(False, False), (True, False), (False, True)])
def test_deferred_parameter_gradients(accumulate, hook):
    """Parameter gradients whose chains are joined only when the backward pass ends are the bits of
    the joined-at-once ones: on the first pass (deferred), on a second pass onto existing .grad
    (not deferred: autograd reads the gradient at once) and with a tensor hook (not deferred)."""
    from repdl_amd.nn import functional as F

    for _ in range(3):
        a = _two_conv_grads(False, accumulate, hook)
        before = F.deferred_stats["jobs"]
        b = _two_conv_grads(True, accumulate, hook)
        # weight and bias of both layers on a first pass (a second pass finds .grad filled and defers nothing);
        # a hook on w1 takes w1 out
        assert F.deferred_stats["jobs"] - before == (3 if hook else 4)
        assert len(a) == len(b) and all(torch.equal(p, q) for p, q in zip(a, b))


def test_deferred_gradient_that_autograd_copies(monkeypatch):
    """If something else holds the gradient tensor, autograd stores a copy of it in .grad -- made
    on the current stream while the chain may still be running on its side stream.  The end-of-pass
    callback writes the finished values into that copy."""
    from repdl_amd import ops

    want = _two_conv_grads(False)
    held = []
    real = ops.conv2d_grad_kernel

    def holding(*args, **kw):
        held.append(real(*args, **kw))
        return held[-1]

    monkeypatch.setattr(ops, "conv2d_grad_kernel", holding)
    from repdl_amd.nn import functional as F

    kept, before = [], F.deferred_stats["copies_rewritten"]
    got = _two_conv_grads(True, keep=kept)
    assert all(torch.equal(p, q) for p, q in zip(want, got))
    assert all(kept[0].data_ptr() != h.data_ptr() for h in held)  # .grad is a copy, not a held tensor
    assert F.deferred_stats["copies_rewritten"] - before == 2     # both layers' weights
