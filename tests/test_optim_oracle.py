"""Pins the oracle's optimizer steps (oracle/repdl_oracle.c, repdl_oracle_adam_step and
repdl_oracle_sgd_step) without a GPU:

* against the sequence of PyTorch CPU tensor operations that RepDL's Adam is
  (repdl/optim.py:56-83, with ops.sqrt and ops.div spelled as the reference's CPU
  branches spell them, repdl/ops.py:98-103, 122-123), over several steps;
* against exact rational arithmetic with one rounding per operation on a few hundred
  elements, which fixes where each rounding sits (a fused or a split multiply-add, a
  reciprocal in place of a division, a dropped eps would all fail it).
NaN results compare as NaN: PyTorch's vector and scalar loops already disagree on NaN
payloads.
"""
import math
from fractions import Fraction

import numpy as np
import pytest
import torch

import gen
from oracle import api as oracle
from test_oracle_pin import fma32, rn32


def bits(t: torch.Tensor) -> np.ndarray:
    """int32 view with every NaN mapped to one pattern."""
    a = t.detach().cpu().contiguous().numpy()
    b = a.view(np.uint32).copy()
    b[np.isnan(a)] = 0x7FC00000
    return b


def data(kind: str, seed: int, n: int):
    """(param, grad) of n elements."""
    if kind == "training":  # weights ~ N(0,1)/8, gradients spread over 40 binades
        return gen.normal_like(seed, n) * 0.125, gen.scaled_normal(seed + 1, n, lo=-30, hi=10)
    if kind == "special":  # zeros, subnormals, infinities, NaNs, extremes
        return gen.elementwise_mix(seed, n), gen.elementwise_mix(seed + 1, n)
    if kind == "tiny":  # squares underflow, v stays subnormal or zero
        return gen.normal_like(seed, n), gen.scaled_normal(seed + 1, n, lo=-80, hi=-60)
    raise ValueError(kind)


def torch_adam_steps(p, grads, lr, betas, eps, wd, amsgrad):
    """The reference's operation sequence on CPU tensors; returns the final state."""
    beta1, beta2 = betas
    p = p.clone()
    m, v = torch.zeros_like(p), torch.zeros_like(p)
    vmax = torch.zeros_like(p) if amsgrad else None
    for step, grad in enumerate(grads, 1):
        bc1, bc2 = 1 - beta1 ** step, 1 - beta2 ** step
        if wd != 0:
            grad = grad.add(p, alpha=wd)
        m.mul_(beta1).add_(grad, alpha=1 - beta1)
        v.mul_(beta2).add_(torch.mul(grad, grad).mul(1 - beta2))
        second = v
        if amsgrad:
            torch.maximum(vmax, v, out=vmax)
            second = vmax
        root = second.to(dtype=torch.float64).sqrt().to(dtype=torch.float32)
        denom = root.div(math.sqrt(bc2)).add_(eps)
        p.add_(torch.div(m, denom).mul(-(lr / bc1)))
    return p, m, v, vmax


def oracle_adam_steps(p, grads, lr, betas, eps, wd, amsgrad):
    p = p.clone()
    m, v = torch.zeros_like(p), torch.zeros_like(p)
    vmax = torch.zeros_like(p) if amsgrad else None
    for step, grad in enumerate(grads, 1):
        oracle.adam_step(p, grad, m, v, vmax, step, lr, betas, eps, wd)
    return p, m, v, vmax


CONFIGS = [
    dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, wd=0.0, amsgrad=False),
    dict(lr=1e-2, betas=(0.9, 0.999), eps=1e-8, wd=1e-2, amsgrad=True),
    dict(lr=3e-4, betas=(0.8, 0.95), eps=1e-6, wd=0.1, amsgrad=False),
    dict(lr=0.5, betas=(0.0, 0.5), eps=1e-3, wd=0.0, amsgrad=True),
]


@pytest.mark.parametrize("kind", ["training", "special", "tiny"])
@pytest.mark.parametrize("cfg", range(len(CONFIGS)))
@pytest.mark.parametrize("n", [1, 7, 8, 1000, 40003])
def test_adam_equals_torch_cpu_sequence(kind, cfg, n):
    """Lengths on both sides of PyTorch's vector width: its vector body and scalar tail
    must both be the fused multiply-add the oracle writes."""
    c = CONFIGS[cfg]
    p, g0 = data(kind, 900 + cfg, n)
    grads = [g0] + [data(kind, 910 + 3 * s + cfg, n)[1] for s in range(3)]
    want = torch_adam_steps(p, grads, **c)
    got = oracle_adam_steps(p, grads, **c)
    for w, g, name in zip(want, got, ("param", "exp_avg", "exp_avg_sq", "max_exp_avg_sq")):
        if w is not None:
            assert np.array_equal(bits(w), bits(g)), name


@pytest.mark.parametrize("n", [1, 5, 8, 4099])
def test_sgd_equals_two_torch_operations(n):
    p, g = data("training", 950, n)
    want = p.clone().sub_(g.mul(0.01))
    got = p.clone()
    oracle.sgd_step(got, g, 0.01)
    assert np.array_equal(bits(want), bits(got))
    # the fused form PyTorch's own SGD uses differs somewhere on enough data
    if n > 1000:
        assert not torch.equal(p.clone().add_(g, alpha=-0.01), got)


def f32(x: float) -> float:
    return float(np.float32(x))


def sqrt32(x: float) -> float:
    """Correctly rounded binary32 square root of a binary32 number, by integer arithmetic."""
    if x == 0:
        return x
    q = Fraction(x)
    # scale to an integer with an even power of two so that isqrt carries 60+ bits
    k = 0
    while q.denominator != 1 or q.numerator.bit_length() < 124 or k % 2:
        q *= 2
        k += 1
    r = math.isqrt(q.numerator)
    exact = r * r == q.numerator
    root = Fraction(r) / Fraction(2) ** (k // 2)
    if exact:
        return rn32(root)
    # the true root lies strictly between r and r+1 (scaled): no binary32 boundary can lie
    # there with 60 spare bits, so rounding the midpoint decides
    return rn32(root + Fraction(1, 2) / Fraction(2) ** (k // 2))


def div32(a: float, b: float) -> float:
    return rn32(Fraction(a) / Fraction(b))


def test_adam_exact_rational():
    c = dict(lr=1e-2, betas=(0.9, 0.999), eps=1e-8, wd=1e-2)
    n = 300
    p0, g = data("training", 970, n)
    m0 = gen.normal_like(971, n) * 0.01
    v0 = (gen.scaled_normal(972, n, lo=-40, hi=0)) ** 2
    x0 = (gen.scaled_normal(973, n, lo=-40, hi=0)) ** 2
    step = 5
    beta1, beta2 = c["betas"]
    b1, c1, b2, c2 = f32(beta1), f32(1 - beta1), f32(beta2), f32(1 - beta2)
    eps, wd = f32(c["eps"]), f32(c["wd"])
    root_bc2 = f32(math.sqrt(1 - beta2 ** step))
    scale = f32(-(c["lr"] / (1 - beta1 ** step)))
    p, m, v, x = p0.clone(), m0.clone(), v0.clone(), x0.clone()
    oracle.adam_step(p, g, m, v, x, step, c["lr"], c["betas"], c["eps"], c["wd"])
    for i in range(n):
        pi, gi, mi, vi, xi = (float(t[i]) for t in (p0, g, m0, v0, x0))
        gi = fma32(wd, pi, gi)
        mi = fma32(c1, gi, rn32(Fraction(mi) * Fraction(b1)))
        gg = rn32(Fraction(gi) * Fraction(gi))
        vi = rn32(Fraction(rn32(Fraction(vi) * Fraction(b2))) + Fraction(rn32(Fraction(gg) * Fraction(c2))))
        xi = max(xi, vi)
        denom = rn32(Fraction(div32(sqrt32(xi), root_bc2)) + Fraction(eps))
        pi = rn32(Fraction(pi) + Fraction(rn32(Fraction(div32(mi, denom)) * Fraction(scale))))
        assert (float(p[i]), float(m[i]), float(v[i]), float(x[i])) == (pi, mi, vi, xi), i


def test_sqrt32_helper():
    x = gen.positive_mix(980, 3000)
    x = x[torch.isfinite(x) & (x > 0)]
    want = x.to(torch.float64).sqrt().to(torch.float32)
    for a, w in zip(x.tolist()[:1500], want.tolist()):
        assert sqrt32(a) == w
