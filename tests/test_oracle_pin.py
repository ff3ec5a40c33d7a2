"""Checks that pin the C oracle independently of the golden digests: exact
rational arithmetic with one rounding per step on tiny inputs, integer-valued
data on which every evaluation order is exact (so PyTorch must agree bit for
bit), order sensitivity, skipped-versus-padded taps, the mean factor, and the
IEEE operators against PyTorch's CPU kernels (what RepDL's div / sqrt are)."""
from fractions import Fraction

import numpy as np
import pytest
import torch

import gen
from oracle import api as oracle


# ---- exact binary32 rounding of a rational, round-to-nearest-even -------------------------
def rn32(q: Fraction) -> float:
    if q == 0:
        return 0.0
    sign = -1 if q < 0 else 1
    a = abs(q)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    # a in [2^e, 2^(e+1)); quantum 2^(e-23), at least 2^-149
    qe = max(e - 23, -149)
    scaled = a / Fraction(2) ** qe
    n = scaled.numerator // scaled.denominator
    rem = scaled - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (n & 1)):
        n += 1
    val = Fraction(n) * Fraction(2) ** qe
    if val >= Fraction(2) ** 128:
        return sign * float("inf")
    return sign * float(val)


def fma32(a: float, b: float, c: float) -> float:
    return rn32(Fraction(a) * Fraction(b) + Fraction(c))


def add32(a: float, b: float) -> float:
    return rn32(Fraction(a) + Fraction(b))


def t32(x):
    return torch.tensor(x, dtype=torch.float32)


def test_rn32_against_numpy():
    rng = np.random.Generator(np.random.PCG64(1))
    for _ in range(2000):
        v = float(rng.standard_normal()) * 10.0 ** float(rng.integers(-44, 38))
        assert rn32(Fraction(v)) == float(np.float32(v))


@pytest.mark.parametrize("tA,tB", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_mm_exact_rational(tA, tB):
    M, N, K = 3, 4, 7
    a = gen.scaled_normal(11, M, K, lo=-12, hi=12)
    b = gen.scaled_normal(12, K, N, lo=-12, hi=12)
    want = torch.empty(M, N)
    for i in range(M):
        for j in range(N):
            s = 0.0
            for k in range(K):
                s = fma32(float(a[i, k]), float(b[k, j]), s)
            want[i, j] = s
    A = a.t().contiguous() if tA else a
    B = b.t().contiguous() if tB else b
    assert torch.equal(oracle.mm(A, B, bool(tA), bool(tB)), want)
    # a fused multiply-add is not a multiply followed by an add: this data tells them apart
    unfused = torch.empty(M, N)
    for i in range(M):
        for j in range(N):
            s = 0.0
            for k in range(K):
                s = add32(rn32(Fraction(float(a[i, k])) * Fraction(float(b[k, j]))), s)
            unfused[i, j] = s
    assert not torch.equal(unfused, want)


def _conv_brute(x, w, sH, sW, pH, pW, groups):
    N, IC, H, W = x.shape
    OC, ICg, KH, KW = w.shape
    OH, OW = (H + 2 * pH - KH) // sH + 1, (W + 2 * pW - KW) // sW + 1
    out = torch.empty(N, OC, OH, OW)
    for n in range(N):
        for oc in range(OC):
            g = oc // (OC // groups)
            for oh in range(OH):
                for ow in range(OW):
                    s = 0.0
                    for i in range(ICg):
                        for kh in range(KH):
                            for kw in range(KW):
                                h, ww = oh * sH - pH + kh, ow * sW - pW + kw
                                if 0 <= h < H and 0 <= ww < W:
                                    s = fma32(float(x[n, g * ICg + i, h, ww]), float(w[oc, i, kh, kw]), s)
                    out[n, oc, oh, ow] = s
    return out


def test_conv2d_exact_rational():
    x = gen.scaled_normal(21, 1, 4, 5, 4, lo=-8, hi=8)
    w = gen.scaled_normal(22, 2, 2, 3, 2, lo=-8, hi=8)
    assert torch.equal(oracle.conv2d(x, w, 2, 1, 1, 1, 2), _conv_brute(x, w, 2, 1, 1, 1, 2))


def test_conv_grads_exact_rational():
    # grad_input and grad_kernel as explicit chains in the reference's loop order
    N, IC, H, W, OC, KH, KW, sH, sW, pH, pW = 2, 2, 5, 4, 3, 3, 2, 2, 1, 1, 1
    OH, OW = (H + 2 * pH - KH) // sH + 1, (W + 2 * pW - KW) // sW + 1
    x = gen.scaled_normal(31, N, IC, H, W, lo=-6, hi=6)
    w = gen.scaled_normal(32, OC, IC, KH, KW, lo=-6, hi=6)
    go = gen.scaled_normal(33, N, OC, OH, OW, lo=-6, hi=6)
    gi = torch.empty(N, IC, H, W)
    for n in range(N):
        for ic in range(IC):
            for h in range(H):
                for ww in range(W):
                    s = 0.0
                    for oc in range(OC):
                        for kh in range(KH):
                            for kw in range(KW):
                                th, tw = h - kh + pH, ww - kw + pW
                                if th % sH or tw % sW:
                                    continue
                                oh, ow = th // sH, tw // sW
                                if 0 <= oh < OH and 0 <= ow < OW and th >= 0 and tw >= 0:
                                    s = fma32(float(go[n, oc, oh, ow]), float(w[oc, ic, kh, kw]), s)
                    gi[n, ic, h, ww] = s
    assert torch.equal(oracle.conv2d_grad_input(go, w, H, W, sH, sW, pH, pW), gi)
    gk = torch.empty(OC, IC, KH, KW)
    for oc in range(OC):
        for ic in range(IC):
            for kh in range(KH):
                for kw in range(KW):
                    s = 0.0
                    for n in range(N):
                        for oh in range(OH):
                            for ow in range(OW):
                                h, ww = oh * sH - pH + kh, ow * sW - pW + kw
                                if 0 <= h < H and 0 <= ww < W:
                                    s = fma32(float(go[n, oc, oh, ow]), float(x[n, ic, h, ww]), s)
                    gk[oc, ic, kh, kw] = s
    assert torch.equal(oracle.conv2d_grad_kernel(go, x, KH, KW, sH, sW, pH, pW), gk)


def test_integer_data_equals_torch():
    """With small integers every product and partial sum is exact, so any correct
    implementation, in any order, gives the same bits."""
    a, b = gen.small_ints(41, 37, 53), gen.small_ints(42, 53, 29)
    assert torch.equal(oracle.mm(a, b), a @ b)
    assert torch.equal(oracle.mm(a.t().contiguous(), b.t().contiguous(), True, True), a @ b)
    x = gen.small_ints(43, 2, 4, 9, 8, lo=-4, hi=4).requires_grad_(True)
    w = gen.small_ints(44, 6, 2, 3, 3, lo=-4, hi=4)
    y = torch.nn.functional.conv2d(x, w, None, (2, 1), (1, 2), 1, 2)
    assert torch.equal(oracle.conv2d(x.detach(), w, 2, 1, 1, 2, 2), y.detach())
    w1 = gen.small_ints(45, 5, 4, 3, 3, lo=-4, hi=4).requires_grad_(True)
    y1 = torch.nn.functional.conv2d(x, w1, None, (2, 1), (1, 2))
    go = gen.small_ints(46, *y1.shape, lo=-4, hi=4)
    y1.backward(go)
    assert torch.equal(oracle.conv2d_grad_input(go, w1.detach(), 9, 8, 2, 1, 1, 2), x.grad)
    assert torch.equal(oracle.conv2d_grad_kernel(go, x.detach(), 3, 3, 2, 1, 1, 2), w1.grad)
    m = gen.small_ints(47, 33, 65, lo=-100, hi=100)
    assert torch.equal(oracle.sum2d_dim0(m), m.sum(0)) and torch.equal(oracle.sum2d_dim1(m), m.sum(1))
    assert torch.equal(oracle.sum1d(m.reshape(-1)), m.sum())
    t4 = gen.small_ints(48, 3, 5, 4, 7, lo=-100, hi=100)
    assert torch.equal(oracle.sum4d_dim023(t4), t4.sum((0, 2, 3)))


def test_sums_are_sequential_chains():
    x = gen.scaled_normal(51, 5000)
    seq = np.add.accumulate(x.numpy(), dtype=np.float32)[-1]  # numpy accumulate is strictly sequential
    assert float(oracle.sum1d(x)) == float(seq)
    assert float(oracle.sum1d(x.flip(0))) != float(seq)  # the order matters on this data
    assert float(oracle.sum1d(x)) != float(x.sum())  # and it is not PyTorch's blocked order
    s = 0.0
    for v in x[:300].tolist():
        s = add32(s, v)
    assert float(oracle.sum1d(x[:300].contiguous())) == s
    m = gen.scaled_normal(52, 40, 60)
    assert torch.equal(oracle.sum2d_dim1(m), torch.from_numpy(np.add.accumulate(m.numpy(), axis=1, dtype=np.float32)[:, -1]))
    assert torch.equal(oracle.sum2d_dim0(m), torch.from_numpy(np.add.accumulate(m.numpy(), axis=0, dtype=np.float32)[-1]))
    t4 = gen.scaled_normal(53, 3, 4, 5, 6)
    per_channel = t4.permute(1, 0, 2, 3).reshape(4, -1).contiguous()  # (n,h,w) order per channel
    assert torch.equal(oracle.sum4d_dim023(t4), oracle.sum2d_dim1(per_channel))


def test_mean_is_one_multiply_by_rounded_reciprocal():
    # backend/cpu/summation.cpp:15,19: float(1.0/N) * sum, not sum / N
    found = False
    for seed in range(200):
        x = gen.uniform_pm1(6000 + seed, 7)
        s = float(oracle.sum1d(x))
        by_mul = float(np.float32(np.float32(1.0 / 7) * np.float32(s)))
        by_div = float(np.float32(s) / np.float32(7))
        assert float(oracle.sum1d(x, True)) == by_mul
        found |= by_mul != by_div
    assert found
    m = gen.uniform_pm1(61, 7, 3)
    assert torch.equal(oracle.sum2d_dim0(m, False, True), (oracle.sum2d_dim0(m) * np.float32(1.0 / 7)))


def test_skipped_taps_are_not_padded_zeros():
    """A tap outside the image is skipped (backend/cpu/convolution.cpp:38-44).
    Multiplying a padded zero instead would turn inf weights into NaN and a -0
    accumulator into +0."""
    x = torch.ones(1, 1, 2, 2)
    w = torch.zeros(1, 1, 3, 3)
    w[0, 0, 1, 1] = 2.0
    w[0, 0, 0, 0] = float("inf")  # only ever meets padding for output (0,0)
    y = oracle.conv2d(x, w, 1, 1, 1, 1, 1)
    assert float(y[0, 0, 0, 0]) == 2.0 and torch.isinf(y[0, 0, 1, 1])
    # -0 accumulator: the only in-image tap underflows to -0; later taps are padding
    xs = torch.full((1, 1, 1, 1), -1e-30)
    ws = torch.zeros(1, 1, 3, 3)
    ws[0, 0, 1, 1] = 1e-30
    ws[0, 0, 2, 2] = 1.0
    z = oracle.conv2d(xs, ws, 1, 1, 1, 1, 1)
    assert gen.words(z, 1)[0] == "80000000"
    # grad_kernel: taps outside the image are skipped as well
    gk = oracle.conv2d_grad_kernel(torch.full((1, 1, 2, 2), float("inf")), torch.ones(1, 1, 2, 2), 3, 3, 1, 1, 1, 1)
    assert torch.isinf(gk).all() and not torch.isnan(gk).any()


def test_div_and_sqrt_equal_torch_cpu():
    """RepDL's div and sqrt ARE PyTorch CPU calls (repdl/ops.py:98-103, 122-123)."""
    a, b = gen.elementwise_mix(71, 1 << 20), gen.elementwise_mix(72, 1 << 20)
    as_int = lambda t: t.view(torch.int32)
    assert torch.equal(as_int(oracle.div(a, b)), as_int(a.div(b)))
    assert torch.equal(as_int(oracle.div(a, 10.0)), as_int(a.div(torch.tensor(10.0))))
    assert torch.equal(as_int(oracle.div(a, 10.0)), as_int(a.div(10.0)))
    assert torch.equal(as_int(oracle.sqrt(a)), as_int(a.to(torch.float64).sqrt().to(torch.float32)))
    sp = torch.from_numpy(gen.SPECIAL_BITS.view(np.float32).copy())
    A, B = sp.repeat_interleave(len(sp)), sp.repeat(len(sp))
    assert torch.equal(as_int(oracle.div(A, B)), as_int(A.div(B)))


def test_exp_log_equal_python_libm():
    import math

    x = gen.normal_like(81, 2000) * 30
    e = oracle.exp(x)
    for xi, ei in zip(x.tolist(), e.tolist()):
        try:
            want = float(np.float32(math.exp(xi)))
        except OverflowError:
            want = float("inf")
        assert ei == want
    p = gen.positive_mix(82, 2000)
    l = oracle.log(p)
    for xi, li in zip(p.tolist(), l.tolist()):
        if xi > 0 and xi != float("inf"):
            assert li == float(np.float32(math.log(xi)))


def test_softmax_and_cross_entropy_compositions():
    x = gen.normal_like(91, 17, 23) * 4
    t = gen.labels(92, 17, 23)
    sh = x - x.max(1, keepdim=True).values
    e = oracle.exp(sh)
    s = oracle.sum2d_dim1(e, True)
    assert torch.equal(oracle.softmax(x), oracle.div(e, s.expand_as(e)))
    l = oracle.log(oracle.sum2d_dim1(e)) - sh.gather(1, t.unsqueeze(-1)).squeeze()
    assert torch.equal(oracle.cross_entropy(x, t), oracle.sum1d(l, True))
    ref = torch.nn.functional.cross_entropy(x, t)
    assert abs(float(oracle.cross_entropy(x, t)) - float(ref)) < 1e-5
