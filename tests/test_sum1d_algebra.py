"""The algebra behind the parallel sequential sum (repdl_amd/csrc/sum1d.hip), restated
in Python and checked against numpy's strictly sequential float32 accumulation:
chunk maps S -> S + a[S & 1] with prefix bounds, their composition, the validity test
and the walk with replay.  Data sets are built to cross binades, change sign, tie and
hover at binade edges.  (The GPU kernel itself is compared with the oracle in the GPU
tests; this pins the method.)"""
import numpy as np
import pytest

BIG, SAT = 1 << 26, 1 << 28
NONE, ANY = -1, 0x200


def clampi(v):
    return max(-SAT, min(SAT, v))


def append(t, ux, sg, e):
    ex = (ux >> 23) & 0xFF
    m = ux & 0x7FFFFF
    if ex == 0:
        ex = 1
    else:
        m |= 0x800000
    if m == 0:
        return t
    neg = (ux >> 31) != sg
    d = e - ex
    if d < 0:
        X = a0 = a1 = -BIG if neg else BIG
    elif d > 25:
        X, a0, a1 = (-1 if neg else 0), 0, 0
    else:
        v = -m if neg else m
        X = v >> d
        rem = v & ((1 << d) - 1)
        half = 0 if d == 0 else 1 << (d - 1)
        gt = 1 if d and rem > half else 0
        tie = 1 if d and rem == half else 0
        a0 = X + gt + (tie & (X & 1))
        a1 = X + gt + (tie & ((X + 1) & 1))
    t0, t1, lo0, hi0, lo1, hi1 = t
    ea0 = a1 if (t0 & 1) else a0
    ea1 = a1 if ((1 + t1) & 1) else a0
    lo0, lo1 = clampi(min(lo0, t0 + X)), clampi(min(lo1, t1 + X))
    t0, t1 = clampi(t0 + ea0), clampi(t1 + ea1)
    return (t0, t1, lo0, max(hi0, t0), lo1, max(hi1, t1))


def compose(a, b):
    p0, p1 = a[0] & 1, (1 + a[1]) & 1
    bt0, blo0, bhi0 = (b[1], b[4], b[5]) if p0 else (b[0], b[2], b[3])
    bt1, blo1, bhi1 = (b[1], b[4], b[5]) if p1 else (b[0], b[2], b[3])
    return (clampi(a[0] + bt0), clampi(a[1] + bt1), clampi(min(a[2], a[0] + blo0)), clampi(max(a[3], a[0] + bhi0)),
            clampi(min(a[4], a[1] + blo1)), clampi(max(a[5], a[1] + bhi1)))


def apply(s, t, hyp):
    if hyp == ANY:
        return s, True
    if hyp < 0 or (s >> 23) != hyp:
        return s, False
    S0 = (s & 0x7FFFFF) | 0x800000
    tt, lo, hi = (t[1], t[4], t[5]) if S0 & 1 else (t[0], t[2], t[3])
    if S0 + lo < 0x800000 or S0 + hi > 0xFFFFFF:
        return s, False
    return (hyp << 23) | ((S0 + tt) & 0x7FFFFF), True


def parallel_sum(x, chunk=16, group=8):
    """chunk tuples under hypotheses from a float64 prefix, groups of chunks composed
    (in a tree, to exercise associativity), then the serial walk with replay."""
    ux = x.view(np.uint32)
    n = len(x)
    approx = np.concatenate([[0.0], np.cumsum(x.astype(np.float64))])
    nch = (n + chunk - 1) // chunk
    tups, hyps = [], []
    for c in range(nch):
        seg = ux[c * chunk:(c + 1) * chunk]
        us = int(np.float32(approx[c * chunk]).view(np.uint32))
        eh = (us >> 23) & 0xFF
        hyp = (us >> 23) if 1 <= eh <= 254 else NONE
        if np.any((seg & 0x7FFFFFFF) >= 0x7F800000):
            hyp = NONE
        if np.all((seg & 0x7FFFFFFF) == 0):
            hyp = ANY
        t = (0, 0, 0, 0, 0, 0)
        if hyp >= 0 and hyp != ANY:
            for u in seg:
                t = append(t, int(u), hyp >> 8, hyp & 0xFF)
        tups.append(t)
        hyps.append(hyp)

    def merge(a, b):
        if a == ANY:
            return b
        if b == ANY:
            return a
        return a if a == b else NONE

    def tree(ts, hs):
        while len(ts) > 1:
            nt, nh = [], []
            for i in range(0, len(ts), 2):
                if i + 1 < len(ts):
                    nt.append(compose(ts[i], ts[i + 1]))
                    nh.append(merge(hs[i], hs[i + 1]))
                else:
                    nt.append(ts[i])
                    nh.append(hs[i])
            ts, hs = nt, nh
        return ts[0], hs[0]

    s = 0
    replayed = 0
    for g0 in range(0, nch, group):
        gt, gh = tree(tups[g0:g0 + group], hyps[g0:g0 + group])
        s2, ok = apply(s, gt, gh)
        if ok:
            s = s2
            continue
        for c in range(g0, min(g0 + group, nch)):
            s2, ok = apply(s, tups[c], hyps[c])
            if ok:
                s = s2
                continue
            replayed += 1
            acc = np.uint32(s).view(np.float32)
            for v in x[c * chunk:(c + 1) * chunk]:
                acc = np.float32(acc + v)
            s = int(acc.view(np.uint32))
    return s, replayed, nch


def sequential(x):
    with np.errstate(all="ignore"):
        return int(np.add.accumulate(x, dtype=np.float32)[-1].view(np.uint32))


def _rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def datasets():
    r = _rng(1)
    yield "uniform_pm1", (r.integers(-2**23, 2**23, 6000) / 2.0**23).astype(np.float32)
    yield "positive_drift", (r.random(6000) * 3).astype(np.float32)
    yield "negative_drift", (-r.random(6000) * 3).astype(np.float32)
    yield "wide_exponents", (r.standard_normal(6000) * np.exp2(r.integers(-30, 30, 6000))).astype(np.float32)
    # hover around a binade edge: +-1 steps around 1024 with tiny noise
    base = np.concatenate([[1024.0], np.where(r.random(5000) < 0.5, 1.0, -1.0) + r.standard_normal(5000) * 1e-3])
    yield "hover_edge", base.astype(np.float32)
    # many exact ties: state 2^24-ish, adding 1.0 (half a quantum of the next binade)
    yield "ties", np.concatenate([[2.0**24], np.ones(3000), [-2.0**23], np.full(3000, 0.5)]).astype(np.float32)
    yield "tiny_after_big", np.concatenate([[1e8], r.random(4000) * 1e-3, [-1e8], r.random(2000)]).astype(np.float32)
    yield "zeros_and_signs", np.concatenate([np.zeros(100), [1.5, -1.5], -np.zeros(50), [2.0**-140, -2.0**-141] * 50, r.standard_normal(500)]).astype(np.float32)
    sp = np.concatenate([r.standard_normal(2000), [np.inf], r.standard_normal(100), [-np.inf], r.standard_normal(50)])
    yield "inf_nan", sp.astype(np.float32)
    yield "subnormal_state", (r.integers(-2**20, 2**20, 3000).astype(np.float64) * 2.0**-149).astype(np.float32)
    yield "cancel_to_zero", np.tile(np.array([3.25, -3.25, 1e-3, -1e-3], dtype=np.float32), 800)


@pytest.mark.parametrize("name,x", list(datasets()), ids=[n for n, _ in datasets()])
def test_parallel_equals_sequential(name, x):
    for chunk, group in ((16, 8), (64, 4), (7, 3)):
        got, replayed, nch = parallel_sum(x, chunk, group)
        assert got == sequential(x), (name, chunk, group)
    if name in ("uniform_pm1", "positive_drift", "negative_drift"):
        assert replayed < nch // 2  # the maps really carry most of the work


def test_composition_is_associative():
    r = _rng(2)
    x = (r.standard_normal(300) * 4 + 700).astype(np.float32).view(np.uint32)
    hyp = int(np.float32(700.0).view(np.uint32)) >> 23
    ts = []
    for i in range(0, 300, 10):
        t = (0, 0, 0, 0, 0, 0)
        for u in x[i:i + 10]:
            t = append(t, int(u), hyp >> 8, hyp & 0xFF)
        ts.append(t)
    left = ts[0]
    for t in ts[1:]:
        left = compose(left, t)
    right = ts[-1]
    for t in reversed(ts[:-1]):
        right = compose(t, right)
    assert left == right
