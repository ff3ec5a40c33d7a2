"""The device math (repdl_amd/csrc/crmath.h) compiled for the CPU and compared, bit
for bit, with the host: glibc exp/log through (float)f((double)x) exactly as
RepDL's backend/cpu/math.cpp:14-17, 32-35 computes them, IEEE sqrt and IEEE
division.  The same source is what the GPU kernels compile, and it uses only
IEEE +,-,*,fma, so agreement here is agreement of the algorithm; the GPU tests
then check the GPU executes it identically.

exp, log and sqrt are swept over ALL 2^32 bit patterns and x/10 over all 2^32
dividends (a few seconds each on 8 cores); set REPDL_SWEEP_STRIDE to thin them.
"""
import os

import mpmath as mp
import numpy as np
import pytest

import crmath_host
import gen

STRIDE = int(os.environ.get("REPDL_SWEEP_STRIDE", "1"))


def _bits(x: float) -> int:
    return int(np.array([x], dtype=np.float32).view(np.uint32)[0])


def _val(u: int) -> float:
    return float(np.array([u], dtype=np.uint32).view(np.float32)[0])


@pytest.mark.parametrize("fn", ["exp", "log", "sqrt"])
def test_unary_exhaustive(fn):
    L = crmath_host.lib()
    bad = np.zeros(64, dtype=np.uint32)
    n = getattr(L, "crmc_sweep_" + fn)(0, (1 << 32) // STRIDE, STRIDE, bad.ctypes.data, 64)
    assert n == 0, [hex(int(b)) for b in bad[: min(n, 16)]]


@pytest.mark.parametrize("divisor", [10.0, 3.0, 0.1, 1e-40, 3.0e38, -7.0])
def test_div_by_scalar_all_dividends(divisor):
    L = crmath_host.lib()
    bad = np.zeros(64, dtype=np.uint32)
    stride = STRIDE if divisor == 10.0 else max(STRIDE, 17)
    n = L.crmc_sweep_div_by(_bits(divisor), 0, (1 << 32) // stride, stride, bad.ctypes.data, 64)
    assert n == 0, [hex(int(b)) for b in bad[: min(n, 16)]]


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_div_random_pairs(mode):
    L = crmath_host.lib()
    bad = np.zeros(128, dtype=np.uint32)
    n = L.crmc_sweep_div_random(2024 + mode, 300_000_000 // max(STRIDE, 1), mode, bad.ctypes.data, 64)
    assert n == 0, [hex(int(b)) for b in bad[: min(2 * n, 16)]]


def test_div_special_pairs():
    L = crmath_host.lib()
    sp = [int(b) for b in gen.SPECIAL_BITS]
    for a in sp:
        for b in sp:
            assert L.crmc_div(a, b) == L.crmc_ref_div(a, b), (hex(a), hex(b))


# Known answers on x86-64 glibc (exp thresholds, signed zeros, NaN payloads):
# independent of the sweep's own reference call.
KNOWN = {
    "exp": {0x7FC00000: 0x7FC00000, 0xFFC00000: 0xFFC00000, 0xFF812345: 0xFFC12345, 0x7F800000: 0x7F800000,
            0xFF800000: 0x00000000, 0x00000000: 0x3F800000, 0x80000000: 0x3F800000, 0xBF800000: 0x3EBC5AB2,
            0x42B17217: 0x7F7FFF84, 0x42B17218: 0x7F800000, 0xC2CFF1B4: 0x00000001, 0xC2CFF1B5: 0x00000000,
            0xC2AEAC4F: 0x00800026, 0xC2AEAC50: 0x007FFFE6, 0x3F800000: 0x402DF854, 0x33000000: 0x3F800000},
    "log": {0x7FC00000: 0x7FC00000, 0xFF812345: 0xFFC12345, 0x7F800000: 0x7F800000, 0xFF800000: 0xFFC00000,
            0x00000000: 0xFF800000, 0x80000000: 0xFF800000, 0xBF800000: 0xFFC00000, 0x00000001: 0xC2CE8ED0,
            0x007FFFFF: 0xC2AEAC50, 0x42B17217: 0x408F895B, 0x3F800000: 0x00000000, 0x33000000: 0xC18AA123},
    "sqrt": {0x7FC00000: 0x7FC00000, 0xFFC00000: 0xFFC00000, 0xFF812345: 0xFFC12345, 0x7F800000: 0x7F800000,
             0xFF800000: 0x7FC00000, 0x00000000: 0x00000000, 0x80000000: 0x80000000, 0xBF800000: 0x7FC00000,
             0x00000001: 0x1A3504F3, 0x007FFFFF: 0x1FFFFFFF, 0x42B17217: 0x4116B55F, 0x33000000: 0x393504F3},
}


@pytest.mark.parametrize("fn", ["exp", "log", "sqrt"])
def test_known_answers(fn):
    L = crmath_host.lib()
    for x, want in KNOWN[fn].items():
        assert getattr(L, "crmc_" + fn)(x) == want, (fn, hex(x))


def _rn32(v) -> int:
    """Correct rounding of an mpmath real to binary32 bits (normal range)."""
    return _bits(float(np.float32(mp.mpf(v))))


def test_exp_log_are_correctly_rounded_on_random_inputs():
    """Independent of libm: for random arguments the result equals the exact value
    rounded once to binary32 (true for all but a handful of the 2^32 inputs)."""
    L = crmath_host.lib()
    mp.mp.prec = 200
    rng = np.random.Generator(np.random.PCG64(5))
    xs = (rng.random(400) * 170 - 85).astype(np.float32)
    for x in xs:
        u = _bits(float(x))
        want = mp.exp(mp.mpf(float(x)))
        got = _val(L.crmc_exp(u))
        lo, hi = np.nextafter(np.float32(got), np.float32(-np.inf)), np.nextafter(np.float32(got), np.float32(np.inf))
        assert abs(mp.mpf(got) - want) <= abs(mp.mpf(float(lo)) - want) and abs(mp.mpf(got) - want) <= abs(mp.mpf(float(hi)) - want)
    ps = np.exp(rng.random(400) * 160 - 80).astype(np.float32)
    for x in ps:
        u = _bits(float(x))
        want = mp.log(mp.mpf(float(x)))
        got = _val(L.crmc_log(u))
        lo, hi = np.nextafter(np.float32(got), np.float32(-np.inf)), np.nextafter(np.float32(got), np.float32(np.inf))
        assert abs(mp.mpf(got) - want) <= abs(mp.mpf(float(lo)) - want) and abs(mp.mpf(got) - want) <= abs(mp.mpf(float(hi)) - want)
