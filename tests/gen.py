"""Deterministic, platform-independent input generators for the parity tests.

Everything is derived from PCG64 *integer* draws followed by exact (or
single, IEEE-defined) float conversions, so the same seed gives the same bytes
in the container that wrote the golden vectors and on the GPU box.
"""
from __future__ import annotations

import hashlib

import numpy as np
import torch


def _rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def normal_like(seed: int, *shape: int) -> torch.Tensor:
    """Approximately N(0,1): centred sum of four uniform 32-bit integers (exact
    in float64), scaled, rounded once to float32."""
    n = int(np.prod(shape)) if shape else 1
    u = _rng(seed).integers(0, 2**32, size=(n, 4), dtype=np.uint64).sum(axis=1)
    x = (u.astype(np.float64) - 2.0 * 2.0**32) * (np.sqrt(3.0) / 2.0**32)
    return torch.from_numpy(x.astype(np.float32).reshape(shape))


def relu_like(seed: int, *shape: int) -> torch.Tensor:
    """normal_like clipped at zero (post-ReLU-like activations)."""
    return normal_like(seed, *shape).clamp_(min=0)


def uniform_pm1(seed: int, *shape: int) -> torch.Tensor:
    """Uniform multiples of 2^-23 in [-1, 1)."""
    n = int(np.prod(shape)) if shape else 1
    k = _rng(seed).integers(-(2**23), 2**23, size=n, dtype=np.int64)
    return torch.from_numpy((k.astype(np.float64) / 2.0**23).astype(np.float32).reshape(shape))


def scaled_normal(seed: int, *shape: int, lo: int = -20, hi: int = 20) -> torch.Tensor:
    """normal_like times 2^e, e a uniform integer in [lo, hi]: magnitudes spread
    over 40 binades, which makes a sum's value depend on its evaluation order."""
    n = int(np.prod(shape)) if shape else 1
    base = normal_like(seed, n).numpy()
    e = _rng(seed + 7919).integers(lo, hi + 1, size=n, dtype=np.int64)
    return torch.from_numpy(np.ldexp(base, e.astype(np.int32)).astype(np.float32).reshape(shape))


def small_ints(seed: int, *shape: int, lo: int = -8, hi: int = 8) -> torch.Tensor:
    """Small integers as float32: every product and partial sum is exact."""
    n = int(np.prod(shape)) if shape else 1
    k = _rng(seed).integers(lo, hi + 1, size=n, dtype=np.int64)
    return torch.from_numpy(k.astype(np.float32).reshape(shape))


SPECIAL_BITS = np.array(
    [
        0x00000000, 0x80000000,  # +-0
        0x00000001, 0x80000001, 0x007FFFFF, 0x807FFFFF, 0x00400000, 0x00000100,  # subnormals
        0x00800000, 0x80800000,  # smallest normals
        0x7F800000, 0xFF800000,  # +-inf
        0x7FC00000, 0xFFC00000, 0x7FC00001, 0xFFC12345, 0x7F812345, 0xFF812345,  # NaNs (quiet, signalling)
        0x7F7FFFFF, 0xFF7FFFFF,  # +-max
        0x42B17217, 0x42B17218, 0x42B17219,  # exp overflow threshold
        0xC2CFF1B4, 0xC2CFF1B5, 0xC2CFF1B6,  # exp underflow to zero
        0xC2AEAC4F, 0xC2AEAC50,  # exp result becomes subnormal
        0x33000000, 0xB3000000, 0x32FFFFFF, 0x33000001, 0xB2800000, 0xB2800001,  # |x| ~ 2^-25
        0x3F800000, 0xBF800000, 0x3F7FFFFF, 0x3F800001,  # +-1 and neighbours
        0x41200000, 0x40000000, 0x3F000000,
    ],
    dtype=np.uint32,
)


def log_uniform_bits(seed: int, n: int) -> np.ndarray:
    """sign * 2^U: random sign, exponent field uniform over the normal range
    1..254, random mantissa."""
    r = _rng(seed)
    sign = r.integers(0, 2, size=n, dtype=np.uint32) << np.uint32(31)
    expo = r.integers(1, 255, size=n, dtype=np.uint32) << np.uint32(23)
    mant = r.integers(0, 2**23, size=n, dtype=np.uint32)
    return sign | expo | mant


def elementwise_mix(seed: int, n: int, special_fraction: float = 0.1) -> torch.Tensor:
    """90 % log-uniform over the normal range with random sign, 10 % special
    values (zeros, subnormals, infinities, NaNs, exp thresholds, random
    subnormals)."""
    bits = log_uniform_bits(seed, n)
    r = _rng(seed + 104729)
    pick = r.random(n) < special_fraction
    k = int(pick.sum())
    choice = r.integers(0, len(SPECIAL_BITS) + 8, size=k)
    sub = (r.integers(0, 2, size=k, dtype=np.uint32) << np.uint32(31)) | r.integers(1, 2**23, size=k, dtype=np.uint32)
    spec = np.where(choice < len(SPECIAL_BITS), SPECIAL_BITS[np.minimum(choice, len(SPECIAL_BITS) - 1)], sub)
    bits[pick] = spec.astype(np.uint32)
    return torch.from_numpy(bits.view(np.float32).copy())


def positive_mix(seed: int, n: int) -> torch.Tensor:
    """elementwise_mix with the sign cleared on 3/4 of the entries, so log and
    sqrt see mostly valid arguments."""
    x = elementwise_mix(seed, n).numpy().view(np.uint32).copy()
    keep = _rng(seed + 31).integers(0, 4, size=n) == 0
    x[~keep] &= np.uint32(0x7FFFFFFF)
    return torch.from_numpy(x.view(np.float32).copy())


def labels(seed: int, n: int, classes: int) -> torch.Tensor:
    return torch.from_numpy(_rng(seed).integers(0, classes, size=n, dtype=np.int64))


def sha256(t: torch.Tensor) -> str:
    """Hash convention of repdl/utils.py:10-13: SHA-256 of the raw bytes."""
    return hashlib.sha256(t.detach().cpu().contiguous().numpy().tobytes()).hexdigest()


def words(t: torch.Tensor, k: int = 4) -> list[str]:
    """First and last k raw 32-bit words, hex (for debugging a hash mismatch)."""
    flat = t.detach().cpu().contiguous().view(-1)
    if flat.numel() == 0:
        return []
    if flat.dtype == torch.float32:
        u = flat.numpy().view(np.uint32)
    else:
        u = flat.numpy().astype(np.uint32)
    idx = list(range(min(k, len(u)))) + list(range(max(len(u) - k, 0), len(u)))
    return ["%08x" % int(u[i]) for i in idx]


GENERATORS = {
    "normal": normal_like,
    "relu": relu_like,
    "uniform_pm1": uniform_pm1,
    "scaled_normal": scaled_normal,
    "small_ints": small_ints,
}


def make(kind: str, seed: int, *shape: int) -> torch.Tensor:
    if kind == "mix":
        return elementwise_mix(seed, int(np.prod(shape))).reshape(shape)
    if kind == "positive_mix":
        return positive_mix(seed, int(np.prod(shape))).reshape(shape)
    return GENERATORS[kind](seed, *shape)
