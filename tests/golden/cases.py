"""The list of golden cases: operator, parameters and input generator specs.

Shared by ``make_golden.py`` (which runs RepDL's own C++ CPU backend on them
and stores SHA-256 digests in ``golden.json``) and by the parity tests (which
run the oracle and the HIP backend on the same inputs).  Inputs are rebuilt
from ``tests/gen.py`` seeds, so no tensor data is stored.
"""
from __future__ import annotations

import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import gen  # noqa: E402

CASES: list[dict] = []


def _add(op: str, name: str, **kw) -> None:
    CASES.append(dict(op=op, name=f"{op}/{name}", **kw))


# ---- mm: (M, N, K, transA, transB), data kind -------------------------------------------
for i, (M, N, K, tA, tB, kind) in enumerate(
    [
        (1, 1, 1, 0, 0, "normal"),
        (3, 4, 0, 0, 0, "normal"),
        (33, 65, 129, 0, 0, "normal"),
        (64, 64, 64, 1, 0, "normal"),
        (17, 130, 77, 0, 1, "normal"),
        (5, 7, 300, 1, 1, "normal"),
        (128, 128, 1024, 0, 1, "scaled_normal"),
        (129, 257, 515, 1, 0, "scaled_normal"),
        (200, 100, 33, 0, 0, "relu"),
        (256, 384, 96, 0, 1, "normal"),
        (1024, 1024, 1024, 0, 0, "normal"),  # BASELINE config 1 shape
    ]
):
    _add("mm", f"{M}x{N}x{K}_tA{tA}_tB{tB}_{kind}", M=M, N=N, K=K, transA=tA, transB=tB, kind=kind, seed=1000 + i)

# ---- conv: (N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, groups) ----------------------------
CONV_SHAPES = [
    (2, 3, 9, 11, 4, 3, 3, 1, 1, 1, 1, 1),
    (2, 4, 10, 9, 6, 3, 2, 2, 1, 0, 1, 2),
    (1, 8, 7, 7, 8, 1, 1, 1, 1, 0, 0, 1),
    (3, 2, 12, 12, 5, 5, 5, 3, 2, 2, 2, 1),
    (2, 5, 8, 8, 7, 3, 3, 2, 2, 1, 1, 1),
    (1, 1, 5, 5, 1, 3, 3, 1, 1, 2, 2, 1),
    (4, 16, 14, 14, 32, 3, 3, 1, 1, 1, 1, 1),
    (2, 6, 6, 7, 6, 2, 3, 1, 2, 1, 0, 3),
    (2, 64, 28, 28, 64, 3, 3, 1, 1, 1, 1, 1),   # BASELINE config 5 layer, reduced image/batch
    (2, 256, 14, 14, 64, 1, 1, 1, 1, 0, 0, 1),  # BASELINE config 5 1x1 layer, reduced
]
for i, s in enumerate(CONV_SHAPES):
    N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, g = s
    tag = "n%d_ic%d_%dx%d_oc%d_k%dx%d_s%d%d_p%d%d_g%d" % s
    p = dict(N=N, IC=IC, H=H, W=W, OC=OC, KH=KH, KW=KW, sH=sH, sW=sW, pH=pH, pW=pW, groups=g)
    _add("conv2d", tag, **p, kind="relu", seed=2000 + i)
    if g == 1:
        _add("conv2d_grad_input", tag, **p, kind="normal", seed=2100 + i)
        _add("conv2d_grad_kernel", tag, **p, kind="relu", seed=2200 + i)

# ---- sums -------------------------------------------------------------------------------
for i, (n, kind) in enumerate(
    [(0, "normal"), (1, "normal"), (63, "uniform_pm1"), (64, "uniform_pm1"), (65, "scaled_normal"),
     (1000, "scaled_normal"), (4097, "uniform_pm1"), (100000, "uniform_pm1"), (100000, "scaled_normal"),
     (1 << 20, "uniform_pm1")]
):
    for avg in (0, 1):
        _add("sum1d", f"n{n}_{kind}_avg{avg}", n=n, average=avg, kind=kind, seed=3000 + i)

for i, (M, N, kind) in enumerate(
    [(1, 1, "normal"), (7, 5, "normal"), (64, 64, "scaled_normal"), (130, 257, "scaled_normal"),
     (1, 300, "uniform_pm1"), (300, 1, "uniform_pm1"), (64, 10, "normal"), (512, 1000, "scaled_normal")]
):
    for avg in (0, 1):
        _add("sum2d_dim0", f"{M}x{N}_{kind}_avg{avg}", M=M, N=N, average=avg, kind=kind, seed=3100 + i)
        _add("sum2d_dim1", f"{M}x{N}_{kind}_avg{avg}", M=M, N=N, average=avg, kind=kind, seed=3200 + i)

for i, (N, C, H, W, kind) in enumerate(
    [(1, 1, 1, 1, "normal"), (2, 3, 4, 5, "scaled_normal"), (4, 16, 7, 7, "scaled_normal"),
     (3, 5, 9, 13, "normal"), (8, 64, 14, 14, "scaled_normal")]
):
    for avg in (0, 1):
        _add("sum4d_dim023", f"{N}x{C}x{H}x{W}_{kind}_avg{avg}", N=N, C=C, H=H, W=W, average=avg, kind=kind,
             seed=3300 + i)

# ---- exp / log (glibc through the reference's exp2d / log1d) ----------------------------
_add("exp", "mix_4096", n=4096, kind="mix", seed=4000)
_add("exp", "mix_1M", n=1 << 20, kind="mix", seed=4001)
_add("exp", "normal_x8_65536", n=65536, kind="normal", seed=4002, scale=8.0)
_add("log", "positive_mix_4096", n=4096, kind="positive_mix", seed=4100)
_add("log", "positive_mix_1M", n=1 << 20, kind="positive_mix", seed=4101)
_add("log", "mix_65536", n=65536, kind="mix", seed=4102)

# ---- softmax / cross_entropy ------------------------------------------------------------
for i, (M, N, scale) in enumerate([(64, 10, 1.0), (5, 1, 1.0), (33, 100, 5.0), (128, 1000, 20.0), (1, 7, 3.0)]):
    _add("softmax", f"{M}x{N}_s{scale}", M=M, N=N, scale=scale, kind="normal", seed=5000 + i)
    _add("cross_entropy", f"{M}x{N}_s{scale}", M=M, N=N, scale=scale, kind="normal", seed=5100 + i)


def inputs(case: dict):
    """Build the input tensors of a case (torch CPU tensors)."""
    op, kind, seed = case["op"], case["kind"], case["seed"]
    if op == "mm":
        M, N, K = case["M"], case["N"], case["K"]
        a = gen.make(kind, seed, *((K, M) if case["transA"] else (M, K)))
        b = gen.make(kind, seed + 500, *((N, K) if case["transB"] else (K, N)))
        return a, b
    if op in ("conv2d", "conv2d_grad_input", "conv2d_grad_kernel"):
        c = case
        OH = (c["H"] + 2 * c["pH"] - c["KH"]) // c["sH"] + 1
        OW = (c["W"] + 2 * c["pW"] - c["KW"]) // c["sW"] + 1
        x = gen.make(kind, seed, c["N"], c["IC"], c["H"], c["W"])
        w = gen.make("normal", seed + 500, c["OC"], c["IC"] // c["groups"], c["KH"], c["KW"]) * 0.125
        go = gen.make("normal", seed + 900, c["N"], c["OC"], OH, OW)
        return x, w, go
    if op == "sum1d":
        return (gen.make(kind, seed, case["n"]),)
    if op in ("sum2d_dim0", "sum2d_dim1"):
        return (gen.make(kind, seed, case["M"], case["N"]),)
    if op == "sum4d_dim023":
        return (gen.make(kind, seed, case["N"], case["C"], case["H"], case["W"]),)
    if op in ("exp", "log"):
        x = gen.make(kind, seed, case["n"])
        if "scale" in case:
            x = x * case["scale"]
        return (x,)
    if op in ("softmax", "cross_entropy"):
        x = gen.make(kind, seed, case["M"], case["N"]) * case["scale"]
        t = gen.labels(seed + 77, case["M"], case["N"])
        return x, t
    raise KeyError(op)


def run(case: dict, backend, math_backend=None):
    """Run a case on a backend object exposing the reference's backend-module
    functions (``backend/cpu/bind.cpp:12-18``); ``math_backend`` supplies
    ``exp2d``/``log1d`` when ``backend`` has no ``exp``/``log``."""
    op = case["op"]
    t = inputs(case)
    c = case
    if op == "mm":
        return backend.mm(t[0], t[1], bool(c["transA"]), bool(c["transB"]))
    if op == "conv2d":
        return backend.conv2d(t[0], t[1], c["sH"], c["sW"], c["pH"], c["pW"], c["groups"])
    if op == "conv2d_grad_input":
        return backend.conv2d_grad_input(t[2], t[1], c["H"], c["W"], c["sH"], c["sW"], c["pH"], c["pW"])
    if op == "conv2d_grad_kernel":
        return backend.conv2d_grad_kernel(t[2], t[0], c["KH"], c["KW"], c["sH"], c["sW"], c["pH"], c["pW"])
    if op == "sum1d":
        return backend.sum1d(t[0], bool(c["average"]))
    if op in ("sum2d_dim0", "sum2d_dim1", "sum4d_dim023"):
        return getattr(backend, op)(t[0], True, bool(c["average"]))
    if op == "exp":
        if hasattr(backend, "exp"):
            return backend.exp(t[0])
        return math_backend.exp2d(t[0].reshape(1, -1)).reshape(-1)
    if op == "log":
        if hasattr(backend, "log"):
            return backend.log(t[0])
        return math_backend.log1d(t[0])
    if op == "softmax":
        return backend.softmax(t[0])
    if op == "cross_entropy":
        return backend.cross_entropy(t[0], t[1])
    raise KeyError(op)
