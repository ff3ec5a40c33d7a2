#!/usr/bin/env python3
"""Benchmark of the reproducible-operator hot path on one MI355X.

Headline (BASELINE.json `metric`): bit-exact fp32 `mm` GFLOP/s at 8192^3 -- the
`repdl.nn.Linear` forward shape x[8192,8192] . W[8192,8192]^T (transB).  A "step"
is one such product with the operands resident in HBM.  The same JSON line also
carries, under "also", the HBM-bound operators of the metric (row-wise and 1-D
sequential sums, exp, log, sqrt, div on 2^28 values), each with its own roofline
entry, and under "parity" the SHA-256 comparison of the GPU outputs with the CPU
checker on the same input bytes.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick] [--only mm]

The CPU baseline is RepDL's own C++ CPU backend (compiled into oracle/_ref from
the reference sources; kind "reference") when that build is present, otherwise
the plain-C restatement (kind "port"), timed on a bounded sample of the same
workload on the host cores.  Only the baseline and parity legs touch oracle/.
"""
from __future__ import annotations

import argparse
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_PEAK_TFLOPS = 157.3  # MI355X vendor fp32 figure (256 CU x 2.4 GHz x 256 flop/clk)
HBM_PEAK_GBS = 8000.0

# HBM bytes per launch from two `rocprofv3 --pmc` runs (FETCH_SIZE, then WRITE_SIZE), each scaled by
# what the same counter reads for a plain 1 GiB elementwise copy kernel (--copy-probe): FETCH_SIZE
# reads 524300 for 1 GiB (factor 1.99995 KiB per count), WRITE_SIZE 1048576 (factor 1.0).  Summary:
# profiles/hbm_traffic_counters.txt.  Valid for the default workload sizes only.
MEASURED_TRAFFIC_BYTES = {
    "mm": 5426902 * 1.99995 * 1024 + 262155 * 1024,       # 1.14e10: operand panels re-read behind L2 (35 % L2 hit rate)
    "exp": 524335 * 1.99995 * 1024 + 1048586 * 1024,      # 2.147e9 = the algorithmic 8 B/element
    "sum2d_dim1": 524389 * 1.99995 * 1024 + 64 * 1024,    # 1.074e9 = the algorithmic 4 B/element
    "adam_step": 524363 * 1.99995 * 1024 + 786443 * 1024,  # 1.879e9 = the algorithmic 28 B/element (2^26 elements)
}


def sha(t) -> str:
    return hashlib.sha256(t.detach().cpu().contiguous().numpy().tobytes()).hexdigest()


SETTLE_MS = 60.0  # secondary legs: launches before the timed ones, after the GPU sat idle behind a CPU checker


def time_gpu(fn, steps: int, warmup: int, settle_ms: float = 0.0):
    """Returns (wall ms per step, mean kernel ms from events on the launch stream, min kernel ms).

    settle_ms > 0 (the secondary legs): after the warm-up launches the same call is repeated until that
    much wall time has passed.  Each secondary leg starts after seconds of GPU idleness (its CPU parity
    check), and the first ~30 launches after such a pause are not steady state: a 0.37 ms log kernel
    reads 0.36, 0.44, 0.55, 0.51, ... 0.42 ms over its first 30 launches and 0.37 from then on.  The
    headline never uses it: exactly `warmup` launches, then `steps` timed ones."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    if settle_ms > 0.0:
        t_end = time.perf_counter() + settle_ms * 1e-3
        while time.perf_counter() < t_end:
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        fn()
        stops[i].record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    ev = [s.elapsed_time(e) for s, e in zip(starts, stops)]
    return wall, sum(ev) / len(ev), min(ev)


def hbm_entry(name, workload, algo_bytes, fn, steps, warmup, parity=None, cpu=None, traffic=None):
    wall, ev_mean, ev_min = time_gpu(fn, steps, warmup, SETTLE_MS)
    gbs = algo_bytes / (ev_mean * 1e-3) / 1e9
    out = {
        "op": name,
        "workload": workload,
        "value": round(gbs, 2),
        "unit": "GB/s",
        "ms_per_step": round(ev_mean, 4),
        "ms_min": round(ev_min, 4),
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": traffic},
    }
    if parity is not None:
        out["parity"] = parity
    if cpu is not None:
        out["cpu_baseline"] = cpu
    return out


def cpu_time(fn, reps=1):
    best = None
    for _ in range(reps):
        t0 = time.perf_counter()
        r = fn()
        dt = time.perf_counter() - t0
        best = dt if best is None or dt < best else best
    return best, r


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--quick", action="store_true", help="headline only, no secondary operators, no full parity")
    ap.add_argument("--only", default="", help="comma list of secondary ops to run (sum2d,sum1d,exp,log,sqrt,div,conv,linear,adam)")
    ap.add_argument("--size", type=int, default=8192, help="mm size (M=N=K); the metric is quoted at 8192")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 1 GiB elementwise copy kernel (torch.add(x, 0)), the known-size kernel "
                         "against which FETCH_SIZE / WRITE_SIZE counters are calibrated")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (every operator shards by outputs with no "
              "cross-device arithmetic, so a second GPU would only add an all-gather of outputs); run with --gpus 1", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    import repdl_amd
    from repdl_amd import _lib, ops

    from oracle import api as oracle  # checker / baseline legs only
    from oracle import ref as oracle_ref

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(dev)
    S = args.size
    only = set(x for x in args.only.split(",") if x)

    # ---------------- headline: mm S^3, Linear forward (NT) ----------------
    g = torch.Generator().manual_seed(0)
    x_h = torch.randn(S, S, generator=g)
    bound = 1.0 / (S ** 0.5)  # torch.nn.Linear default init: U(-1/sqrt(in), 1/sqrt(in))
    w_h = (torch.rand(S, S, generator=g) * 2 - 1) * bound
    x_d, w_d = x_h.to(dev), w_h.to(dev)
    out_holder = {}

    def step():
        out_holder["y"] = ops.mm(x_d, w_d, transB=True)

    wall_ms, ev_ms, ev_min = time_gpu(step, args.steps, args.warmup)
    flop = 2.0 * S * S * S
    gflops = flop / (wall_ms * 1e-3) / 1e9
    kern_tflops = flop / (ev_ms * 1e-3) / 1e12

    # parity of the headline output against the CPU checker on the same bytes
    parity = {}
    y_gpu = out_holder["y"]
    if not args.quick:
        t0 = time.perf_counter()
        y_cpu = oracle.mm(x_h, w_h, False, True)
        parity["mm"] = {"sha256_gpu": sha(y_gpu), "sha256_cpu": sha(y_cpu), "checker": "oracle (C restatement)",
                        "checker_s": round(time.perf_counter() - t0, 2)}
        parity["mm"]["equal"] = parity["mm"]["sha256_gpu"] == parity["mm"]["sha256_cpu"]
        del y_cpu

    # CPU baseline: the reference's own CPU backend on a row slab of the same product
    refmods = oracle_ref.load()
    rows = 256 if not args.quick else 64
    rows = min(rows, S)
    if refmods is not None:
        cpu_fn, kind = (lambda: refmods[0].mm(x_h[:rows], w_h, False, True)), "reference"
    else:
        cpu_fn, kind = (lambda: oracle.mm(x_h[:rows], w_h, False, True)), "port"
    dt, y_slab = cpu_time(cpu_fn)
    slab_equal = torch.equal(y_slab, y_gpu[:rows].cpu())
    cpu_baseline = {
        "value": round(2.0 * rows * S * S / dt / 1e9, 3), "unit": "GFLOP/s", "cores": oracle.threads(),
        "kind": kind,
        "sample": "first %d of %d output rows of the same %dx%dx%d NT product (%.1f s); GPU rows bit-equal: %s"
                  % (rows, S, S, S, S, dt, slab_equal),
    }
    del x_d, w_d, y_gpu, out_holder

    if _lib.lib().repdl_hip_matrix_path() == 1:
        kernel_name = "mm_mfma_fast_kernel<NT, 256x256x16 tile, 512 threads>"
        kernel_note = ("fp32 matrix-instruction peak; v_mfma_f32_32x32x2_f32, checked on this device to be a "
                       "k-ascending chain of single-rounding FMAs before use")
    else:
        kernel_name = "mm_kernel<NT>"
        kernel_note = ("fp32 compute peak; the matrix-instruction check failed on this device, so the kernel issues "
                       "v_fma_f32 only, whose issue-rate ceiling is half of this peak")
    result = {
        "metric": "bit-exact fp32 mm GFLOP/s at 8192^3",
        "value": round(gflops, 1),
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic (seeded host randn / uniform, same bytes for GPU and CPU checker)",
        "config": {"workload": "repdl.ops.mm fp32 %dx%dx%d, transB (nn.Linear forward), configs[3]" % (S, S, S),
                   "device": props.name, "cus": props.multi_processor_count},
        "roofline": {"bound": "mfma", "achieved": round(kern_tflops, 3), "peak": FP32_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(kern_tflops / FP32_PEAK_TFLOPS, 4),
                     "traffic": round(MEASURED_TRAFFIC_BYTES["mm"]) if S == 8192 and MEASURED_TRAFFIC_BYTES["mm"] else None,
                     "kernel": kernel_name, "kernel_ms": round(ev_ms, 4), "kernel_ms_min": round(ev_min, 4),
                     "note": kernel_note},
        "cpu_baseline": cpu_baseline,
        "parity": parity,
        "also_settle_ms": SETTLE_MS,
        "also": [],
    }

    if not args.quick:
        n = 1 << 28
        want = lambda k: (not only) or (k in only)
        sample = 1 << 24

        if want("sum2d"):
            R = 16384
            g = torch.Generator().manual_seed(1)
            m_h = torch.randn(R, R, generator=g) * torch.exp2(torch.rand(R, R, generator=g) * 40 - 20)
            m_d = m_h.to(dev)
            hold = {}
            def f(): hold["y"] = ops.sum2d_dim1(m_d)
            f()
            y_cpu = oracle.sum2d_dim1(m_h)
            par = {"equal": sha(hold["y"]) == sha(y_cpu), "sha256_gpu": sha(hold["y"])}
            dt, _ = cpu_time(lambda: (refmods[0].sum2d_dim1(m_h[:2048], False, False) if refmods else oracle.sum2d_dim1(m_h[:2048])))
            cpu = {"value": round(2048 * R * 4 / dt / 1e9, 3), "unit": "GB/s", "cores": oracle.threads(),
                   "kind": kind, "sample": "first 2048 rows"}
            result["also"].append(hbm_entry("sum2d_dim1", "row sums of 16384x16384 N(0,1)*2^U(-20,20)", 4.0 * R * R + 4 * R,
                                            f, args.steps, args.warmup, par, cpu,
                                            round(MEASURED_TRAFFIC_BYTES["sum2d_dim1"])))
            del m_d, m_h, hold

        if want("sum1d"):
            g = torch.Generator().manual_seed(2)
            v_h = torch.rand(n, generator=g) * 2 - 1
            v_d = v_h.to(dev)
            hold = {}
            def f(): hold["y"] = ops.sum1d(v_d)
            f()
            dt, y_cpu = cpu_time(lambda: (refmods[0].sum1d(v_h, False) if refmods else oracle.sum1d(v_h)))
            par = {"equal": sha(hold["y"]) == sha(y_cpu), "gpu": float(hold["y"]), "cpu": float(y_cpu)}
            cpu = {"value": round(n * 4 / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": kind,
                   "sample": "the full 2^28 vector (the reference's sum1d is single-threaded)"}
            result["also"].append(hbm_entry("sum1d", "sequential sum of 2^28 uniform[-1,1]", 4.0 * n, f,
                                            max(2, args.steps // 5), 1, par, cpu))
            del v_d, v_h, hold

        ew = [k for k in ("exp", "log", "sqrt", "div") if want(k)]
        if ew:
            sys.path.insert(0, os.path.join(ROOT, "tests"))
            import gen  # deterministic config-3 mix (90 % log-uniform, 10 % specials)

            e_h = gen.elementwise_mix(3, n)
            e_d = e_h.to(dev)
            for k in ew:
                hold = {}
                if k == "div":
                    fns = [("div_scalar", "x/10.0 on 2^28 mixed values", 8.0 * n, lambda: ops.div(e_d, 10.0),
                            lambda t: oracle.div(t, 10.0), lambda t: t.div(10.0))]
                    e2_h = gen.elementwise_mix(4, n)
                    e2_d = e2_h.to(dev)
                    fns.append(("div", "x/y on 2^28 mixed values", 12.0 * n, lambda: ops.div(e_d, e2_d), None,
                                lambda t: t.div(e2_h[: t.numel()])))
                else:
                    fns = [(k, "%s on 2^28 mixed values" % k, 8.0 * n, (lambda kk: (lambda: getattr(ops, kk)(e_d)))(k),
                            (lambda kk: (lambda t: getattr(oracle, kk)(t)))(k), None)]
                for name, wl, nbytes, gfn, ofn, tfn in fns:
                    def f(): hold["y"] = gfn()
                    f()
                    y_gpu_s = hold["y"][:sample].cpu()
                    if ofn is None:
                        y_cpu_s = oracle.div(e_h[:sample], e2_h[:sample])
                        dt, _ = cpu_time(lambda: oracle.div(e_h[:sample], e2_h[:sample]))
                    else:
                        y_cpu_s = ofn(e_h[:sample])
                        dt, _ = cpu_time(lambda: ofn(e_h[:sample]))
                    par = {"equal_on_first_2^24": sha(y_gpu_s) == sha(y_cpu_s)}
                    cpu = {"value": round(nbytes / n * sample / dt / 1e9, 3), "unit": "GB/s",
                           "cores": oracle.threads(), "kind": "port", "sample": "first 2^24 elements"}
                    result["also"].append(hbm_entry(name, wl, nbytes, f, args.steps, args.warmup, par, cpu,
                                                    round(MEASURED_TRAFFIC_BYTES["exp"]) if name == "exp" else None))
                    hold.clear()

        if want("conv"):
            for (N, IC, H, W, OC, Kk, st, pd) in [(64, 64, 56, 56, 64, 3, 1, 1), (64, 256, 56, 56, 64, 1, 1, 0)]:
                g = torch.Generator().manual_seed(5 + Kk)
                x_h = torch.randn(N, IC, H, W, generator=g).clamp_(min=0)
                w_h = torch.randn(OC, IC, Kk, Kk, generator=g) * (2.0 / (IC * Kk * Kk)) ** 0.5  # Kaiming normal
                OH, OW = (H + 2 * pd - Kk) // st + 1, (W + 2 * pd - Kk) // st + 1
                go_h = torch.randn(N, OC, OH, OW, generator=g)
                x_d, w_d, go_d = x_h.to(dev), w_h.to(dev), go_h.to(dev)
                flop = 2.0 * N * OC * OH * OW * IC * Kk * Kk
                legs = [
                    ("conv2d", lambda: ops.conv2d(x_d, w_d, (st, st), (pd, pd), 1),
                     lambda: oracle.conv2d(x_h, w_h, st, st, pd, pd, 1)),
                    ("conv2d_grad_input", lambda: ops.conv2d_grad_input(x_h.shape, w_d, go_d, (st, st), (pd, pd)),
                     lambda: oracle.conv2d_grad_input(go_h, w_h, H, W, st, st, pd, pd)),
                    ("conv2d_grad_kernel", lambda: ops.conv2d_grad_kernel(x_d, w_h.shape, go_d, (st, st), (pd, pd)),
                     lambda: oracle.conv2d_grad_kernel(go_h, x_h, Kk, Kk, st, st, pd, pd)),
                ]
                for name, gfn, ofn in legs:
                    hold = {}
                    def f(): hold["y"] = gfn()
                    wall, ev_mean, ev_min = time_gpu(f, args.steps, args.warmup, SETTLE_MS)
                    dt, y_cpu = cpu_time(ofn)
                    tf = flop / (ev_mean * 1e-3) / 1e12
                    result["also"].append({
                        "op": name, "workload": "batch %d, %dx%d conv %d->%d at %dx%d" % (N, Kk, Kk, IC, OC, H, W),
                        "value": round(tf * 1e3, 1), "unit": "GFLOP/s", "ms_per_step": round(ev_mean, 4),
                        "roofline": {"bound": "mfma", "achieved": round(tf, 3), "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                                     "frac": round(tf / FP32_PEAK_TFLOPS, 4), "traffic": None},
                        "parity": {"equal": sha(hold["y"]) == sha(y_cpu), "sha256_gpu": sha(hold["y"])},
                        "cpu_baseline": {"value": round(flop / dt / 1e9, 2), "unit": "GFLOP/s", "cores": oracle.threads(),
                                         "kind": "port", "sample": "the full layer"}})
                del x_d, w_d, go_d

        if want("linear"):
            # the other Linear shapes of the metric's GEMM configuration: grad-input (NN, tall K) and
            # grad-weight (TN, the batch dimension as K); parity on a slab of output rows
            for (M, N, K, tA, what) in ((4096, 4096, 32768, 0, "NN, Linear grad-input shape"),
                                         (4096, 4096, 65536, 1, "TN, Linear grad-weight shape (batch as K)")):
                g = torch.Generator().manual_seed(11 + tA)
                a_h = torch.randn((K, M) if tA else (M, K), generator=g)
                b_h = (torch.rand(K, N, generator=g) * 2 - 1) * (1.0 / (K ** 0.5)) if not tA else torch.randn(K, N, generator=g)
                a_d, b_d = a_h.to(dev), b_h.to(dev)
                hold = {}
                def f(): hold["y"] = ops.mm(a_d, b_d, bool(tA), False)
                wall, ev_mean, ev_min = time_gpu(f, max(2, args.steps // 2), 1, SETTLE_MS)
                rows = 64
                slab = a_h[:, :rows].contiguous() if tA else a_h[:rows]
                dt, y_slab = cpu_time(lambda: (refmods[0].mm(slab, b_h, bool(tA), False) if refmods else oracle.mm(slab, b_h, bool(tA), False)))
                flop = 2.0 * M * N * K
                tf = flop / (ev_mean * 1e-3) / 1e12
                result["also"].append({
                    "op": "mm", "workload": "%dx%dx%d %s" % (M, N, K, what), "value": round(tf * 1e3, 1), "unit": "GFLOP/s",
                    "ms_per_step": round(ev_mean, 4),
                    "roofline": {"bound": "mfma", "achieved": round(tf, 3), "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                                 "frac": round(tf / FP32_PEAK_TFLOPS, 4), "traffic": None},
                    "parity": {"equal": torch.equal(y_slab, hold["y"][:rows].cpu()), "rows_checked": rows, "sha256_gpu": sha(hold["y"])},
                    "cpu_baseline": {"value": round(2.0 * rows * N * K / dt / 1e9, 2), "unit": "GFLOP/s", "cores": oracle.threads(),
                                     "kind": kind, "sample": "first %d of %d output rows" % (rows, M)}})
                del a_d, b_d, a_h, b_h, hold

        if want("adam"):
            import ctypes
            import math

            na = 1 << 26
            g = torch.Generator().manual_seed(7)
            p_h, g_h = torch.randn(na, generator=g) * 0.05, torch.randn(na, generator=g) * torch.exp2(torch.rand(na, generator=g) * 20 - 20)
            m_h, v_h = torch.randn(na, generator=g) * 1e-3, torch.rand(na, generator=g) * 1e-5
            lr, betas, eps, wd, t = 1e-3, (0.9, 0.999), 1e-8, 1e-2, 10
            dev_t = [x.to(dev) for x in (p_h, g_h, m_h, v_h)]
            desc = (_lib.AdamTensor * 1)(_lib.AdamTensor(dev_t[0].data_ptr(), dev_t[1].data_ptr(), dev_t[2].data_ptr(),
                                                         dev_t[3].data_ptr(), None, na, math.sqrt(1 - betas[1] ** t),
                                                         -(lr / (1 - betas[0] ** t))))
            stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
            def f(): _lib.call("repdl_hip_adam_step", desc, 1, betas[0], 1 - betas[0], betas[1], 1 - betas[1], eps, wd, stream)
            f()  # one step on both sides, compared before the timed steps run on
            dt, _ = cpu_time(lambda: oracle.adam_step(p_h, g_h, m_h, v_h, None, t, lr, betas, eps, wd))
            par = {"equal": all(sha(a) == sha(b) for a, b in zip(dev_t, (p_h, g_h, m_h, v_h))), "sha256_gpu": sha(dev_t[0])}
            cpu = {"value": round(28.0 * na / dt / 1e9, 3), "unit": "GB/s", "cores": oracle.threads(), "kind": "port",
                   "sample": "the full 2^26 elements, one step"}
            result["also"].append(hbm_entry("adam_step", "one fused Adam step (weight decay on) over 2^26 parameters",
                                            28.0 * na, f, args.steps, args.warmup, par, cpu,
                                            round(MEASURED_TRAFFIC_BYTES["adam_step"])))
            del dev_t

    if args.copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 0.0, out=dst)  # an elementwise kernel: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
