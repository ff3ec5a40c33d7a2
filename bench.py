#!/usr/bin/env python3
"""Benchmark of the reproducible-operator hot path on one MI355X.

Headline (BASELINE.json `metric`): bit-exact fp32 `mm` GFLOP/s at 8192^3 -- the
`repdl.nn.Linear` forward shape x[8192,8192] . W[8192,8192]^T (transB).  A "step"
is one such product with the operands resident in HBM.  The same JSON line also
carries, under "also", every other operator of the metric's configurations (the
1024^3 product, the same 8192^3 product on the v_fma_f32 kernels, the sequential
sums, exp/log/sqrt/div on 2^28 values, softmax / cross_entropy, the convolution
layers, the other Linear shapes, a fused Adam step and the end-to-end CNN step),
each with its own roofline entry, its parity against the CPU checker on the same
input bytes, and the reference's CPU implementation timed beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick] [--only mm1024,sum1d,...]

Three more modes turn rocprofv3 output of a bench run into the summaries kept under
profiles/ (they need no GPU):

    python bench.py --summarise-trace DIR [--steps K]    per-kernel durations; for each kernel also
                                                         the mean of its LAST K dispatches (the timed ones)
    python bench.py --summarise-counters DIR [DIR ...]   per-kernel means of whatever --pmc counters DIR holds
    python bench.py --write-traffic FETCH_DIR WRITE_DIR  profiles/hbm_traffic.json: HBM bytes per call of each
                                                         leg, from FETCH_SIZE / WRITE_SIZE runs with --copy-probe

The CPU baseline is RepDL's own CPU implementation wherever it has one: its C++ backend
compiled into oracle/_ref from the reference sources (kind "reference"), and for sqrt / div
the two PyTorch-CPU expressions that *are* RepDL's definition of those operators
(repdl/ops.py:98-103, 122-123).  Where oracle/_ref is absent the plain-C restatement stands in
(kind "port").  Only the baseline and parity legs touch oracle/.
"""
from __future__ import annotations

import argparse
import csv
import glob
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_PEAK_TFLOPS = 157.3  # MI355X vendor fp32 figure (256 CU x 2.4 GHz x 256 flop/clk)
HBM_PEAK_GBS = 8000.0
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "hbm_traffic.json")

# Which kernels make up a call of each leg (substrings of the kernel names rocprofv3 reports), for
# --write-traffic.  The LAST entry is the kernel that ends a call.  Several legs may share kernels
# (the sequential sums do): "grid" then names the launch size, in threads, of the leg's first kernel
# at the bench's workload.  "split": the bench runs that many workloads through these kernels one
# after the other, an equal number of calls each; they get a traffic entry each, in that order.
_S1 = ["sum1d_blocksum_kernel", "sum1d_prefix_kernel", "sum1d_tuple_kernel", "sum1d_super_kernel", "sum1d_plan_kernel",
       "sum1d_cand_walk_kernel", "sum1d_compose_kernel", "sum1d_compose2_kernel", "sum1d_resolve_kernel", "sum1d_walk_kernel"]
LEG_KERNELS = {
    "mm": {"kernels": ["mm_dma_kernel<false, true, 4, 2, 2, 4, 4"]},
    "mm_fma": {"kernels": ["mm_kernel<false, true"]},
    "mm1024": {"kernels": ["mm_dma_kernel<false, false, 1, 2, 4, 2, 16, 1, 3"]},
    "sum2d_dim1": {"kernels": ["rowchain_kernel<32, 128, true, false>"]},
    "sum2d_dim0": {"kernels": ["coltile_kernel<16, true, 2>"]},
    "sum4d_dim023": {"kernels": _S1, "grid": 49 * 256 * 64},
    "sum1d": {"kernels": _S1, "grid": 65536 * 256, "split": ["sum1d", "sum1d_drift"]},
    "exp": {"kernels": ["unary_kernel<0>"]},
    "log": {"kernels": ["unary_kernel<1>"]},
    "sqrt": {"kernels": ["unary_kernel<2>"]},
    "div_scalar": {"kernels": ["unary_kernel<3>"]},
    "div": {"kernels": ["div_kernel"]},
    "softmax": {"kernels": ["rows_onchip_kernel<8, 32, true>"]},
    "cross_entropy": {"kernels": ["rows_onchip_kernel<8, 32, false>"]},
    "conv3x3_fwd": {"kernels": ["conv_tapdma_prep_kernel", "conv_tapdma_kernel<0,"]},
    "conv3x3_dgrad": {"kernels": ["conv_tapdma_prep_kernel", "conv_tapdma_kernel<1,"]},
    "conv3x3_wgrad": {"kernels": ["conv_wgrad_mfma_kernel<14, 1, 8, 32, false>"]},
    "conv1x1_fwd": {"kernels": ["mm_dma_kernel<false, false, 2, 2, 2, 2, 4"]},
    "conv1x1_dgrad": {"kernels": ["conv_point_kernel<1>"]},
    "conv1x1_wgrad": {"kernels": ["conv_wgrad_mfma_kernel<14, 1, 8, 16, true>"]},
    "adam_step": {"kernels": ["adam_kernel"]},
}


def sha(t) -> str:
    return hashlib.sha256(t.detach().cpu().contiguous().numpy().tobytes()).hexdigest()


# ----------------------------------------------------------------------------------------------
# rocprofv3 summaries (no GPU needed)
# ----------------------------------------------------------------------------------------------
def _short(name: str) -> str:
    return name.replace("(anonymous namespace)::", "").replace("void ", "")


def _find(dirname: str, pattern: str) -> str:
    hits = sorted(glob.glob(os.path.join(dirname, "**", pattern), recursive=True))
    if not hits:
        raise SystemExit("no %s under %s" % (pattern, dirname))
    return hits[0]


def summarise_trace(dirname: str, last: int) -> None:
    rows = list(csv.DictReader(open(_find(dirname, "*kernel_trace.csv"))))
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    per = {}
    for r in rows:
        per.setdefault(_short(r["Kernel_Name"]), []).append(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]))
    total = sum(sum(v) for v in per.values())
    print("%-100s %7s %14s %12s %12s %7s" % ("kernel", "calls", "total_ns", "avg_ns", "avg_last%d" % last, "share%"))
    for name, v in sorted(per.items(), key=lambda kv: -sum(kv[1])):
        tail = v[-last:]
        print("%-100s %7d %14d %12.0f %12.0f %7.3f" % (name[:100], len(v), sum(v), sum(v) / len(v), sum(tail) / len(tail),
                                                      100.0 * sum(v) / total))


def _counter_means(dirname: str):
    agg = {}
    for row in csv.DictReader(open(_find(dirname, "*counter_collection.csv"))):
        agg.setdefault((_short(row["Kernel_Name"]), row["Counter_Name"]), []).append(float(row["Counter_Value"]))
    return agg


def summarise_counters(dirnames) -> None:
    print("%-100s %-30s %7s %18s" % ("kernel", "counter", "calls", "mean per dispatch"))
    for d in dirnames:
        for (k, c), v in sorted(_counter_means(d).items()):
            print("%-100s %-30s %7d %18.1f" % (k[:100], c, len(v), sum(v) / len(v)))


def _leg_calls(dirname: str, counter: str, spec):
    """The counter summed over each call of a leg: the leg's dispatches in launch order, cut after
    every dispatch of the leg's last kernel; only calls whose first kernel has the leg's launch size
    (the one seen most often, if the leg names none: the bench's own workload makes most of the calls)."""
    subs, end = spec["kernels"], spec["kernels"][-1]
    rows = [r for r in csv.DictReader(open(_find(dirname, "*counter_collection.csv")))
            if r["Counter_Name"] == counter and any(x in _short(r["Kernel_Name"]) for x in subs)]
    rows.sort(key=lambda r: int(r["Dispatch_Id"]))
    calls, cur = [], []
    for r in rows:
        cur.append(r)
        if end in _short(r["Kernel_Name"]):
            calls.append(cur)
            cur = []
    if not calls:
        return []
    first_grid = lambda c: max(int(r["Grid_Size"]) for r in c if subs[0] in _short(r["Kernel_Name"])) if any(subs[0] in _short(r["Kernel_Name"]) for r in c) else 0
    grids = [first_grid(c) for c in calls]
    grid = spec.get("grid") or max(set(grids), key=grids.count)
    return [sum(float(r["Counter_Value"]) for r in c) for c in calls if first_grid(c) == grid]


def _median(v):
    v = sorted(v)
    return v[len(v) // 2]


def write_traffic(fetch_dir: str, write_dir: str) -> None:
    """FETCH_SIZE / WRITE_SIZE count in device-specific units: both are scaled by what the same counter
    reads for the --copy-probe kernel, which reads exactly 1 GiB and writes exactly 1 GiB per dispatch.
    Per leg: the median over its calls (a call of a leg that shares a set-up kernel with the leg before
    it can pick up that leg's last set-up launches)."""
    probe = {"kernels": ["trunc"]}
    pf, pw = _leg_calls(fetch_dir, "FETCH_SIZE", probe), _leg_calls(write_dir, "WRITE_SIZE", probe)
    if not pf or not pw:
        raise SystemExit("the copy-probe kernel is missing from the counter runs (run bench.py with --copy-probe)")
    f_unit, w_unit = float(1 << 30) / _median(pf), float(1 << 30) / _median(pw)
    legs, detail = {}, {}
    for leg, spec in LEG_KERNELS.items():
        rd, wr = _leg_calls(fetch_dir, "FETCH_SIZE", spec), _leg_calls(write_dir, "WRITE_SIZE", spec)
        if not rd or not wr:
            continue
        names = spec.get("split", [leg])
        for i, name in enumerate(names):
            part = lambda v: v[len(v) * i // len(names):len(v) * (i + 1) // len(names)]
            r, w = _median(part(rd)) * f_unit, _median(part(wr)) * w_unit
            legs[name] = round(r + w)
            detail[name] = {"read_bytes_per_call": round(r), "written_bytes_per_call": round(w), "calls_profiled": len(part(rd))}
    out = {"source": "rocprofv3 --pmc FETCH_SIZE / --pmc WRITE_SIZE over `bench.py --copy-probe`, one run per counter",
           "calibration": {"fetch_bytes_per_count": f_unit, "write_bytes_per_count": w_unit,
                           "probe": "torch.trunc(x, out=y) on 2^28 floats: 1 GiB read, 1 GiB written per dispatch"},
           "bytes_per_call": legs, "detail": detail}
    with open(TRAFFIC_JSON, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps(legs))


def measured_traffic(leg: str, default_size: bool = True):
    """HBM bytes per call of a leg from profiles/hbm_traffic.json, or (None, why)."""
    if not default_size:
        return None, "the traffic figures were measured at the default sizes only"
    if not os.path.exists(TRAFFIC_JSON):
        return None, "profiles/hbm_traffic.json is absent"
    with open(TRAFFIC_JSON) as f:
        legs = json.load(f).get("bytes_per_call", {})
    if leg not in legs:
        return None, "no FETCH_SIZE / WRITE_SIZE run covers this leg's kernels"
    return legs[leg], None


# ----------------------------------------------------------------------------------------------
# timing
# ----------------------------------------------------------------------------------------------
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


def cpu_time(fn, reps=1):
    best = None
    for _ in range(reps):
        t0 = time.perf_counter()
        r = fn()
        dt = time.perf_counter() - t0
        best = dt if best is None or dt < best else best
    return best, r


# Legs that a sequential chain keeps off the throughput roofline: the order of the additions (or of the
# multiply-adds) of one output is fixed, so a launch cannot be shorter than its longest chain at the
# latency of a dependent instruction (about 10 clocks for v_add_f32 in a lone wave, 35 for a dependent
# v_mfma_f32_16x16x4_f32 = 8.75 per k), whatever the bandwidth.
CHAIN_LIMITS = {
    "sum2d_dim0": "one workgroup per CU (256 groups of 16 columns, 65536 rows each), whose tile rows are half cache lines: a CU "
                  "brings in 16 GB/s of those whatever is in flight or walked (0.262 ms even with the walk switched off); the chains "
                  "themselves, 65536 dependent additions at 6.7 clocks, would take 0.18 ms",
    "sum4d_dim023": "chain latency: 64 chains of 200704 additions (0.85 ms if every addition were made one after the other; the "
                    "interval maps of the parallel evaluation skip about half of them)",
    "sum1d": "one chain of 2^28 additions (1.1 s at 10 clocks each): evaluated exactly in parallel by interval maps over candidate "
             "states, three passes over the input and about nine rounds of speculative walks",
    "sum1d_drift": "one chain of 2^28 additions: as above, fewer rounds because the sum's magnitude only grows",
    "conv3x3_wgrad": "chain latency: every output is a chain of 200704 multiply-adds; 50176 dependent 16x16x4 matrix instructions "
                     "at 35 clocks = 0.75-0.80 ms (measured with everything but the chain switched off: 0.80 ms)",
    "conv1x1_wgrad": "chain latency: as the 3x3 layer, 200704-term chains on 64 blocks of 16x16 outputs (floor 0.80 ms)",
    "softmax": "vector ALU: the correctly rounded exp (about 30 instructions per element) and the division, plus a 1000-term chain per row",
    "cross_entropy": "vector ALU: the correctly rounded exp (about 30 instructions per element), plus a 1000-term chain per row",
}


def leg_entry(name, workload, bound, work, fn, steps, warmup, parity, cpu, traffic_leg=None, default_size=True, short=None):
    """One "also" entry: `work` is the algorithmic bytes (bound "hbm") or flop (bound "mfma") of one call.
    `short`: the workload's label in the printed line (`workload` itself goes to the detail file)."""
    wall, ev_mean, ev_min = time_gpu(fn, steps, warmup, SETTLE_MS)
    if bound == "hbm":
        rate, unit, peak = work / (ev_mean * 1e-3) / 1e9, "GB/s", HBM_PEAK_GBS
        value, vunit = rate, "GB/s"
    else:
        rate, unit, peak = work / (ev_mean * 1e-3) / 1e12, "TFLOP/s", FP32_PEAK_TFLOPS
        value, vunit = rate * 1e3, "GFLOP/s"
    traffic, why = measured_traffic(traffic_leg, default_size) if traffic_leg else (None, "no FETCH_SIZE / WRITE_SIZE run covers this leg's kernels")
    roof = {"bound": bound, "achieved": round(rate, 3), "peak": peak, "unit": unit, "frac": round(rate / peak, 4), "traffic": traffic}
    if traffic is None:
        roof["traffic_note"] = why
    limit = CHAIN_LIMITS.get(traffic_leg)
    if limit is not None and default_size:
        roof["limited_by"] = limit  # what keeps this leg off the roofline named in "bound"
    out = {"op": name, "workload": workload, "short": short or workload, "value": round(value, 2), "unit": vunit,
           "ms_per_step": round(ev_mean, 4), "ms_min": round(ev_min, 4), "roofline": roof}
    if parity is not None:
        out["parity"] = parity
    if cpu is not None:
        out["cpu_baseline"] = cpu
    return out


LINE_LIMIT = 7000  # bytes of the printed line: harnesses that keep only the tail of stdout must still see every leg
DETAIL_JSON = os.environ.get("REPDL_BENCH_DETAIL", "bench_detail.json")  # every leg in full (digests, notes), beside the printed line
# per bound of a secondary leg: unit and peak of its `roofline.achieved`, unit of its `cpu_baseline.value` (unless the leg names another)
ALSO_UNITS = {"hbm": {"unit": "GB/s", "peak": HBM_PEAK_GBS, "cpu_unit": "GB/s"},
              "mfma": {"unit": "TFLOP/s", "peak": FP32_PEAK_TFLOPS, "cpu_unit": "GFLOP/s"}}


def compact_leg(e, cores=None):
    """A secondary leg as it is printed: numbers and short labels only.  `roofline.unit` / `roofline.peak` are those of
    its bound (top-level "also_units"), `cpu_baseline.cores` is "also_units.cpu_cores" unless the leg states another;
    digests, notes and what limits a leg go to the detail file."""
    r = e["roofline"]
    sig4 = lambda x: x if x is None else float("%.4g" % x)
    out = {"op": e["op"], "wl": e["short"], "ms": e["ms_per_step"],
           "roofline": {"bound": r["bound"], "achieved": sig4(r["achieved"]), "frac": r["frac"], "traffic": r["traffic"]}}
    if "parity" in e:
        out["equal"] = e["parity"].get("equal")
    c = e.get("cpu_baseline")
    if c is not None:
        out["cpu_baseline"] = {"value": sig4(c["value"]), "kind": c["kind"], "sample": c["short"]}
        if c["cores"] != cores:
            out["cpu_baseline"]["cores"] = c["cores"]
        if c["unit"] != ALSO_UNITS[r["bound"]]["cpu_unit"]:
            out["cpu_baseline"]["unit"] = c["unit"]
    return out


def compact_line(result) -> str:
    """The one printed line: the headline in full, the secondary legs compacted."""
    out = {k: v for k, v in result.items() if k != "also"}
    cores = result["cpu_baseline"]["cores"]
    out["also_units"] = dict(ALSO_UNITS, cpu_cores=cores)
    out["also"] = [compact_leg(e, cores) for e in result["also"]]
    return json.dumps(out, separators=(",", ":"))


# ----------------------------------------------------------------------------------------------
def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=10)  # 77 ms of headline launches: the first tens of ms after idle are not steady state
    ap.add_argument("--quick", action="store_true", help="headline only, no secondary operators, no full parity")
    ap.add_argument("--only", default="", help="comma list of secondary legs to run (mm1024,mm64,mm_fma,sum2d,sum2d_dim0,sum4d,sum1d,"
                                               "exp,log,sqrt,div,loss,conv,linear,adam,cnn)")
    ap.add_argument("--size", type=int, default=8192, help="mm size (M=N=K); the metric is quoted at 8192")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 1 GiB elementwise kernel (torch.trunc(x, out=y)), the known-size kernel "
                         "against which FETCH_SIZE / WRITE_SIZE counters are calibrated")
    ap.add_argument("--summarise-trace", metavar="DIR")
    ap.add_argument("--summarise-counters", metavar="DIR", nargs="+")
    ap.add_argument("--write-traffic", metavar="DIR", nargs=2)
    args = ap.parse_args()
    if args.summarise_trace:
        summarise_trace(args.summarise_trace, args.steps)
        return 0
    if args.summarise_counters:
        summarise_counters(args.summarise_counters)
        return 0
    if args.write_traffic:
        write_traffic(*args.write_traffic)
        return 0
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

    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import gen  # deterministic generators shared with the parity tests

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(dev)
    S = args.size
    only = set(x for x in args.only.split(",") if x)
    want = lambda k: (not only) or (k in only)
    refmods = oracle_ref.load()
    kind = "reference" if refmods is not None else "port"
    cores = oracle.threads()

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
    sha_headline = sha(y_gpu)
    if not args.quick:
        t0 = time.perf_counter()
        y_cpu = oracle.mm(x_h, w_h, False, True)
        sha_cpu = sha(y_cpu)
        parity["mm"] = {"equal": sha_headline == sha_cpu, "sha256_gpu": sha_headline[:16], "sha256_cpu": sha_cpu[:16],
                        "checker": "oracle, whole output", "checker_s": round(time.perf_counter() - t0, 2)}
        del y_cpu

    # CPU baseline: the reference's own CPU backend on a row slab of the same product
    rows = 256 if not args.quick else 64
    rows = min(rows, S)
    if refmods is not None:
        cpu_fn = lambda: refmods[0].mm(x_h[:rows], w_h, False, True)
    else:
        cpu_fn = lambda: oracle.mm(x_h[:rows], w_h, False, True)
    dt, y_slab = cpu_time(cpu_fn)
    slab_equal = torch.equal(y_slab, y_gpu[:rows].cpu())
    cpu_baseline = {
        "value": round(2.0 * rows * S * S / dt / 1e9, 3), "unit": "GFLOP/s", "cores": cores, "kind": kind,
        "sample": "first %d of %d output rows of the same product (%.1f s); GPU rows bit-equal: %s" % (rows, S, dt, slab_equal),
    }
    del y_gpu, out_holder

    if _lib.lib().repdl_hip_matrix_path() == 1:
        kernel_name = "mm_dma_kernel<NT>"
        kernel_note = "v_mfma_f32_16x16x4_f32, checked on this device to be a k-ascending chain of single-rounding FMAs"
    else:
        kernel_name = "mm_kernel<NT>"
        kernel_note = "matrix-instruction check failed on this device: v_fma_f32 only, ceiling half of this peak"
    traffic, why = measured_traffic("mm", S == 8192)
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
        "data": "synthetic (seeded, same bytes for GPU and CPU checker)",
        "config": {"workload": "repdl.ops.mm fp32 %dx%dx%d transB (nn.Linear forward), configs[3]" % (S, S, S),
                   "device": props.name, "cus": props.multi_processor_count},
        "roofline": {"bound": "mfma", "achieved": round(kern_tflops, 3), "peak": FP32_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(kern_tflops / FP32_PEAK_TFLOPS, 4), "traffic": traffic,
                     "kernel": kernel_name, "kernel_ms": round(ev_ms, 4), "kernel_ms_min": round(ev_min, 4),
                     "note": kernel_note},
        "cpu_baseline": cpu_baseline,
        "parity": parity,
        "also": [],
    }
    if traffic is None:
        result["roofline"]["traffic_note"] = why
    also = result["also"]

    if not args.quick:
        n = 1 << 28

        if want("mm_fma"):
            # the same product on the v_fma_f32 kernels: explicit FMA chains along K, one per output
            _lib.call("repdl_hip_set_matrix_path", 0)
            hold = {}
            def f(): hold["y"] = ops.mm(x_d, w_d, transB=True)
            f()
            par = {"equal": sha(hold["y"]) == sha_headline, "against": "the matrix-instruction kernel's output (itself checked against the oracle)"}
            also.append(leg_entry("mm (v_fma_f32 kernels)", "the headline's %dx%dx%d NT product, matrix instructions off" % (S, S, S), "mfma", flop,
                                  f, max(2, args.steps // 2), 1, par, dict(cpu_baseline, short="as headline"), "mm_fma", S == 8192, short="%d^3 NT, matrix path off" % S))
            also[-1]["roofline"]["note"] = "v_fma_f32 only: the issue-rate ceiling of this path is 78.6 TFLOP/s, half the peak quoted"
            _lib.call("repdl_hip_set_matrix_path", -1)
            hold.clear()
        del x_d, w_d

        if want("mm1024"):
            g = torch.Generator().manual_seed(10)
            a_h, b_h = torch.randn(1024, 1024, generator=g), torch.randn(1024, 1024, generator=g)
            a_d, b_d = a_h.to(dev), b_h.to(dev)
            hold = {}
            def f(): hold["y"] = ops.mm(a_d, b_d)
            f()
            dt, y_cpu = cpu_time(lambda: (refmods[0].mm(a_h, b_h, False, False) if refmods else oracle.mm(a_h, b_h, False, False)))
            par = {"equal": sha(hold["y"]) == sha(y_cpu), "sha256_gpu": sha(hold["y"])}
            cpu = {"value": round(2.0 * 1024 ** 3 / dt / 1e9, 3), "unit": "GFLOP/s", "cores": cores, "kind": kind, "sample": "the full product", "short": "full"}
            also.append(leg_entry("mm", "1024x1024x1024 NN, N(0,1) entries (configs[0])", "mfma", 2.0 * 1024 ** 3, f, args.steps * 4, args.warmup, par, cpu, "mm1024",
                                  short="1024^3 NN cfg0"))
            del a_d, b_d

        if want("mm64"):
            # a Linear layer at batch 64: 64 output rows, every SIMD one chain of dependent matrix instructions
            g = torch.Generator().manual_seed(15)
            a_h = torch.randn(64, 4096, generator=g)
            b_h = (torch.rand(4096, 4096, generator=g) * 2 - 1) / 64.0
            a_d, b_d = a_h.to(dev), b_h.to(dev)
            hold = {}
            def f(): hold["y"] = ops.mm(a_d, b_d, False, True)
            f()
            dt, y_cpu = cpu_time(lambda: (refmods[0].mm(a_h, b_h, False, True) if refmods else oracle.mm(a_h, b_h, False, True)))
            par = {"equal": sha(hold["y"]) == sha(y_cpu), "sha256_gpu": sha(hold["y"])}
            cpu = {"value": round(2.0 * 64 * 4096 * 4096 / dt / 1e9, 3), "unit": "GFLOP/s", "cores": cores, "kind": kind, "sample": "the full product",
                   "short": "full"}
            also.append(leg_entry("mm", "64x4096x4096 NT (nn.Linear forward at batch 64)", "mfma", 2.0 * 64 * 4096 * 4096, f, args.steps * 4, args.warmup,
                                  par, cpu, short="64x4096x4096 NT"))
            del a_d, b_d

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
            cpu = {"value": round(2048 * R * 4 / dt / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": kind, "sample": "first 2048 rows", "short": "2048 rows"}
            also.append(leg_entry("sum2d_dim1", "row sums of 16384x16384 N(0,1)*2^U(-20,20)", "hbm", 4.0 * R * R + 4 * R, f, args.steps, args.warmup,
                                  par, cpu, "sum2d_dim1", short="16384^2 rows cfg1"))
            del m_d, m_h, hold

        if want("sum2d_dim0"):
            M, N = 65536, 4096  # grad-bias of the Linear configuration: grad_output [batch, out]
            g = torch.Generator().manual_seed(12)
            m_h = torch.randn(M, N, generator=g)
            m_d = m_h.to(dev)
            hold = {}
            def f(): hold["y"] = ops.sum2d_dim0(m_d)
            f()
            dt, y_cpu = cpu_time(lambda: (refmods[0].sum2d_dim0(m_h, False, False) if refmods else oracle.sum2d_dim0(m_h)))
            par = {"equal": sha(hold["y"]) == sha(y_cpu), "sha256_gpu": sha(hold["y"])}
            cpu = {"value": round(M * N * 4 / dt / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": kind, "sample": "the full matrix", "short": "full"}
            also.append(leg_entry("sum2d_dim0", "column sums of 65536x4096 N(0,1) (Linear grad-bias shape)", "hbm", 4.0 * M * N + 4 * N, f, args.steps,
                                  args.warmup, par, cpu, "sum2d_dim0", short="65536x4096 cols"))
            del m_d, m_h, hold

        if want("sum4d"):
            shape = (64, 64, 56, 56)  # grad-bias of the convolution configuration
            g = torch.Generator().manual_seed(13)
            t_h = torch.randn(*shape, generator=g)
            t_d = t_h.to(dev)
            hold = {}
            def f(): hold["y"] = ops.sum4d_dim023(t_d)
            f()
            dt, y_cpu = cpu_time(lambda: (refmods[0].sum4d_dim023(t_h, False, False) if refmods else oracle.sum4d_dim023(t_h)))
            par = {"equal": sha(hold["y"]) == sha(y_cpu), "sha256_gpu": sha(hold["y"])}
            cpu = {"value": round(t_h.numel() * 4 / dt / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": kind, "sample": "the full tensor", "short": "full"}
            also.append(leg_entry("sum4d_dim023", "channel sums of [64,64,56,56] N(0,1) (conv grad-bias shape)", "hbm", 4.0 * t_h.numel(), f,
                                  args.steps, args.warmup, par, cpu, "sum4d_dim023", short="[64,64,56,56]"))
            del t_d, t_h, hold

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
                   "sample": "the full 2^28 vector (the reference's sum1d is single-threaded)", "short": "full"}
            also.append(leg_entry("sum1d", "sequential sum of 2^28 uniform[-1,1)", "hbm", 4.0 * n, f, args.steps, args.warmup, par, cpu, "sum1d",
                                  short="2^28 U[-1,1) cfg1"))
            v_d.abs_()  # the drifting case: uniform[0,1), the sum stops growing at 2^24
            v_h.abs_()
            f()
            dt, y_cpu = cpu_time(lambda: (refmods[0].sum1d(v_h, False) if refmods else oracle.sum1d(v_h)))
            par = {"equal": sha(hold["y"]) == sha(y_cpu), "gpu": float(hold["y"]), "cpu": float(y_cpu)}
            cpu = {"value": round(n * 4 / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": kind, "sample": "the full 2^28 vector", "short": "full"}
            also.append(leg_entry("sum1d", "sequential sum of 2^28 uniform[0,1) (drifting)", "hbm", 4.0 * n, f, args.steps, args.warmup, par, cpu, "sum1d_drift",
                                  short="2^28 U[0,1) drift"))
            del v_d, v_h, hold

        ew = [k for k in ("exp", "log", "sqrt", "div") if want(k)]
        if ew:
            e_h = gen.elementwise_mix(3, n)  # config-3 mix: 90 % log-uniform, 10 % specials
            e_d = e_h.to(dev)
            ns = 1 << 24  # CPU baseline sample
            tth = torch.get_num_threads()
            for k in ew:
                hold = {}
                if k == "div":
                    e2_h = gen.elementwise_mix(4, n)
                    e2_d = e2_h.to(dev)
                    ten = torch.tensor(10.0)
                    legs = [("div_scalar", "x/10.0 on 2^28 mixed values", 8.0 * n, lambda: ops.div(e_d, 10.0), lambda: oracle.div(e_h, 10.0),
                             lambda: e_h[:ns].div(ten), "torch CPU x.div(tensor(10.)) -- RepDL's div is this expression (repdl/ops.py:98-103)", tth),
                            ("div", "x/y on 2^28 mixed values", 12.0 * n, lambda: ops.div(e_d, e2_d), lambda: oracle.div(e_h, e2_h),
                             lambda: e_h[:ns].div(e2_h[:ns]), "torch CPU x.div(y) -- RepDL's div is this expression (repdl/ops.py:98-103)", tth)]
                elif k == "sqrt":
                    legs = [("sqrt", "sqrt on 2^28 mixed values", 8.0 * n, lambda: ops.sqrt(e_d), lambda: oracle.sqrt(e_h),
                             lambda: e_h[:ns].to(torch.float64).sqrt().to(torch.float32),
                             "torch CPU x.double().sqrt().float() -- RepDL's sqrt is this expression (repdl/ops.py:122-123)", tth)]
                else:
                    if refmods is not None:
                        rfn = (lambda: refmods[1].exp2d(e_h[:ns].view(4096, 4096))) if k == "exp" else (lambda: refmods[1].log1d(e_h[:ns]))
                        rnote = "the reference's %s (backend/cpu/math.cpp)" % ("exp2d" if k == "exp" else "log1d")
                    else:
                        rfn, rnote = (lambda kk: (lambda: getattr(oracle, kk)(e_h[:ns])))(k), "oracle"
                    legs = [(k, "%s on 2^28 mixed values" % k, 8.0 * n, (lambda kk: (lambda: getattr(ops, kk)(e_d)))(k),
                             (lambda kk: (lambda: getattr(oracle, kk)(e_h)))(k), rfn, rnote, cores)]
                for name, wl, nbytes, gfn, ofn, rfn, rnote, rcores in legs:
                    def f(): hold["y"] = gfn()
                    f()
                    y_cpu = ofn()  # the whole 2^28 output against the checker
                    par = {"equal": sha(hold["y"]) == sha(y_cpu), "elements_checked": n}
                    dt, y_ref = cpu_time(rfn)
                    par["reference_sample_equal"] = torch.equal(y_ref.reshape(-1).view(torch.int32), y_cpu[:ns].view(torch.int32))
                    del y_cpu, y_ref
                    cpu = {"value": round(nbytes / n * ns / dt / 1e9, 3), "unit": "GB/s", "cores": rcores,
                           "kind": "reference" if (refmods is not None or k in ("sqrt", "div")) else "port", "sample": "first 2^24 elements; " + rnote,
                           "short": "2^24"}
                    also.append(leg_entry(name, wl, "hbm", nbytes, f, args.steps, args.warmup, par, cpu, name, short="2^28 mix cfg2"))
                    hold.clear()
            del e_d, e_h

        if want("loss"):
            M, N = 65536, 1000
            g = torch.Generator().manual_seed(14)
            z_h = torch.randn(M, N, generator=g) * 4
            t_h = torch.randint(0, N, (M,), generator=g, dtype=torch.int64)
            z_d, t_d = z_h.to(dev), t_h.to(dev)
            ms = 4096  # rows of the CPU baseline sample
            for name, gfn, ofn, rfn, nbytes in (
                    ("softmax", lambda: ops.softmax(z_d), lambda: oracle.softmax(z_h),
                     (lambda: refmods[0].softmax(z_h[:ms])) if refmods else (lambda: oracle.softmax(z_h[:ms])), 8.0 * M * N),
                    ("cross_entropy", lambda: ops.cross_entropy(z_d, t_d), lambda: oracle.cross_entropy(z_h, t_h),
                     (lambda: refmods[0].cross_entropy(z_h[:ms], t_h[:ms])) if refmods else (lambda: oracle.cross_entropy(z_h[:ms], t_h[:ms])),
                     4.0 * M * N + 8.0 * M)):
                hold = {}
                def f(): hold["y"] = gfn()
                f()
                y_cpu = ofn()
                par = {"equal": sha(hold["y"]) == sha(y_cpu), "sha256_gpu": sha(hold["y"])}
                dt, _ = cpu_time(rfn)
                cpu = {"value": round(nbytes / M * ms / dt / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": kind, "sample": "first %d rows" % ms,
                       "short": "%d rows" % ms}
                also.append(leg_entry(name, "%s of 65536x1000 logits N(0,16)" % name, "hbm", nbytes, f, args.steps, args.warmup, par, cpu,
                                      name, short="65536x1000"))
                del y_cpu
            del z_d, z_h

        if want("conv"):
            nb = 8  # images of the CPU baseline sample
            for (N, IC, H, W, OC, Kk, st, pd) in [(64, 64, 56, 56, 64, 3, 1, 1), (64, 256, 56, 56, 64, 1, 1, 0)]:
                g = torch.Generator().manual_seed(5 + Kk)
                x_h = torch.randn(N, IC, H, W, generator=g).clamp_(min=0)
                w_h = torch.randn(OC, IC, Kk, Kk, generator=g) * (2.0 / (IC * Kk * Kk)) ** 0.5  # Kaiming normal
                OH, OW = (H + 2 * pd - Kk) // st + 1, (W + 2 * pd - Kk) // st + 1
                go_h = torch.randn(N, OC, OH, OW, generator=g)
                x_d, w_d, go_d = x_h.to(dev), w_h.to(dev), go_h.to(dev)
                cflop = 2.0 * N * OC * OH * OW * IC * Kk * Kk
                xs, gs = x_h[:nb].contiguous(), go_h[:nb].contiguous()
                R = refmods[0] if refmods else None
                legs = [
                    ("conv2d", lambda: ops.conv2d(x_d, w_d, (st, st), (pd, pd), 1),
                     lambda: oracle.conv2d(x_h, w_h, st, st, pd, pd, 1),
                     (lambda: R.conv2d(xs, w_h, st, st, pd, pd, 1)) if R else (lambda: oracle.conv2d(xs, w_h, st, st, pd, pd, 1))),
                    ("conv2d_grad_input", lambda: ops.conv2d_grad_input(x_h.shape, w_d, go_d, (st, st), (pd, pd)),
                     lambda: oracle.conv2d_grad_input(go_h, w_h, H, W, st, st, pd, pd),
                     (lambda: R.conv2d_grad_input(gs, w_h, H, W, st, st, pd, pd)) if R else (lambda: oracle.conv2d_grad_input(gs, w_h, H, W, st, st, pd, pd))),
                    ("conv2d_grad_kernel", lambda: ops.conv2d_grad_kernel(x_d, w_h.shape, go_d, (st, st), (pd, pd)),
                     lambda: oracle.conv2d_grad_kernel(go_h, x_h, Kk, Kk, st, st, pd, pd),
                     (lambda: R.conv2d_grad_kernel(gs, xs, Kk, Kk, st, st, pd, pd)) if R else (lambda: oracle.conv2d_grad_kernel(gs, xs, Kk, Kk, st, st, pd, pd))),
                ]
                for name, gfn, ofn, rfn in legs:
                    hold = {}
                    def f(): hold["y"] = gfn()
                    f()
                    y_cpu = ofn()
                    par = {"equal": sha(hold["y"]) == sha(y_cpu), "sha256_gpu": sha(hold["y"])}
                    dt, _ = cpu_time(rfn)
                    cpu = {"value": round(cflop * nb / N / dt / 1e9, 2), "unit": "GFLOP/s", "cores": cores, "kind": kind,
                           "sample": "the first %d of %d images (for grad-kernel: chains %d times shorter)" % (nb, N, N // nb),
                           "short": "%d/%d img" % (nb, N)}
                    tleg = "conv%dx%d_%s" % (Kk, Kk, {"conv2d": "fwd", "conv2d_grad_input": "dgrad", "conv2d_grad_kernel": "wgrad"}[name])
                    also.append(leg_entry(name, "batch %d, %dx%d conv %d->%d at %dx%d" % (N, Kk, Kk, IC, OC, H, W), "mfma", cflop, f, args.steps,
                                          args.warmup, par, cpu, tleg, short="b%d %dx%d %d>%d @%d cfg4" % (N, Kk, Kk, IC, OC, H)))
                    del y_cpu
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
                f()
                rws = 64
                slab = a_h[:, :rws].contiguous() if tA else a_h[:rws]
                dt, y_slab = cpu_time(lambda: (refmods[0].mm(slab, b_h, bool(tA), False) if refmods else oracle.mm(slab, b_h, bool(tA), False)))
                par = {"equal": torch.equal(y_slab, hold["y"][:rws].cpu()), "rows_checked": rws, "sha256_gpu": sha(hold["y"])}
                cpu = {"value": round(2.0 * rws * N * K / dt / 1e9, 2), "unit": "GFLOP/s", "cores": cores, "kind": kind,
                       "sample": "first %d of %d output rows" % (rws, M), "short": "%d rows" % rws}
                also.append(leg_entry("mm", "%dx%dx%d %s" % (M, N, K, what), "mfma", 2.0 * M * N * K, f, max(2, args.steps // 2), 1, par, cpu,
                                      short="4096^2xK%d %s cfg3" % (K, "TN" if tA else "NN")))
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

            def reference_adam_step(p, grad, m, v):
                """repdl/optim.py:64-83 on CPU tensors, ops.sqrt / ops.div as their CPU branches (repdl/ops.py:98-103, 122-123)."""
                bc1, bc2 = 1 - betas[0] ** t, 1 - betas[1] ** t
                grad = grad.add(p, alpha=wd)
                m.mul_(betas[0]).add_(grad, alpha=1 - betas[0])
                v.mul_(betas[1]).add_(torch.mul(grad, grad).mul(1 - betas[1]))
                denom = v.to(dtype=torch.float64).sqrt().to(dtype=torch.float32).div(math.sqrt(bc2)).add_(eps)
                p.add_(torch.div(m, denom).mul(-(lr / bc1)))

            ref_t = [x.clone() for x in (p_h, g_h, m_h, v_h)]
            dt, _ = cpu_time(lambda: reference_adam_step(*ref_t))
            oracle.adam_step(p_h, g_h, m_h, v_h, None, t, lr, betas, eps, wd)
            par = {"equal": all(sha(a) == sha(b) for a, b in zip(dev_t, (p_h, g_h, m_h, v_h))), "sha256_gpu": sha(dev_t[0]),
                   "reference_equal": all(sha(a) == sha(b) for a, b in zip(dev_t, ref_t))}
            cpu = {"value": round(28.0 * na / dt / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "reference",
                   "sample": "the full 2^26 elements, one step of the reference's own sequence of PyTorch CPU tensor operations (repdl/optim.py:64-83)",
                   "short": "full"}
            also.append(leg_entry("adam_step", "one fused Adam step (weight decay on) over 2^26 parameters", "hbm", 28.0 * na, f, args.steps, args.warmup,
                                  par, cpu, "adam_step", short="2^26 params"))
            del ref_t
            del dev_t

        if want("cnn"):
            # configs[4], end to end: from_torch_module on a 2-conv + 2-FC CNN, batch 64 of 1x28x28 uniform[0,1) images,
            # 10 random classes, three SGD steps at lr 0.01; the same glue runs on CPU tensors with the oracle behind it
            import models
            from oracle_ops import oracle_for_cpu_tensors

            xi, yi = models.images(21, 64), gen.labels(22, 64, 10)
            hashes = {}
            with oracle_for_cpu_tensors():
                for where in ("cpu", "cuda"):
                    m = repdl_amd.from_torch_module(models.cnn(0)).to(where)
                    opt = repdl_amd.optim.SGD(m.parameters(), 0.01)
                    logits, _ = models.train_steps(m, repdl_amd.nn.CrossEntropyLoss(), opt, xi.to(where), yi.to(where), 3)
                    hashes[where] = (repdl_amd.utils.get_hash(m), repdl_amd.utils.get_hash(logits))
            m = repdl_amd.from_torch_module(models.cnn(0)).to(dev)
            opt = repdl_amd.optim.SGD(m.parameters(), 0.01)
            lossf, xd, yd = repdl_amd.nn.CrossEntropyLoss(), xi.to(dev), yi.to(dev)

            def f():
                opt.zero_grad()
                lossf(m(xd), yd).backward()
                opt.step()

            wall, ev_mean, ev_min = time_gpu(f, args.steps, args.warmup, SETTLE_MS)
            with oracle_for_cpu_tensors():
                mc = repdl_amd.from_torch_module(models.cnn(0))
                optc = repdl_amd.optim.SGD(mc.parameters(), 0.01)
                def fc():
                    optc.zero_grad()
                    lossf(mc(xi), yi).backward()
                    optc.step()
                dt, _ = cpu_time(fc, 3)
            also.append({"op": "cnn_step", "workload": "2-conv + 2-FC CNN via from_torch_module, batch 64 of 1x28x28, SGD lr 0.01 (forward, backward, update)",
                         "short": "b64 1x28x28 SGD cfg4",
                         "value": round(1e3 / wall, 1), "unit": "steps/s", "ms_per_step": round(wall, 4),
                         "roofline": {"bound": "hbm", "achieved": None, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": None, "traffic": None,
                                      "traffic_note": "a chain of ~60 small launches: bound by launch latency, not by a roofline"},
                         "parity": {"equal": hashes["cpu"] == hashes["cuda"], "sha256_weights_after_3_steps": hashes["cuda"][0],
                                    "sha256_logits_after_3_steps": hashes["cuda"][1]},
                         "cpu_baseline": {"value": round(1.0 / dt, 2), "unit": "steps/s", "cores": cores, "kind": "port",
                                          "sample": "the same step through the same glue with the oracle's operators on CPU tensors",
                                          "short": "same glue on oracle"}})

            # the same step captured into one graph (forward, loss, backward with its side streams, the fused
            # update) and replayed: what a launch-bound loop costs without its launches
            mg = repdl_amd.from_torch_module(models.cnn(0)).to(dev)
            optg = repdl_amd.optim.SGD(mg.parameters(), 0.01)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):  # (eager steps first: the first ones create optimizer state and streams)
                    optg.zero_grad(set_to_none=True)
                    lossf(mg(xd), yd).backward()
                    optg.step()
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            optg.zero_grad(set_to_none=True)
            with torch.cuda.graph(graph):
                lossf(mg(xd), yd).backward()
                optg.step()
            replays = 0

            def fg():
                nonlocal replays
                graph.replay()
                replays += 1

            wallg, _, _ = time_gpu(fg, args.steps, args.warmup, SETTLE_MS)
            torch.cuda.synchronize()
            me = repdl_amd.from_torch_module(models.cnn(0)).to(dev)  # the same number of eager steps
            opte = repdl_amd.optim.SGD(me.parameters(), 0.01)
            for _ in range(3 + replays):
                opte.zero_grad(set_to_none=True)
                lossf(me(xd), yd).backward()
                opte.step()
            also.append({"op": "cnn_step_graph", "workload": "the same training step captured into one graph and replayed",
                         "short": "one graph replay",
                         "value": round(1e3 / wallg, 1), "unit": "steps/s", "ms_per_step": round(wallg, 4),
                         "roofline": {"bound": "hbm", "achieved": None, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": None, "traffic": None,
                                      "traffic_note": "the launches of cnn_step as one graph launch"},
                         "parity": {"equal": repdl_amd.utils.get_hash(mg) == repdl_amd.utils.get_hash(me), "replays": replays,
                                    "sha256_weights": repdl_amd.utils.get_hash(mg)},
                         "cpu_baseline": dict(also[-1]["cpu_baseline"], short="as cnn_step")})

    if args.copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.trunc(src, out=dst)  # an elementwise kernel no leg uses: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()

    try:
        if os.path.dirname(DETAIL_JSON):
            os.makedirs(os.path.dirname(DETAIL_JSON), exist_ok=True)
        with open(DETAIL_JSON, "w") as f:
            json.dump(result, f, indent=1)
            f.write("\n")
    except OSError as err:  # (a read-only tree: the printed line is what counts)
        print("bench.py: detail file not written: %s" % err, file=sys.stderr)
    line = compact_line(result)
    if len(line) > LINE_LIMIT:
        print("bench.py: the printed line has %d bytes, more than %d" % (len(line), LINE_LIMIT), file=sys.stderr)
    print(line)
    return 0


if __name__ == "__main__":
    sys.exit(main())
