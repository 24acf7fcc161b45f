#!/usr/bin/env python3
"""Benchmark of the builtin-operation kernels on one MI355X.

One "step" is one pass of the elementwise bandwidth sweep: fadd, fmul,
fdivide, fsigmoid, fcopy and ffill(3.0), each as a single kernel over fp32
tensors of 2^26 elements that are already resident in HBM.  `value` is the
algorithmic bytes of the whole sweep divided by the wall time of the timed
steps.  After the timed region the same run measures ftranspose 12345x6789,
the 4096^3 fp32 matmul in all four transpose variants, and the CPU oracle on
the host cores (a reported baseline only).

Per-kernel durations come from HIP events attached to every launch on the
library's own stream (each pair takes the kernel's own begin and end
timestamps), so they are comparable with a profiler's kernel durations;
launches are issued back to back, the way a graph of such operations issues
them, and every kernel outside the headline sweep cycles through several sets
of buffers so that no launch is served from a cache the previous one filled.
`value` and `ms_per_step` use the host wall clock around the timed region and
therefore include launch gaps.

Prints ONE JSON line on stdout; progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_FP32_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix, published

N_SWEEP = 1 << 26
# algorithmic bytes per element (reads + writes, fp32, scalars free)
BYTES_PER_ELEMENT = {"fadd": 12, "fmul": 12, "fdivide": 12, "fsigmoid": 8,
                     "fcopy": 8, "ffill": 4, "flogloss": 12, "fmulconcat": 8,
                     "ftranspose": 8}
SWEEP = ["fadd", "fmul", "fdivide", "fsigmoid", "fcopy", "ffill"]
# HBM-side bytes per launch at the sizes below come from two `rocprofv3 --pmc`
# runs of this script (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch), each
# scaled by what the same counter reads for the plain copy kernel fcopy.  They
# cannot be measured from inside this process, so they are read from the table
# that summarises those runs; an operation whose kernels the table does not
# hold reports null.
LIB_PROBES = os.path.join(ROOT, "bench_probes", "libpolar_hip_probes.so")  # built by bench_probes/Makefile
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "bench_kernels_pmc_traffic.md")
TRAFFIC_KERNELS = {  # operation -> name fragments of the kernels one call launches
    "fadd": ["<AddOp,"], "fmul": ["<MulOp,"], "fdivide": ["<DivOp,"], "fsigmoid": ["<SigmoidOp,"],
    "fcopy": ["<CopyOp,"], "ffill": ["<FillOp,"], "flogloss": ["<LogLossOp,"], "fmulconcat": ["<ScaleOp,"],
    "frelu": ["<ReluOp,"], "fsoftmax": ["expSumKernel", "finishSumKernel", "<SoftmaxScaleOp,"],
    "ftranspose": ["transpose"], "fmatmul": ["matmulKernel<"], "fconv2d": ["conv2d"], "fpool": ["poolSquareKernel"],
    "fpool_3x3_stride2": ["poolStagedKernel<3,3,true> stride 2"], "fpool_3x3_stride1": ["poolStagedKernel<3,3,true> stride 1"],
    "fpool_5x5_stride2": ["poolMarchKernel<5,2"],
}


def load_measured_traffic(path=TRAFFIC_TABLE):
    """{operation: HBM bytes per call}: the `traffic bytes` column of the
    profile table, summed over the kernels of one call; the mean over the rows
    where several instantiations of one kernel match (the four matmul layouts)."""
    rows = {}
    try:
        with open(path) as f:
            for line in f:
                cells = [c.strip() for c in line.strip().strip("|").split("|")]
                if len(cells) >= 4 and cells[0].startswith("`") and cells[3].replace(".", "").isdigit():
                    rows[cells[0].strip("`")] = float(cells[3])
    except OSError:
        return {}
    out = {}
    for op, fragments in TRAFFIC_KERNELS.items():
        total = 0.0
        for frag in fragments:
            hits = [v for k, v in rows.items() if frag in k]
            if not hits:
                total = None
                break
            total += sum(hits) / len(hits)
        if total is not None:
            out[op] = int(round(total))
    return out


MEASURED_TRAFFIC_BYTES = load_measured_traffic()
T_ROWS, T_COLS = 12345, 6789
MM = 4096


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_inputs(n):
    rng = np.random.default_rng(20240607)
    a = (rng.random(n, dtype=np.float32) * 2 - 1).astype(np.float32)      # U[-1,1)
    b = (rng.random(n, dtype=np.float32) * 2 - 1).astype(np.float32)      # U[-1,1)
    den = (rng.random(n, dtype=np.float32) * 1.5 + 0.5).astype(np.float32)  # U[0.5,2)
    return a, b, den


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--elements", type=int, default=N_SWEEP,
                    help="elements per tensor in the sweep (default 2^26)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-matmul", action="store_true", help="skip the matmul/transpose legs")
    ap.add_argument("--no-ragged", action="store_true",
                    help="skip the ragged-shape leg (keeps a profile to one problem size per kernel)")
    ap.add_argument("--no-probes", action="store_true",
                    help="skip the memory-pattern probes (pattern ceilings measured beside the builtins)")
    ap.add_argument("--legs", default="transpose,matmul,next,ragged,mid,copies",
                    help="which legs follow the sweep (comma-separated, of transpose, matmul, next, ragged, mid, "
                         "copies): a counter run names the ones whose kernels it is after")
    ap.add_argument("--no-graphs", action="store_true",
                    help="skip the model-graph legs (keeps a profile to one problem size per kernel)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this runtime drives one GPU; --gpus must be 1 "
                 "(no multi-GPU path exists in this build)")

    import __graft_entry__ as entry
    entry.load_package()
    from polarai_framework_amd import capi

    n = args.elements
    dev = capi.Device(0)
    info = dev.info()
    log(f"device: {info.name.decode()} {info.arch.decode()} CUs={info.compute_units} "
        f"clock={info.clock_khz / 1e6:.2f} GHz memclk={info.memory_clock_khz / 1e6:.2f} GHz "
        f"bus={info.memory_bus_bits} bit")

    a, b, den = make_inputs(n)
    da, db, dden = dev.array(a), dev.array(b), dev.array(den)
    outs = {op: dev.empty(n) for op in SWEEP}

    def launch(op):
        if op == "fadd":
            dev.fadd(da, 1.0, db, 1.0, outs[op])
        elif op == "fmul":
            dev.fmul(da, db, outs[op])
        elif op == "fdivide":
            dev.fdivide(da, dden, outs[op])
        elif op == "fsigmoid":
            dev.fsigmoid(da, outs[op])
        elif op == "fcopy":
            dev.fcopy(da, outs[op])
        elif op == "ffill":
            dev.ffill(3.0, outs[op])

    def step(events=None, only=None):
        for op in SWEEP:
            if events is not None and (only is None or op == only):
                events.append(dev.time_next_kernel())
            launch(op)

    def durations(pairs):
        ms = [e0.elapsed_ms(e1) for e0, e1 in pairs]
        for e0, e1 in pairs:
            e0.release(); e1.release()
        return ms

    # Warm-up, with a pair of events on every launch: tells which kernel of the
    # sweep is the slowest.  A pair of events costs a launch a few microseconds
    # of queue time (3-5 % of the sweep's wall-clock rate when every launch
    # carries one), so the timed region below instruments that kernel only; the
    # table of all six comes from a further, untimed pass.
    warm = []
    for _ in range(args.warmup):
        ev = []
        step(ev)
        warm.append(ev)
    dev.synchronize()
    warm_ms = {op: [] for op in SWEEP}
    for ev in warm:
        for op, d in zip(SWEEP, durations(ev)):
            warm_ms[op].append(d)
    # without a warm-up step: the three-stream kernel with the division
    dominant = max(SWEEP, key=lambda op: np.mean(warm_ms[op])) if warm else "fdivide"

    dominant_events = []
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(dominant_events, only=dominant)
    dev.synchronize()
    t1 = time.perf_counter()
    wall = t1 - t0
    dominant_ms = durations(dominant_events)

    all_events = []
    for _ in range(args.steps):
        ev = []
        step(ev)
        all_events.append(ev)
    dev.synchronize()
    per_op_ms = {op: [] for op in SWEEP}
    for ev in all_events:
        for op, d in zip(SWEEP, durations(ev)):
            per_op_ms[op].append(d)
    step_bytes = sum(BYTES_PER_ELEMENT[op] * n for op in SWEEP)
    value = step_bytes * args.steps / wall / 1e9

    per_op = {}
    for op in SWEEP:
        ms = float(np.mean(per_op_ms[op]))
        gbs = BYTES_PER_ELEMENT[op] * n / (ms * 1e-3) / 1e9
        per_op[op] = {"ms": round(ms, 5), "min_ms": round(float(np.min(per_op_ms[op])), 5),
                      "GB/s": round(gbs, 1), "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
                      "algorithmic_bytes": BYTES_PER_ELEMENT[op] * n,
                      "traffic": MEASURED_TRAFFIC_BYTES.get(op) if n == N_SWEEP else None}
        log(f"{op:10s} {ms * 1e3:9.1f} us  {gbs:8.1f} GB/s  {100 * gbs / HBM_PEAK_GBS:5.1f}% of HBM peak")
    dom_ms = float(np.mean(dominant_ms))
    dom_gbs = BYTES_PER_ELEMENT[dominant] * n / (dom_ms * 1e-3) / 1e9
    log(f"timed region: {wall / args.steps * 1e3:.4f} ms/step, {value:.1f} GB/s; slowest kernel {dominant} "
        f"{dom_ms * 1e3:.1f} us in the timed region")
    roofline = {"bound": "hbm", "kernel": dominant,
                "achieved": round(dom_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(dom_gbs / HBM_PEAK_GBS, 4),
                "launch_us": round(dom_ms * 1e3, 2), "launches_timed": len(dominant_ms),
                "traffic": per_op[dominant]["traffic"]}

    # quick sanity of what was timed (full parity lives in tests/)
    probe = outs["fadd"].download()[:1024]
    assert np.array_equal(probe, (a[:1024] + b[:1024]).astype(np.float32)), "fadd output is wrong"

    result = {
        "metric": "elementwise GB/s + fp32 matmul GFLOP/s, % of MI355X roofline, 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "elementwise bandwidth sweep: fadd fmul fdivide fsigmoid fcopy "
                               f"ffill(3.0), fp32, {n} elements per tensor, one kernel each",
                   "elements": n, "bytes_per_step": step_bytes},
        "device": {"name": info.name.decode(), "arch": info.arch.decode(),
                   "compute_units": info.compute_units, "clock_khz": info.clock_khz,
                   "memory_clock_khz": info.memory_clock_khz, "memory_bus_bits": info.memory_bus_bits},
        "roofline": roofline,
        "per_op_timing": "a pair of events on every launch, in a pass of `steps` steps after the timed region; "
                         "the timed region itself (value, ms_per_step) carries events on the slowest kernel only "
                         "(roofline), because a pair of events costs a launch a few microseconds of queue time",
        "per_op": per_op,
    }

    for buf in list(outs.values()) + [dden]:
        buf.free()

    legs = set(args.legs.split(",")) if not args.no_matmul else set()
    unknown = legs - {"transpose", "matmul", "next", "ragged", "mid", "copies", ""}
    if unknown:
        sys.exit(f"bench.py: unknown leg(s) {sorted(unknown)}")
    if args.no_ragged:
        legs -= {"ragged", "mid", "copies"}
    if "transpose" in legs:
        result["transpose"] = bench_transpose(dev, args)
    if "matmul" in legs:
        result["matmul"] = bench_matmul(dev, args)
    if "next" in legs:
        result["next_builtins"] = bench_next_builtins(dev, da, n, args)
    if "ragged" in legs:
        result["ragged"] = bench_ragged(dev, args)
    if "mid" in legs:
        result["matmul_mid_size"] = bench_matmul_mid(dev, args)
    if "copies" in legs:
        result["copies"] = bench_copies(dev)
    da.free(); db.free()
    dev.close()
    dev = None
    if not args.no_probes:
        result["ceilings"] = bench_ceilings(args, n)
    if not args.no_graphs:
        result["graphs"] = bench_graphs()

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(a, b, den, n)

    if dev is not None:
        dev.close()
    summary = summarise_into_roofline(result)
    print(json.dumps(result), flush=True)
    if summary:
        log(summary)  # last line of the run: the whole metric at a glance


RAGGED_PROBES = {  # ragged matmul entry -> the memory-pattern probe that moves the same operands
    "fmatmul_f_f 65536x127x33 as (M,K,N)": "65536 rows of 127 floats in, 65536 rows of 33 floats out",
    "fmatmul_f_f 65536x127x33 as (M,N,K)": "65536 rows of 33 floats in, 65536 rows of 127 floats out",
    "fmatmul_f_f 33x65536x127 as (M,N,K)": "127 rows of 65536 floats in, 33 rows of 65536 floats out",
}


def summarise_into_roofline(result):
    """The metric has two halves (elementwise GB/s, fp32 matmul GFLOP/s) and the
    configurations name a transpose and ragged matmuls: their roofline fractions
    go into `roofline` beside the sweep's dominant kernel, so that one object
    holds all of them.  Returns a one-line summary."""
    roof = result["roofline"]
    parts = [f"sweep {result['value']:.0f} GB/s ({roof['kernel']} {roof['frac']:.3f} of HBM peak)"]
    mm = result.get("matmul")
    if mm:
        variants = mm["variants"].values()
        roof["matmul"] = {"bound": "mfma", "workload": mm["workload"], "achieved": mm["roofline"]["achieved"],
                          "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": mm["roofline"]["frac"],
                          "worst_variant_frac": mm["roofline"]["worst_variant_frac"],
                          "after_idle_frac": round(float(np.mean([v["isolated_frac_mfma_fp32_peak"] for v in variants])), 4),
                          "launch_us": round(float(np.mean([v["ms"] for v in variants])) * 1e3, 1),
                          "launches_before_timing": MM_WARM_LAUNCHES, "traffic": mm["roofline"]["traffic"]}
        parts.append(f"matmul 4096^3 {roof['matmul']['achieved']:.1f} TFLOP/s ({roof['matmul']['frac']:.3f} of fp32 MFMA "
                     f"peak settled, {roof['matmul']['after_idle_frac']:.3f} after idle)")
    tr = result.get("transpose")
    if tr:
        roof["transpose"] = dict(tr["roofline"], workload=tr["workload"], launch_us=round(tr["ms"] * 1e3, 1))
        parts.append(f"transpose {tr['roofline']['frac']:.3f} of HBM peak")
    ragged = result.get("ragged")
    if ragged:
        probes = result.get("ceilings", {}).get("ragged_matmul_pattern", {})
        entries = {k: v for k, v in ragged.items() if k.startswith("fmatmul")}
        for name, v in entries.items():
            probe = probes.get(RAGGED_PROBES.get(name, ""))
            if probe:
                v["pattern_probe_us"] = probe["us"]
                v["first_kernel_vs_probe"] = round(v["first_kernel_us"] / probe["us"], 3)
        worst = min(entries, key=lambda k: entries[k]["frac_hbm_peak"])
        roof["ragged_matmul"] = {k: {"frac_hbm": v["frac_hbm_peak"], "us": v["us"],
                                     "first_kernel_vs_probe": v.get("first_kernel_vs_probe")} for k, v in entries.items()}
        roof["ragged_worst"] = {"entry": worst, "frac_hbm": entries[worst]["frac_hbm_peak"], "us": entries[worst]["us"],
                                "buffers_rotated": True}
        parts.append(f"ragged matmuls {min(v['frac_hbm_peak'] for v in entries.values()):.3f}-"
                     f"{max(v['frac_hbm_peak'] for v in entries.values()):.3f} of HBM peak on compulsory bytes")
    mid = result.get("matmul_mid_size")
    if mid:
        entries = {k: v for k, v in mid.items() if k.startswith("fmatmul")}
        mlp = {k: v for k, v in entries.items() if v["M"] * v["N"] * v["K"] == 1024 * 4096 * 1024}
        roof["matmul_mid_size"] = {k: {"frac_mfma": v["frac_mfma_fp32_peak"], "cold_frac_mfma": v["cold_frac_mfma_fp32_peak"],
                                       "us": v["us"]} for k, v in entries.items()}
        parts.append(f"MLP-shape matmuls {min(v['frac_mfma_fp32_peak'] for v in mlp.values()):.3f}-"
                     f"{max(v['frac_mfma_fp32_peak'] for v in mlp.values()):.3f} of fp32 MFMA peak settled "
                     f"({min(v['cold_frac_mfma_fp32_peak'] for v in mlp.values()):.3f}-"
                     f"{max(v['cold_frac_mfma_fp32_peak'] for v in mlp.values()):.3f} cold)")
    return "summary: " + "; ".join(parts)


def time_kernel(dev, fn, warmup, reps):
    """Per-launch kernel durations of `reps` launches issued back to back, as a
    graph of such operations issues them: every launch carries its own pair of
    events, nothing waits in between.  fn(i) launches exactly one kernel; i
    counts launches, so callers can rotate through several sets of buffers."""
    for i in range(warmup):
        fn(i)
    dev.synchronize()
    pairs = []
    for i in range(reps):
        pairs.append(dev.time_next_kernel())
        fn(warmup + i)
    dev.synchronize()
    ms = []
    for e0, e1 in pairs:
        ms.append(e0.elapsed_ms(e1))
        e0.release(); e1.release()
    return ms


def time_calls(dev, fn, warmup, reps):
    """Durations of calls that may launch several kernels: an event before and
    after each call, calls issued back to back."""
    for i in range(warmup):
        fn(i)
    dev.synchronize()
    marks = [dev.record()]
    for i in range(reps):
        fn(warmup + i)
        marks.append(dev.record())
    dev.synchronize()
    ms = [marks[i].elapsed_ms(marks[i + 1]) for i in range(reps)]
    for e in marks:
        e.release()
    return ms


def time_batches(dev, fn, warmup, batch, runs=5):
    """Seconds per call of `batch` calls issued back to back between ONE pair of
    events (median of `runs` such batches): what a stream of these calls takes per
    call.  An event between every two calls, as time_calls records, puts a marker
    packet between the kernels and costs each call about 3 us."""
    for i in range(warmup):
        fn(i)
    samples = []
    for r in range(runs):
        first = dev.record()
        for i in range(batch):
            fn(warmup + r * batch + i)
        last = dev.record()
        dev.synchronize()
        samples.append(first.elapsed_ms(last) * 1e-3 / batch)
        first.release()
        last.release()
    return float(np.median(samples))


def device_copies(dev, src, count, copies):
    """`copies` buffers holding the same `count` floats as `src` (src is the first)."""
    out = [src]
    for _ in range(copies - 1):
        d = dev.empty(count)
        dev.fcopy(src, d, count)
        out.append(d)
    dev.synchronize()
    return out


ROTATE = 4  # sets of buffers a timed kernel cycles through (each set >= 256 MiB at the sizes below)


def bench_transpose(dev, args):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((T_ROWS, T_COLS), dtype=np.float32)
    dxs = device_copies(dev, dev.array(x), x.size, ROTATE)
    dts = [dev.empty(x.size) for _ in range(ROTATE)]
    ms = time_kernel(dev, lambda i: dev.ftranspose(dxs[i % ROTATE], dts[i % ROTATE], T_ROWS, T_COLS),
                     args.warmup, args.steps)
    for dt in dts[:min(ROTATE, args.warmup + args.steps)]:
        got = dt.download((T_COLS, T_ROWS))
        assert np.array_equal(got[:64], x.T[:64]), "transpose output is wrong"
    for t in dxs + dts:
        t.free()
    nbytes = 8 * T_ROWS * T_COLS
    gbs = nbytes / (np.mean(ms) * 1e-3) / 1e9
    log(f"ftranspose {np.mean(ms) * 1e3:9.1f} us  {gbs:8.1f} GB/s  {100 * gbs / HBM_PEAK_GBS:5.1f}% of HBM peak")
    return {"workload": f"ftranspose {T_ROWS}x{T_COLS} fp32", "ms": round(float(np.mean(ms)), 5),
            "min_ms": round(float(np.min(ms)), 5), "GB/s": round(gbs, 1),
            "buffers_rotated": True, "buffer_sets": ROTATE,
            "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                         "traffic": MEASURED_TRAFFIC_BYTES.get("ftranspose")}}


def bench_next_builtins(dev, dx, n, args):
    """flogloss and fmulconcat (the elementwise builtins outside the headline
    sweep), then the builtins the reference has only as generated code: frelu /
    fsoftmax on the sweep's first input, fconv2d 3x3 and fpool 2x2/2 on an
    8192 x 8192 image.  Every kernel cycles through ROTATE sets of input and
    output buffers (2 GiB or more in total at the default sizes), so that no
    launch finds its operands in a cache the previous launch filled."""
    out = {"buffers_rotated": True, "buffer_sets": ROTATE,
           "rotated_bytes_per_operand": int(4 * n * ROTATE)}
    R = ROTATE

    def report(name, workload, ms, nbytes):
        gbs = nbytes / (np.mean(ms) * 1e-3) / 1e9
        log(f"{name:10s} {np.mean(ms) * 1e3:9.1f} us  {gbs:8.1f} GB/s  {100 * gbs / HBM_PEAK_GBS:5.1f}% of HBM peak")
        out[name] = {"workload": workload, "ms": round(float(np.mean(ms)), 5),
                     "min_ms": round(float(np.min(ms)), 5), "GB/s": round(gbs, 1),
                     "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4), "algorithmic_bytes": int(nbytes),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(name) if n == N_SWEEP else None}

    douts = [dev.empty(n) for _ in range(R)]
    # the two elementwise builtins that are not part of the headline sweep
    rng0 = np.random.default_rng(7)
    dtruths = device_copies(dev, dev.array((rng0.random(n, dtype=np.float32) < 0.1).astype(np.float32)), n, R)
    dpreds = device_copies(dev, dev.array(rng0.random(n, dtype=np.float32)), n, R)
    ms = time_kernel(dev, lambda i: dev.flogloss(dpreds[i % R], dtruths[i % R], douts[i % R]), args.warmup, args.steps)
    report("flogloss", f"{n} elements, predictions U[0,1), labels Bernoulli(0.1), 2R+1W", ms, 12 * n)
    ms = time_kernel(dev, lambda i: dev.fmulconcat(dtruths[i % R], dpreds[i % R], douts[i % R]), args.warmup, args.steps)
    report("fmulconcat", f"{n} elements scaled by gradient[0], 1R+1W", ms, 8 * n)
    for t in dtruths + dpreds:
        t.free()
    dxs = device_copies(dev, dx, n, R)
    ms = time_kernel(dev, lambda i: dev.frelu(dxs[i % R], douts[i % R]), args.warmup, args.steps)
    report("frelu", f"{n} elements, 1R+1W", ms, 8 * n)
    # fsoftmax is three launches (partial sums, total, scale): time per call of a stream of calls
    ms = [time_batches(dev, lambda i: dev.fsoftmax(dxs[i % R], douts[i % R]), args.warmup, max(8, args.steps // 2)) * 1e3]
    report("fsoftmax", f"{n} elements over the whole tensor, 2R+1W (sum pass, scale pass)", ms, 12 * n)
    for t in douts + dxs[1:]:
        t.free()

    h = w = 8192
    rng = np.random.default_rng(8)
    img = rng.standard_normal((h, w), dtype=np.float32)
    k = rng.standard_normal((3, 3), dtype=np.float32)
    dimgs, dk = device_copies(dev, dev.array(img), h * w, R), dev.array(k)
    dconvs = [dev.empty((h - 2) * (w - 2)) for _ in range(R)]
    ms = time_kernel(dev, lambda i: dev.fconv2d(dimgs[i % R], dk, dconvs[i % R], h, w, 3, 3), args.warmup, args.steps)
    report("fconv2d", f"{h}x{w} image, 3x3 kernel, valid correlation", ms, 4 * (h * w + (h - 2) * (w - 2)) + 36)
    for t in dconvs:
        t.free()
    dpools = [dev.empty((h // 2) * (w // 2)) for _ in range(R)]
    ms = time_kernel(dev, lambda i: dev.fpool(dimgs[i % R], dpools[i % R], h, w, (2, 2), (2, 2)), args.warmup, args.steps)
    report("fpool", f"{h}x{w} image, max, window 2x2, stride 2x2", ms, 4 * (h * w + (h // 2) * (w // 2)))
    # an overlapping window (the common CNN pooling): the staged kernel
    oh3, ow3 = (h - 3) // 2 + 1, (w - 3) // 2 + 1
    dpool3 = [dev.empty(oh3 * ow3) for _ in range(R)]
    ms = time_kernel(dev, lambda i: dev.fpool(dimgs[i % R], dpool3[i % R], h, w, (3, 3), (2, 2)), args.warmup, args.steps)
    report("fpool_3x3_stride2", f"{h}x{w} image, max, window 3x3, stride 2x2", ms, 4 * (h * w + oh3 * ow3))
    for t in dpool3:
        t.free()
    # a stride-1 window (as much written as read) and a 5x5 one (the marching kernel)
    for key, win, stride in (("fpool_3x3_stride1", 3, 1), ("fpool_5x5_stride2", 5, 2)):
        oh, ow = (h - win) // stride + 1, (w - win) // stride + 1
        dp = [dev.empty(oh * ow) for _ in range(R)]
        ms = time_kernel(dev, lambda i: dev.fpool(dimgs[i % R], dp[i % R], h, w, (win, win), (stride, stride)),
                         args.warmup, args.steps)
        report(key, f"{h}x{w} image, max, window {win}x{win}, stride {stride}x{stride}", ms, 4 * (h * w + oh * ow))
        got = dp[0].download((oh, ow))[:4, :64]
        want = np.lib.stride_tricks.sliding_window_view(img[:(4 - 1) * stride + win, :(64 - 1) * stride + win],
                                                        (win, win))[::stride, ::stride].max(axis=(2, 3))
        assert np.array_equal(got, want), f"{key} output is wrong"
        for t in dp:
            t.free()
    got = dpools[0].download((h // 2, w // 2))[:8]
    assert np.array_equal(got, img[:16].reshape(8, 2, w // 2, 2).max(axis=(1, 3))), "pool output is wrong"
    for t in dimgs + dpools + [dk]:
        t.free()
    return out


def bench_ceilings(args, n):
    """Memory-pattern probes (kernels that move a builtin's bytes in its pattern
    and do none of its work) timed in this run on this GPU: what HBM delivers
    for streams of reads and writes in the ratios the builtins have, and for the
    reads and writes of a tiled transpose of the benchmark's matrix."""
    import ctypes as C
    lib = C.CDLL(LIB_PROBES)
    reps, warm = max(10, args.steps), max(2, args.warmup)
    us = (C.c_float * reps)()

    def run(fn, *a):
        status = fn(*a, ROTATE, warm, reps, us)
        if status != 0:
            raise RuntimeError(f"{fn.__name__} failed with hipError {status}")
        return float(np.mean(list(us)))

    lib.polar_probe_streams.argtypes = [C.c_int, C.c_uint64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                        C.POINTER(C.c_float)]
    lib.polar_probe_read.argtypes = [C.c_uint64, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_float)]
    lib.polar_probe_transpose_pattern.argtypes = [C.c_uint32, C.c_uint32, C.c_int, C.c_int, C.c_int, C.c_int,
                                                  C.c_int, C.POINTER(C.c_float)]
    lib.polar_probe_panels.argtypes = [C.c_int, C.c_uint32, C.c_uint32, C.c_uint32, C.c_int, C.c_int, C.c_int,
                                       C.POINTER(C.c_float)]
    out = {"note": "probe kernels, not builtins: same bytes and pattern, no work; back-to-back launches, "
                   f"{ROTATE} buffer sets in rotation", "streams": {}, "read_only": {}, "transpose_pattern": {}}
    for reads, like in ((0, "ffill"), (1, "fcopy frelu fsigmoid fconv2d"), (2, "fadd fmul fdivide flogloss"),
                        (4, "fpool 2x2 (4 reads per write)")):
        for ranges in (0, 1):
            t = run(lib.polar_probe_streams, reads, n, ranges, 0, 0)
            gbs = 4 * n * (reads + 1) / (t * 1e-6) / 1e9
            order = "a contiguous eighth per XCD" if ranges else "pieces dealt round-robin to the XCDs"
            out["streams"][f"{reads}R+1W, {order}"] = {"us": round(t, 2), "GB/s": round(gbs, 1),
                                                       "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
                                                       "pattern_of": like}
            log(f"probe {reads}R+1W streams, {order}: {t:7.1f} us  {gbs:7.1f} GB/s  "
                f"{100 * gbs / HBM_PEAK_GBS:5.1f}%   ({like})")
    # a copy whose output is off the line / 16-byte grid: what stores that straddle lines cost
    out["misaligned_copy"] = {}
    for shift, plain in ((0, 1), (4, 0), (4, 1), (2, 0), (2, 1)):
        t = run(lib.polar_probe_streams, 1, n, 0, shift, plain)
        gbs = 8 * n / (t * 1e-6) / 1e9
        label = f"output {4 * shift} B behind a line boundary, {'plain' if plain else 'write-through streaming'} stores"
        out["misaligned_copy"][label] = {"us": round(t, 2), "GB/s": round(gbs, 1),
                                         "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
        log(f"probe copy, {label}: {t:7.1f} us  {gbs:7.1f} GB/s  {100 * gbs / HBM_PEAK_GBS:5.1f}%")
    for unroll in (2, 4, 8, 16):
        t = run(lib.polar_probe_read, n, unroll)
        gbs = 4 * n / (t * 1e-6) / 1e9
        out["read_only"][f"{unroll} x 16 B per lane"] = {"us": round(t, 2), "GB/s": round(gbs, 1),
                                                         "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
        log(f"probe read only, {unroll:2d} loads per lane: {t:7.1f} us  {gbs:7.1f} GB/s  {100 * gbs / HBM_PEAK_GBS:5.1f}%")
    best = max(out["read_only"].values(), key=lambda v: v["GB/s"])
    out["read_only"]["best_GB/s"] = best["GB/s"]
    names = {0: "32x256 tile, 1024 lanes", 1: "32x128 tile, 512 lanes", 2: "32x128 tile, 256 lanes",
             3: "64x256 tile, 1024 lanes", 4: "32x64 tile, 256 lanes",
             5: "128x64 tile, 512 lanes (512-byte chunks per output row)"}
    orders = {0: "row tiles fastest", 1: "column tiles fastest", 2: "column-tile range per XCD"}
    nbytes = 8 * T_ROWS * T_COLS
    for variant in names:
        for order in orders:
            t = run(lib.polar_probe_transpose_pattern, T_ROWS, T_COLS, variant, order)
            gbs = nbytes / (t * 1e-6) / 1e9
            out["transpose_pattern"][f"{names[variant]}, {orders[order]}"] = {
                "us": round(t, 2), "GB/s": round(gbs, 1), "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
            log(f"probe transpose pattern {names[variant]}, {orders[order]}: {t:7.1f} us  {gbs:7.1f} GB/s  "
                f"{100 * gbs / HBM_PEAK_GBS:5.1f}%")
    best = max(out["transpose_pattern"].values(), key=lambda v: v["GB/s"])
    out["transpose_pattern"]["best_GB/s"] = best["GB/s"]
    # the ragged matmuls' memory patterns: rows of the long operand in, rows of C out, no arithmetic
    out["ragged_matmul_pattern"] = {}
    for label, wide, long_dim, in_short, out_short in (
            ("65536 rows of 127 floats in, 65536 rows of 33 floats out", 0, 65536, 127, 33),
            ("65536 rows of 33 floats in, 65536 rows of 127 floats out", 0, 65536, 33, 127),
            ("127 rows of 65536 floats in, 33 rows of 65536 floats out", 1, 65536, 127, 33)):
        nbytes = 4 * long_dim * (in_short + out_short)
        psets = int(RAGGED_ROTATE_BYTES // nbytes) + 1
        status = lib.polar_probe_panels(wide, long_dim, in_short, out_short, psets, max(warm, psets), reps, us)
        if status != 0:
            raise RuntimeError(f"polar_probe_panels failed with hipError {status}")
        t = float(np.mean(list(us)))
        gbs = nbytes / (t * 1e-6) / 1e9
        out["ragged_matmul_pattern"][label] = {"us": round(t, 2), "GB/s": round(gbs, 1),
                                               "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4), "buffer_sets": psets}
        log(f"probe ragged matmul pattern, {label}: {t:7.1f} us  {gbs:7.1f} GB/s  {100 * gbs / HBM_PEAK_GBS:5.1f}%")
    # the plain copy of the transpose's byte count
    nt = (T_ROWS * T_COLS) // 4 * 4
    t = run(lib.polar_probe_streams, 1, nt, 0, 0, 0)
    out["copy_of_transpose_bytes"] = {"us": round(t, 2), "GB/s": round(8 * nt / (t * 1e-6) / 1e9, 1)}
    log(f"probe copy of {8 * nt} bytes: {t:7.1f} us  {8 * nt / (t * 1e-6) / 1e9:7.1f} GB/s")
    return out


def bench_copies(dev):
    """Device::copyToDevice / copyToHost as the plugin performs them (pageable host
    memory): wall time per call including completion, per transfer size."""
    out = {}
    for nbytes in (4 << 10, 256 << 10, 4 << 20, 256 << 20):
        host = np.ones(nbytes // 4, dtype=np.float32)
        back = np.empty_like(host)
        buf = dev.empty(nbytes // 4)
        reps = 5 if nbytes > (64 << 20) else 50
        for _ in range(2):
            dev.copy_to_device(buf.ptr, host.ctypes.data, nbytes); dev.copy_to_host(back.ctypes.data, buf.ptr, nbytes)
        dev.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            dev.copy_to_device(buf.ptr, host.ctypes.data, nbytes)
        dev.synchronize()
        up = (time.perf_counter() - t0) / reps
        t0 = time.perf_counter()
        for _ in range(reps):
            dev.copy_to_host(back.ctypes.data, buf.ptr, nbytes)
        down = (time.perf_counter() - t0) / reps
        assert back[0] == 1.0 and back[-1] == 1.0
        label = f"{nbytes >> 10} KiB" if nbytes < (1 << 20) else f"{nbytes >> 20} MiB"
        out[label] = {"to_device_us": round(up * 1e6, 1), "to_device_GB/s": round(nbytes / up / 1e9, 2),
                      "to_host_us": round(down * 1e6, 1), "to_host_GB/s": round(nbytes / down / 1e9, 2)}
        log(f"copy {label:8s}: to device {up * 1e6:9.1f} us ({nbytes / up / 1e9:6.2f} GB/s), "
            f"to host {down * 1e6:9.1f} us ({nbytes / down / 1e9:6.2f} GB/s)")
        buf.free()
        # the same transfers out of and into a pinned block of the library (no staging)
        block = dev.host_alloc(nbytes)
        try:
            import ctypes
            pinned = np.ctypeslib.as_array(ctypes.cast(block, ctypes.POINTER(ctypes.c_float)), shape=(nbytes // 4,))
            pinned[:] = 1.0
            buf = dev.empty(nbytes // 4)
            for _ in range(2):
                dev.copy_to_device(buf.ptr, block, nbytes); dev.copy_to_host(block, buf.ptr, nbytes)
            dev.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                dev.copy_to_device(buf.ptr, block, nbytes)   # returns with the transfer queued
            dev.synchronize()
            up = (time.perf_counter() - t0) / reps
            t0 = time.perf_counter()
            for _ in range(reps):
                dev.copy_to_host(block, buf.ptr, nbytes)
            down = (time.perf_counter() - t0) / reps
            assert pinned[0] == 1.0 and pinned[-1] == 1.0
            out[label + " pinned block"] = {"to_device_us": round(up * 1e6, 1), "to_device_GB/s": round(nbytes / up / 1e9, 2),
                                            "to_host_us": round(down * 1e6, 1), "to_host_GB/s": round(nbytes / down / 1e9, 2)}
            log(f"     pinned : to device {up * 1e6:9.1f} us ({nbytes / up / 1e9:6.2f} GB/s), "
                f"to host {down * 1e6:9.1f} us ({nbytes / down / 1e9:6.2f} GB/s)")
            buf.free()
        finally:
            dev.host_free(block)
    return out


RAGGED_ROTATE_BYTES = 320 << 20  # bytes a ragged kernel's buffer sets add up to: more than the 256 MB Infinity Cache


def bench_ragged(dev, args):
    """The ragged configuration: fadd/fmul on 1 000 003 elements and the two matmul
    shapes 65536x127x33 / 33x65536x127 under both readings of the triple, (M, K, N)
    and (M, N, K).  These are small: both roofline bounds are reported.  `us` is
    the time per call of a stream of calls (batches of 20 between one pair of
    events, median of 5; kernels that follow a first one are included),
    `us_event_per_call` the same with an event recorded between every two calls
    (about 3 us more: the marker packets), `first_kernel_us` the execution time
    of the call's first kernel alone.  Every kernel cycles through
    as many sets of operands as it takes to exceed the Infinity Cache, so no call
    finds its operands where the previous call left them."""
    out = {"buffers_rotated": True, "rotated_bytes": RAGGED_ROTATE_BYTES}
    n = 1000003
    reps = max(20, args.steps)
    rng = np.random.default_rng(9)
    sets = RAGGED_ROTATE_BYTES // (12 * n) + 1
    ha, hb = rng.random(n, dtype=np.float32), rng.random(n, dtype=np.float32)
    das, dbs = device_copies(dev, dev.array(ha), n, sets), device_copies(dev, dev.array(hb), n, sets)
    dcs = [dev.empty(n) for _ in range(sets)]
    for name, fn in (("fadd", lambda i: dev.fadd(das[i % sets], 1.0, dbs[i % sets], 1.0, dcs[i % sets])),
                     ("fmul", lambda i: dev.fmul(das[i % sets], dbs[i % sets], dcs[i % sets]))):
        ms = time_kernel(dev, fn, max(args.warmup, sets), max(reps, 2 * sets))
        gbs = 12 * n / (np.mean(ms) * 1e-3) / 1e9
        out[f"{name}_{n}"] = {"us": round(float(np.mean(ms)) * 1e3, 2), "GB/s": round(gbs, 1),
                              "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4), "buffer_sets": sets}
        log(f"{name} n={n}: {np.mean(ms) * 1e3:7.1f} us  {gbs:7.1f} GB/s")
    for t in das + dbs + dcs:
        t.free()
    for label, (m, nn, k) in (("65536x127x33 as (M,K,N)", (65536, 33, 127)), ("65536x127x33 as (M,N,K)", (65536, 127, 33)),
                              ("33x65536x127 as (M,K,N)", (33, 127, 65536)), ("33x65536x127 as (M,N,K)", (33, 65536, 127))):
        flops, nbytes = 2.0 * m * nn * k, 4.0 * (m * k + k * nn + m * nn)
        sets = int(RAGGED_ROTATE_BYTES // nbytes) + 1
        das = device_copies(dev, dev.array(rng.standard_normal((m, k), dtype=np.float32)), m * k, sets)
        dbs = device_copies(dev, dev.array(rng.standard_normal((k, nn), dtype=np.float32)), k * nn, sets)
        dcs = [dev.empty(m * nn) for _ in range(sets)]
        call = lambda i: dev.fmatmul(0, 0, das[i % sets], dbs[i % sets], dcs[i % sets], m, nn, k)
        with_events = float(np.mean(time_calls(dev, call, max(3, args.warmup, sets), reps))) * 1e-3
        t = time_batches(dev, call, sets, 20)
        first = float(np.mean(time_kernel(dev, call, sets, reps))) * 1e-3
        out[f"fmatmul_f_f {label}"] = {"M": m, "N": nn, "K": k, "us": round(t * 1e6, 2),
                                       "us_event_per_call": round(with_events * 1e6, 2),
                                       "first_kernel_us": round(first * 1e6, 2),
                                       "GFLOP/s": round(flops / t / 1e9, 1),
                                       "frac_mfma_fp32_peak": round(flops / t / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4),
                                       "min_bytes_GB/s": round(nbytes / t / 1e9, 1),
                                       "frac_hbm_peak": round(nbytes / t / 1e9 / HBM_PEAK_GBS, 4),
                                       "buffer_sets": sets}
        log(f"fmatmul {label}: {t * 1e6:7.1f} us per call ({with_events * 1e6:.1f} with an event per call; first kernel {first * 1e6:.1f} us)  "
            f"{flops / t / 1e12:6.2f} TFLOP/s  {nbytes / t / 1e9:7.1f} GB/s of compulsory traffic  ({sets} operand sets)")
        for x in das + dbs + dcs:
            x.free()
    return out


MID_SETTLE_S = 0.03   # matrix work before the settled timing: what the clock takes to settle
MID_BATCH = 20        # calls between the two events of one settled sample


def bench_matmul_mid(dev, args):
    """Matmuls between the two extremes: the MLP configuration's products (batch 1024,
    1024 -> 4096 -> 1024, forward and gradient graphs) and a few cubes.  Two figures
    per shape, over four rotating sets of operands (a split contraction's reduction
    kernel included in both):
      us        the time per call inside a running job: 30 ms of the same calls first
                (the clock has settled, as for the 4096^3 figure), then the mean of
                20 calls issued back to back between two events, median of 5 such runs;
      cold_us   as a graph evaluated on an idle device meets it: after a synchronize and
                50 ms of sleep, six untimed calls, then the median of calls each between
                its own pair of events (the event records add about 2 us per call)."""
    out = {"timing": f"us: after {MID_SETTLE_S * 1e3:.0f} ms of the same calls, mean of {MID_BATCH} calls back to back "
                     "between two events, median of 5 runs; cold_us: after 50 ms idle, 6 untimed calls, median of "
                     "calls each between its own events; 4 rotating sets of operands"}
    rng = np.random.default_rng(12)
    reps = max(20, args.steps)
    sets = 4
    for ta, tb, m, n, k in ((0, 0, 1024, 4096, 1024), (0, 0, 1024, 1024, 4096), (0, 1, 1024, 4096, 1024),
                            (1, 0, 1024, 4096, 1024), (1, 0, 4096, 1024, 1024), (0, 0, 512, 512, 512),
                            (0, 0, 1024, 1024, 1024), (0, 0, 2048, 2048, 2048), (0, 0, 3072, 3072, 3072)):
        sa, sb = ((k, m) if ta else (m, k)), ((n, k) if tb else (k, n))
        das = device_copies(dev, dev.array(rng.standard_normal(sa, dtype=np.float32)), m * k, sets)
        dbs = device_copies(dev, dev.array(rng.standard_normal(sb, dtype=np.float32)), k * n, sets)
        dcs = [dev.empty(m * n) for _ in range(sets)]
        call = lambda i: dev.fmatmul(ta, tb, das[i % sets], dbs[i % sets], dcs[i % sets], m, n, k)
        flops = 2.0 * m * n * k
        # cold first (the device has just been idle: uploads and allocation)
        dev.synchronize()
        time.sleep(0.05)
        cold = float(np.median(time_calls(dev, call, 6, reps))) * 1e-3
        # settled: enough of the same calls to fill MID_SETTLE_S at the cold rate, then batches
        for i in range(int(MID_SETTLE_S / cold) + 1):
            call(i)
        t = time_batches(dev, call, 0, MID_BATCH)
        config, splits, tile = dev.fmatmul_plan(m, n, k)
        name = f"fmatmul_{'t' if ta else 'f'}_{'t' if tb else 'f'} {m}x{n}x{k}"
        out[name] = {"M": m, "N": n, "K": k, "us": round(t * 1e6, 1), "TFLOP/s": round(flops / t / 1e12, 1),
                     "frac_mfma_fp32_peak": round(flops / t / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4),
                     "cold_us": round(cold * 1e6, 1),
                     "cold_frac_mfma_fp32_peak": round(flops / cold / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4),
                     "tile": "x".join(map(str, tile)), "k_splits": splits}
        log(f"{name:34s} {t * 1e6:8.1f} us  {flops / t / 1e12:6.1f} TFLOP/s  "
            f"({flops / t / 1e12 / MFMA_FP32_PEAK_TFLOPS * 100:.0f} % of the fp32 matrix peak; cold {cold * 1e6:.1f} us, "
            f"{flops / cold / 1e12 / MFMA_FP32_PEAK_TFLOPS * 100:.0f} %; tile {'x'.join(map(str, tile))}, {splits} k-split(s))")
        for x in das + dbs + dcs:
            x.free()
    return out


MM_WARM_LAUNCHES = 40  # back-to-back launches before timing: the GPU clock needs about 30 ms of
                       # continuous matrix work to settle, and a launch timed before that runs ~15 % slower
MM_SETS = 6            # sets of A, B, C the timed launches cycle through (6 x 192 MiB)


def bench_matmul(dev, args):
    rng = np.random.default_rng(6)
    a = rng.standard_normal((MM, MM), dtype=np.float32)
    b = rng.standard_normal((MM, MM), dtype=np.float32)
    das = device_copies(dev, dev.array(a), MM * MM, MM_SETS)
    dbs = device_copies(dev, dev.array(b), MM * MM, MM_SETS)
    dcs = [dev.empty(MM * MM) for _ in range(MM_SETS)]
    flops = 2.0 * MM ** 3
    reps = max(10, args.steps)
    out = {"workload": f"fmatmul {MM}x{MM}x{MM} fp32 N(0,1), C overwritten",
           "timing": f"{reps} launches issued back to back after {MM_WARM_LAUNCHES} untimed ones (settled clock), "
                     f"each with its own pair of events; `isolated_ms` = a launch that follows an idle GPU, "
                     "mean of 5, each after a synchronize and 50 ms of sleep",
           "buffers_rotated": True, "buffer_sets": MM_SETS, "variants": {}}
    worst = None
    for ta in (0, 1):
        for tb in (0, 1):
            name = f"fmatmul_{'t' if ta else 'f'}_{'t' if tb else 'f'}"
            run = lambda i: dev.fmatmul(ta, tb, das[i % MM_SETS], dbs[i % MM_SETS], dcs[i % MM_SETS], MM, MM, MM)
            isolated = []
            run(0)
            for i in range(5):
                dev.synchronize()
                time.sleep(0.05)
                isolated += time_kernel(dev, run, 0, 1)
            ms = time_kernel(dev, run, MM_WARM_LAUNCHES, reps)
            tf = flops / (np.mean(ms) * 1e-3) / 1e12
            # spot check: 4 rows of every result buffer against an fp64 product
            A = a.T if ta else a
            B = b.T if tb else b
            ref = A[:4].astype(np.float64) @ B.astype(np.float64)
            for dc in dcs:
                got = dc.download((MM, MM))[:4]
                err = np.linalg.norm(got - ref) / np.linalg.norm(ref)
                assert err < 1e-4, (name, err)
            out["variants"][name] = {"ms": round(float(np.mean(ms)), 5), "min_ms": round(float(np.min(ms)), 5),
                                     "max_ms": round(float(np.max(ms)), 5),
                                     "GFLOP/s": round(tf * 1e3, 1),
                                     "frac_mfma_fp32_peak": round(tf / MFMA_FP32_PEAK_TFLOPS, 4),
                                     "isolated_ms": round(float(np.mean(isolated)), 5),
                                     "isolated_frac_mfma_fp32_peak": round(
                                         flops / (np.mean(isolated) * 1e-3) / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4)}
            log(f"{name} {np.mean(ms):8.3f} ms  {tf:7.2f} TFLOP/s  {100 * tf / MFMA_FP32_PEAK_TFLOPS:5.1f}% of fp32 MFMA peak"
                f"  (after idle: {np.mean(isolated):.3f} ms)")
            if worst is None or tf < worst:
                worst = tf
    for x in das + dbs + dcs:
        x.free()
    mean_tf = float(np.mean([v["GFLOP/s"] for v in out["variants"].values()])) / 1e3
    out["GFLOP/s"] = round(mean_tf * 1e3, 1)
    out["roofline"] = {"bound": "mfma", "achieved": round(mean_tf, 2), "peak": MFMA_FP32_PEAK_TFLOPS,
                       "unit": "TFLOP/s", "frac": round(mean_tf / MFMA_FP32_PEAK_TFLOPS, 4),
                       "worst_variant_frac": round(worst / MFMA_FP32_PEAK_TFLOPS, 4),
                       "traffic": MEASURED_TRAFFIC_BYTES.get("fmatmul")}
    return out


def bench_graphs():
    """The two model configurations as kernel DAGs through the runtime plugin
    (initContext -> Device::launch per node, barrier per cluster): latency-bound
    at these sizes, so wall-clock per evaluation is what is reported."""
    from polarai_framework_amd import LIB_PLUGIN, graphs, harness
    out = {}
    rng = np.random.default_rng(61)
    x = rng.random((256, 784), dtype=np.float32)
    w = (rng.standard_normal((784, 10)) * 0.01).astype(np.float32)
    bias = np.zeros((256, 10), dtype=np.float32)
    y = (rng.random((256, 10)) < 0.1).astype(np.float32)
    g, _ = graphs.logreg_forward(x, w, bias, y)

    def evaluate(h, n=50):
        for _ in range(5):
            h.run()
        c0 = h.counters()
        ts = []
        for _ in range(n):
            t0 = time.perf_counter(); h.run(); ts.append(time.perf_counter() - t0)
        c = h.counters()
        # host wall time per evaluation, mean of the n: the input nodes' host-side loads; per compute
        # node allocate + lock (uploads happen here), the launch call, the releases; the barriers
        phases = {name: round((getattr(c, "ns_" + name) - getattr(c0, "ns_" + name)) / n / 1e3, 1)
                  for name in ("input_nodes", "allocate_and_lock", "launch", "release", "barrier")}
        return {"evaluate_us": round(float(np.median(ts)) * 1e6, 1), "min_us": round(float(np.min(ts)) * 1e6, 1),
                "mean_us": round(float(np.mean(ts)) * 1e6, 1), "phase_us": phases,
                "uploads_per_evaluate": int((c.copies_to_device - c0.copies_to_device) // n),
                "upload_bytes_per_evaluate": int((c.bytes_to_device - c0.bytes_to_device) // n)}

    def fused(h):
        X, W, B, Y = h.input(x), h.input(w), h.input(bias), h.input(y)
        h.end_cluster()
        p = h.fmatmul_fadd_fsigmoid(False, False, X, W, 1.0, B, 1.0)
        h.end_cluster()
        # flogloss consumes the sigmoid; the fused sigmoid+logloss would need the pre-activation,
        # which the first fused launch does not keep
        h.flogloss(p, Y)
        h.end_cluster()

    for key, pinned in (("logreg_forward", False), ("logreg_forward_plugin_ram", True)):
        with harness.Harness(plugin=LIB_PLUGIN, plugin_host_memory=pinned) as h:
            graphs.emit(g, h, {})
            r = evaluate(h)
        r["workload"] = ("X[256x784] W[784x10]: 4 input nodes, fmatmul_f_f -> fadd -> fsigmoid -> flogloss, "
                         "one barrier per cluster, inputs re-loaded every evaluation as the framework does; "
                         + ("the caller's RAM-side blocks in the plugin's pinned host memory (optional "
                            "polarHostMemory* symbols): uploads are not staged" if pinned else
                            "the caller's RAM-side blocks on the heap, as the framework's allocator keeps them"))
        r["launches_per_evaluate"] = 4
        out[key] = r
        log(f"  phases (us): {r['phase_us']}")
        log(f"{key} through the plugin: {r['evaluate_us']} us per evaluation")
    # the same forward pass with the extended (fused) builtins: 2 launches instead of 4
    for key, pinned in (("logreg_forward_fused", False), ("logreg_forward_fused_plugin_ram", True)):
        with harness.Harness(plugin=LIB_PLUGIN, plugin_host_memory=pinned) as h:
            fused(h)
            r = evaluate(h)
        r["workload"] = ("same inputs; fmatmul_f_f_fadd_fsigmoid -> flogloss (extended builtins)"
                         + ("; RAM-side blocks in the plugin's pinned host memory" if pinned else ""))
        r["launches_per_evaluate"] = 2
        out[key] = r
        log(f"{key}: {r['evaluate_us']} us per evaluation")
    rng = np.random.default_rng(71)
    x = rng.random((1024, 1024), dtype=np.float32)
    w1 = (rng.standard_normal((1024, 4096)) / 32).astype(np.float32)
    w2 = (rng.standard_normal((4096, 1024)) / 64).astype(np.float32)
    y = (rng.random((1024, 1024)) < 0.5).astype(np.float32)
    f, gr, u, _ = graphs.mlp_graphs(x, w1, w2, y)
    for key, pinned in (("mlp_forward_backward", False), ("mlp_forward_backward_plugin_ram", True)):
        with harness.Harness(plugin=LIB_PLUGIN, plugin_host_memory=pinned) as h:
            tensors = {}
            times, spread = {}, {}
            for graph in (f, gr, u):
                graphs.emit(graph, h, tensors)
                h.run()  # first evaluation allocates
                ts = []
                for _ in range(7):
                    t0 = time.perf_counter(); h.run(); ts.append(time.perf_counter() - t0)
                times[graph.name] = float(np.median(ts))
                spread[graph.name] = [round(min(ts) * 1e3, 3), round(max(ts) * 1e3, 3)]
                h.clear_program()
            out[key] = {
                "workload": "batch 1024, 1024->4096->1024, sigmoid, logloss; forward, the framework's gradient "
                            "graph and its in-place weight update, each evaluated through the plugin"
                            + ("; RAM-side blocks in the plugin's pinned host memory" if pinned else ""),
                "forward_ms": round(times["mlp_forward"] * 1e3, 3),
                "gradient_ms": round(times["mlp_gradient"] * 1e3, 3),
                "update_ms": round(times["mlp_update"] * 1e3, 3),
                "min_max_ms": spread,  # of the 7 evaluations whose median is reported
                "nodes": {gph.name: len(gph.nodes) for gph in (f, gr, u)}}
            log(f"{key}: forward {times['mlp_forward'] * 1e3:.2f} ms, gradient "
                f"{times['mlp_gradient'] * 1e3:.2f} ms, update {times['mlp_update'] * 1e3:.2f} ms  (min, max: {spread})")
    return out


def cpu_baseline(a, b, den, n):
    """The CPU oracle (a restatement of the reference's host kernels; the
    reference's own host runtime cannot be built here) timed on this box's
    host cores on the same inputs: one full sweep with all cores, one with a
    single thread, and a 1024^3 matmul with a single thread."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import polar_oracle as o
    cores = o.hw_threads()
    lib = o.lib()
    out = np.empty(n, dtype=np.float32)

    def sweep():
        lib.polar_oracle_fadd(a, 1.0, b, 1.0, out, n)
        lib.polar_oracle_fmul(a, b, out, n)
        lib.polar_oracle_fdivide(a, den, out, n)
        lib.polar_oracle_fsigmoid(a, out, n)
        lib.polar_oracle_fcopy(a, out, n)
        lib.polar_oracle_ffill(3.0, out, n)

    step_bytes = sum(BYTES_PER_ELEMENT[op] * n for op in SWEEP)
    res = {}
    for threads in (cores, 1):
        o.set_threads(threads)
        sweep()  # warm-up (page faults of `out`)
        reps = 3 if threads > 1 else 1
        t0 = time.perf_counter()
        for _ in range(reps):
            sweep()
        dt = (time.perf_counter() - t0) / reps
        res[threads] = step_bytes / dt / 1e9
        log(f"cpu oracle sweep, {threads} thread(s): {dt * 1e3:.1f} ms/step, {res[threads]:.2f} GB/s")
    o.set_threads(1)
    k = 1024
    rng = np.random.default_rng(8)
    ma = rng.standard_normal((k, k), dtype=np.float32)
    mb = rng.standard_normal((k, k), dtype=np.float32)
    t0 = time.perf_counter()
    o.fmatmul(False, False, ma, mb)
    mm_dt = time.perf_counter() - t0
    log(f"cpu oracle fmatmul_f_f 1024^3, 1 thread: {mm_dt:.2f} s, {2 * k ** 3 / mm_dt / 1e9:.2f} GFLOP/s")
    # the GPU leg's own matmul, the whole 4096^3 product, once, with all host threads
    o.set_threads(cores)
    rng = np.random.default_rng(6)
    big_a = rng.standard_normal((MM, MM), dtype=np.float32)
    big_b = rng.standard_normal((MM, MM), dtype=np.float32)
    rows = MM
    t0 = time.perf_counter()
    o.fmatmul(False, False, big_a, big_b, rows=(0, rows))
    big_dt = time.perf_counter() - t0
    big_gflops = 2.0 * rows * MM * MM / big_dt / 1e9
    log(f"cpu oracle fmatmul_f_f {MM}^3, {cores} threads, the whole product: {big_dt:.2f} s, {big_gflops:.2f} GFLOP/s")
    return {"value": round(res[cores], 2), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"the full sweep ({n} elements per tensor, same inputs), {cores} host threads, "
                      "mean of 3 passes after one warm-up pass",
            "single_thread_value": round(res[1], 2),
            "matmul_1024_single_thread_GFLOP/s": round(2 * k ** 3 / mm_dt / 1e9, 3),
            "matmul_4096": {"value": round(big_gflops, 3), "unit": "GFLOP/s", "cores": cores, "kind": "port",
                            "seconds": round(big_dt, 2),
                            "extrapolated": False, "rows": rows,
                            "sample": f"the whole {MM}x{MM}x{MM} fmatmul_f_f, once (same operands as the GPU leg), "
                                      f"{cores} host threads"}}


if __name__ == "__main__":
    main()
