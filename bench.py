#!/usr/bin/env python3
"""Benchmark of the Gaussian dfmmv hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C1|C2|C3|C4|C5] [--no-cpu-baseline]

A step is one ``GaussianKernel.dmmv`` call (K^T (K v + w)) on inputs that are already
resident in HBM; packing of X and C is part of every step.  The headline workload is
the HIGGS-shaped configuration C2: N=1,000,000 x d=28 standard-normal rows, M=20,000
centres drawn from them, sigma=3.8, fp32, one right-hand side.  One JSON line goes to stdout.

Without ``--workload`` the line carries C2 as the headline (with its fp64 twin and the opt-in bf16x3 mode as
sub-records) and a ``configs`` map with one sub-record per other configuration: C1 (fmmv fp64), C3 (dfmmv fp32),
C4 (fmmv and dfmmv, fp32 and fp64) and C5 (Falkon.fit + predict at full size, and the CPU pipeline on a reduced
problem for the prediction-error check).  Every sub-record has its own timed steps, ``roofline`` (product kernel,
average launch time from HIP events on its stream) and ``cpu_baseline`` (the CPU path on the first N' rows: 3 warm-ups,
5 repetitions, min and median).  All GPU measurements are taken first, the CPU legs follow; a wall-clock budget
(``--budget-s``) shortens the CPU legs' repetitions (never below 3) if the box is slower than planned, and every
record says what was run.  With ``--workload`` only that configuration runs and the line is its record.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_PEAK_TFLOPS = 157.3   # MI355X fp32 matrix peak = fp32 vector peak (vendor figure)
FP64_PEAK_TFLOPS = 78.6    # MI355X fp64 matrix peak = fp64 vector peak
BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak


def split_roofline(pairs, d, kern_ms, algorithmic_flop, traffic=None, pairs_cols=1):
    """Roofline of the bf16x3 product kernel: it executes 6 partial products over the features padded to whole
    k-steps of 16 (two of them carry the half norms), on the bf16 matrix cores."""
    ksteps = (d + 2 + 15) // 16
    executed = pairs * 6 * 2 * 16 * ksteps
    achieved = executed / (kern_ms * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": achieved, "peak": BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": achieved / BF16_PEAK_TFLOPS, "traffic": traffic,
            "kernel": ("mmv_split_kernel" if d <= 62 and pairs_cols <= 4 else
                       "mmv_split_wide_kernel" if d <= 62 else "mmv_split_large_kernel"),
            "avg_launch_ms": kern_ms, "flop_per_launch": executed,
            "note": "achieved = bf16 MFMA flops the kernel executes (6 partial products, padded features); "
                    "algorithmic fp32 flops per launch and their rate are given beside it",
            "algorithmic_flop_per_launch": algorithmic_flop,
            "algorithmic_tflops": algorithmic_flop / (kern_ms * 1e-3) / 1e12,
            "algorithmic_frac_of_fp32_peak": algorithmic_flop / (kern_ms * 1e-3) / 1e12 / FP32_PEAK_TFLOPS}

WORKLOADS = {
    # name: (seed, N, d, M, T, has_w)
    "C2": (1002, 1_000_000, 28, 20_000, 1, True),
    "C3": (1003, 10_000_000, 9, 50_000, 1, False),
    "C4": (1004, 500_000, 784, 10_000, 10, True),
}

# HBM bytes per launch of the product kernel come from profiles/hbm_traffic.json, written together with the
# rocprofv3 counter summaries under profiles/ (FETCH_SIZE and WRITE_SIZE in KiB per dispatch, mean over the launches of
# the kernel, each scaled by what the same counter reads for a plain 1 GiB device copy; the file names the commit
# the counters were taken on and the commands).  None where a workload has no entry.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def measured_traffic(workload, dtype, cross_term="f32"):
    """(bytes per launch, provenance) of the product kernel on `workload`, or (None, None)."""
    try:
        with open(TRAFFIC_FILE) as fh:
            table = json.load(fh)
    except (OSError, ValueError):
        return None, None
    entry = table.get("kernels", {}).get(f"{workload}/{dtype}/{cross_term}")
    if not entry:
        return None, None
    cal = table.get("copy_calibration", {})
    nbytes = int((entry["fetch_kib"] * cal.get("fetch_factor", 1.0) + entry["write_kib"] * cal.get("write_factor", 1.0)) * 1024)
    return nbytes, {"file": "profiles/hbm_traffic.json", "commit": table.get("commit"), "kernel": entry.get("kernel")}


def product_kernel_name(d, T, dtype):
    """The kernel the library picks for d features and T right-hand sides (csrc/mmv_small_f32.hip, mmv_small_f64.hip)."""
    if d > 64:      # fp32 with up to four columns: the register-resident kernel up to 128 features
        return "mmv_small_f32_kernel" if dtype == "f32" and d <= 128 and T <= 4 else "mmv_large_kernel"
    if dtype == "f32":
        steps = (d + 1) // 2
        fma_cols = 6 if 8 < steps <= 16 else 4
        return "mmv_small_f32_wide_kernel" if T > fma_cols else "mmv_small_f32_kernel"
    return "mmv_small_f64_wide_kernel" if T > (3 if d > 48 else 4) else "mmv_small_f64_kernel"


def split_kernels_serve(d, T):
    """Whether the bf16x3 kernels serve a call of the bf16x3 mode with d features and T right-hand sides, or the fp32
    kernels do (split_applies in csrc/api.hip)."""
    if d <= 4:
        return False
    if T <= 4:
        return True
    if d > 62:
        return True
    return d > 8 or (T <= 16 and d > 5)


def make_inputs(name, rhs=0):
    """Synthetic inputs of the named configuration (draw order X, idx, sigma, v, w); rhs > 0 replaces the
    configuration's number of right-hand sides."""
    seed, N, d, M, T, has_w = WORKLOADS[name]
    T = rhs or T
    rng = np.random.default_rng(seed)
    if name == "C2":
        X = rng.standard_normal((N, d), dtype=np.float32)
    elif name == "C3":
        X = rng.random((N, d), dtype=np.float32) * 2.0 - 1.0
    else:                                   # C4: uniform[0,1) with 80 % of the entries zeroed, stored dense
        X = rng.random((N, d), dtype=np.float32)
        X *= rng.random((N, d), dtype=np.float32) < 0.2
    idx = rng.choice(N, size=M, replace=False)
    if name == "C2":
        sigma = torch.tensor([3.8], dtype=torch.float64)
    elif name == "C3":
        sigma = torch.from_numpy(rng.uniform(0.5, 2.0, d))
    else:
        sigma = torch.tensor([10.0], dtype=torch.float64)
    v = rng.standard_normal((M, T)).astype(np.float32)
    w = rng.standard_normal((N, T)).astype(np.float32) if has_w else None
    C = np.ascontiguousarray(X[idx])
    return (torch.from_numpy(X), torch.from_numpy(C), sigma, torch.from_numpy(v),
            torch.from_numpy(w) if w is not None else None)


CPU_MEM = 16 * 2**30           # max_cpu_mem of the CPU path (the reference's default of inf would allocate N x M)


def _rel(a, b):
    """Norm-wise relative error per output column, worst column."""
    a, b = a.double().cpu(), b.double().cpu()
    return float(((a - b).norm(dim=0) / b.norm(dim=0)).max())


def note(msg):
    """Progress on stderr (stdout carries the one JSON line): a run of several minutes must not look hung."""
    print(f"[bench {time.strftime('%H:%M:%S')}] {msg}", file=sys.stderr, flush=True)


class Budget:
    """Wall-clock plan of the CPU legs.  Each leg has a nominal cost in seconds; when a leg starts it may spend its
    nominal cost, scaled down if what is left of the run's budget no longer covers the nominal cost of all the legs
    still to come."""

    def __init__(self, total_s, legs):
        self.t0, self.total, self.legs = time.perf_counter(), total_s, dict(legs)

    def elapsed(self):
        return time.perf_counter() - self.t0

    def allowance(self, leg):
        pending = sum(self.legs.values())
        nominal = self.legs.pop(leg)
        left = self.total - self.elapsed()
        return nominal * min(1.0, max(left, 0.0) / max(pending, 1e-9))


def cpu_timed(run, warm, allowance_s, want_warm=3, want_reps=5):
    """`want_warm` untimed calls of `warm` and `want_reps` timed calls of `run`; the counts shrink (to no fewer than
    1 and 3) when `allowance_s` seconds do not cover them.  Returns (sorted times, last result, warm-ups done)."""
    t0 = time.perf_counter()
    warmed = 0
    for _ in range(want_warm):
        warm()
        warmed += 1
        note(f"  cpu warm-up {warmed} done")
        if time.perf_counter() - t0 > 0.3 * allowance_s:
            break
    times, res = [], None
    for _ in range(want_reps):
        s0 = time.perf_counter()
        res = run()
        times.append(time.perf_counter() - s0)
        note(f"  cpu repetition {len(times)}: {times[-1]:.2f} s")
        if len(times) >= 3 and (time.perf_counter() - t0) + times[-1] > allowance_s:
            break
    return sorted(times), res, warmed


def cpu_baseline(op, X, C, sigma, v, w, rows, warm_rows, gpu_same, gpu_f64, allowance_s, anchor=None,
                 kernel_name="gaussian", anchor_share=0.22):
    """Reference-equivalent CPU path (the oracle restatement, torch CPU ops) on the first `rows` rows of X with the
    full M, max_cpu_mem = 16 GiB.

    Timing: 3 warm-ups (on the first `warm_rows` rows: the same code path and block size at a fraction of the cost)
    and 5 timed repetitions over the `rows` rows, min and median.  Parity: the result of the timed runs (the data's
    dtype) and the same path in fp64 on the same rows as the anchor (`anchor` if the caller already has it, else one
    more pass) -- every distance is to a CPU-computed result; `gpu_same` / `gpu_f64` are the GPU results on those
    rows in the data's dtype and in fp64 (the latter is only reported beside the anchors)."""
    from oracle import mmv_ref                      # checker only; never on the product path
    M, T = v.shape

    def path(Xr, wr, vv, CC):
        if op == "dmmv":
            return mmv_ref.fdmmv_ref(Xr, CC, vv, wr, sigma, max_cpu_mem=CPU_MEM, kernel_name=kernel_name)
        return mmv_ref.fmmv_ref(Xr, CC, vv, sigma, max_cpu_mem=CPU_MEM, kernel_name=kernel_name)

    Xs = X[:rows].contiguous()
    ws = w[:rows].contiguous() if (w is not None and op == "dmmv") else None
    Xw = X[:warm_rows].contiguous()
    ww = w[:warm_rows].contiguous() if ws is not None else None
    if X.dtype == torch.float32 and anchor is None:
        allowance_s *= 1.0 - anchor_share              # the fp64 pass for the anchor comes out of the same allowance
    times, cpu_same, warmed = cpu_timed(lambda: path(Xs, ws, v, C), lambda: path(Xw, ww, v, C), allowance_s)
    med = times[len(times) // 2]
    name = "dfmmv" if op == "dmmv" else "fmmv"
    base = {"value": rows * M * T / med, "unit": "kernel entries/s", "cores": torch.get_num_threads(),
            "kind": "port", "host_cpus": os.cpu_count(),
            "sample": f"{name} on the first {rows} rows of X with the full M={M} (linear in N), max_cpu_mem=16GiB, "
                      f"{warmed} warm-ups (on the first {warm_rows} rows) + {len(times)} repetitions: "
                      f"median {med:.2f} s, min {times[0]:.2f} s",
            "value_at_min_time": rows * M * T / times[0], "seconds_median": med, "seconds_min": times[0],
            "warmups": warmed, "repetitions": len(times), "parity_rows": rows}
    tol32, tol64 = 1e-5, 1e-11
    if X.dtype == torch.float64:
        e = _rel(gpu_same, cpu_same)
        base.update({"rel_err_gpu_f64_vs_cpu_f64": e, "fp64_within_1e-11": e <= tol64,
                     "parity_statement": f"GPU fp64 result {e:.2e} from the fp64 CPU path (bar {tol64:g})"})
        return base, cpu_same
    if anchor is None:
        t0 = time.perf_counter()
        anchor = path(Xs.double(), ws.double() if ws is not None else None, v.double(), C.double())
        base["anchor_f64_s"] = time.perf_counter() - t0
        note(f"  cpu fp64 anchor: {base['anchor_f64_s']:.2f} s")
    e_gpu32, e_cpu32, e_pair = _rel(gpu_same, anchor), _rel(cpu_same, anchor), _rel(gpu_same, cpu_same)
    if e_pair <= tol32:
        statement = f"GPU fp32 result within {tol32:g} of the fp32 CPU path ({e_pair:.2e})"
    else:
        statement = (f"fp32 CPU path is {e_cpu32:.2e} from its fp64 twin (CPU), the GPU fp32 result {e_gpu32:.2e}: "
                     f"the two fp32 results differ by {e_pair:.2e} > {tol32:g} because of the CPU path's own fp32 "
                     f"accumulation; the 1e-5 bar is read as 'no further from the fp64 CPU result than the fp32 CPU path'")
    base.update({  # every anchor below is computed on the CPU
                 "rel_err_gpu_f32_vs_cpu_f64": e_gpu32, "rel_err_cpu_f32_vs_cpu_f64": e_cpu32,
                 "rel_err_gpu_f32_vs_cpu_f32": e_pair, "parity_statement": statement})
    if gpu_f64 is not None:
        e64 = _rel(gpu_f64, anchor)
        base.update({"rel_err_gpu_f64_vs_cpu_f64": e64, "fp64_within_1e-11": e64 <= tol64,
                     "rel_err_gpu_f32_vs_gpu_f64": _rel(gpu_same, gpu_f64)})   # extra: GPU against GPU, not an anchor
    return base, anchor


def measure_products(lib, call, steps, warmup):
    """`warmup` untimed and `steps` timed calls of `call` (host clock around the timed calls, a synchronisation on
    both sides), with the library's HIP events around every product-kernel launch of the timed calls."""
    from falkon_amd import _backend
    first_ms = None
    for i in range(warmup):
        t0 = time.perf_counter()
        call()
        if i == 0:                                   # the first call of the process: cold caches, lazy module load
            torch.cuda.synchronize()
            first_ms = (time.perf_counter() - t0) * 1e3
    torch.cuda.synchronize()
    lib.flk_kernel_timing_enable(1)                  # HIP events around each product-kernel launch, on its stream
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        call()
        marks[i + 1].record()                        # per-step spread only; the headline uses the host clock
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
    tot_ms, launches = ctypes.c_double(), ctypes.c_int64()
    _backend.raise_for_status(lib.flk_kernel_timing_read(ctypes.byref(tot_ms), ctypes.byref(launches)), "flk_kernel_timing_read")
    lib.flk_kernel_timing_enable(0)
    return {"s_per_step": elapsed / steps, "kern_ms": tot_ms.value / max(launches.value, 1), "launches": launches.value,
            "per_step": per_step, "first_ms": first_ms, "steps": steps, "warmup": warmup}


SIGMA_TEXT = {"C2": "sigma=3.8", "C3": "per-dimension sigma", "C4": "sigma=10"}


def product_record(workload, op, dtype, N, d, M, T, meas, kernel_name="gaussian", split=False, traffic_ok=True):
    """The JSON record of one timed product workload from `measure_products`' figures."""
    peak = FP32_PEAK_TFLOPS if dtype == "f32" else FP64_PEAK_TFLOPS
    s_step, kern_ms, launches, steps = meas["s_per_step"], meas["kern_ms"], meas["launches"], meas["steps"]
    # one launch of the product kernel evaluates all N*M pairs once: (2d+4) flop per kernel value + 2T to contract
    flop_per_launch = N * M * (2 * d + 4 + 2 * T)
    achieved = flop_per_launch / (kern_ms * 1e-3) / 1e12 if kern_ms > 0 else 0.0
    traffic, traffic_src = measured_traffic(workload, dtype, "bf16x3" if split else "f32") \
        if (traffic_ok and op == "dmmv" and kernel_name == "gaussian") else (None, None)
    per_step = meas["per_step"]
    name = "dfmmv" if op == "dmmv" else "fmmv"
    res = {
        "metric": f"{name} kernel-entries/sec (N*M*T/s) {'fp32' if dtype == 'f32' else 'fp64'}, 1 MI355X",
        "value": N * M * T / s_step, "unit": "kernel entries/s", "n_gpus": 1, "steps": steps, "warmup": meas["warmup"],
        "ms_per_step": s_step * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype if not split else "f32 (cross term: bf16x3 split, fp32 accumulate)", "data": "synthetic",
        "config": {"workload": f"{workload}: {kernel_name} {'dfmmv K^T(Kv+w)' if op == 'dmmv' else 'fmmv K v'}, N={N}, d={d}, M={M}, T={T}, "
                               f"{SIGMA_TEXT[workload]}, {'fp32' if dtype == 'f32' else 'fp64'}, "
                               f"{'cross term on the bf16 matrix cores from a 3-way bfloat16 split, ' if split else ''}"
                               f"inputs resident in HBM, packing included in every step"},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
                     "frac": achieved / peak,
                     "traffic": traffic, "traffic_source": traffic_src,
                     "kernel": product_kernel_name(d, T, dtype),
                     "launches_per_step": launches / steps,
                     "avg_launch_ms": kern_ms, "flop_per_launch": flop_per_launch},
        "whole_step_flop_frac": (N * M * ((2 if op == "dmmv" else 1) * (2 * d + 4 + 2 * T))) / s_step / 1e12 / peak,
        "ms_per_step_min": per_step[0] if per_step else None,
        "ms_per_step_median": per_step[len(per_step) // 2] if per_step else None,
        "ms_first_call": meas["first_ms"],
    }
    if op == "dmmv":
        # the conservative count: one kernel evaluation per pair, as if K were stored between the two products
        res["single_evaluation_flop_frac"] = (N * M * (2 * d + 4 + 4 * T)) / s_step / 1e12 / peak
    if launches == 0:
        # many right-hand sides: the drivers stored blocks of K (kernel-matrix kernel + rocBLAS GEMMs), no product
        # kernel ran and K was evaluated once per step: the rate is that flop count (E(d) + 2T or 4T per pair) over
        # the step time
        once = res.get("single_evaluation_flop_frac", res["whole_step_flop_frac"])
        res["roofline"] = {"bound": "mfma", "achieved": once * peak, "peak": peak, "unit": "TFLOP/s", "frac": once,
                           "traffic": None, "kernel": "kernel-matrix kernel + rocBLAS GEMMs on stored blocks of K",
                           "launches_per_step": 0.0, "avg_launch_ms": None, "flop_per_launch": None}
        if split and d > 64:
            # the stored blocks come from the bf16x3 kernel-matrix kernel: priced, like the bf16x3 product kernels,
            # on the bf16 matrix flops executed (one evaluation of K per step), the fp32 count kept beside it
            executed = N * M * 6 * 2 * 16 * ((d + 2 + 15) // 16)
            res["roofline"].update(achieved=executed / s_step / 1e12, peak=BF16_PEAK_TFLOPS,
                                   frac=executed / s_step / 1e12 / BF16_PEAK_TFLOPS,
                                   algorithmic_frac_of_fp32_peak=once)
    if split and launches > 0 and split_kernels_serve(d, T):
        res["roofline"] = dict(split_roofline(N * M, d, kern_ms, flop_per_launch, traffic, pairs_cols=T),
                               launches_per_step=launches / steps, traffic_source=traffic_src)
    return res


def run_c1(args, lib, defer_cpu=False):
    """Configuration 1 (N = 20 000, d = 8, M = 1 000, one right-hand side, fp64 fmmv): a launch-bound call.  Reports the
    time of a call the host waits for, the rate of calls issued back to back, the product kernel's share, and the
    result against the whole CPU path (the case is small enough to run it in full)."""
    from falkon_amd import GaussianKernel, _backend
    dev = torch.device("cuda:0")
    N, d, M, T = 20_000, 8, 1_000, 1
    rng = np.random.default_rng(1001)                # draw order X, idx, v
    X = torch.from_numpy(rng.standard_normal((N, d)))
    C = X[torch.from_numpy(rng.choice(N, size=M, replace=False))].contiguous()
    v = torch.from_numpy(rng.standard_normal((M, T)))
    tdt = torch.float64 if args.dtype == "f64" else torch.float32
    X, C, v = X.to(tdt), C.to(tdt), v.to(tdt)
    Xg, Cg, vg = X.to(dev), C.to(dev), v.to(dev)
    kernel = GaussianKernel(2.0)
    out = torch.empty(N, T, dtype=tdt, device=dev)
    for _ in range(max(args.warmup, 20)):
        kernel.mmv(Xg, Cg, vg, out=out)
    torch.cuda.synchronize()
    waits = []
    for _ in range(200):
        t0 = time.perf_counter()
        kernel.mmv(Xg, Cg, vg, out=out)
        torch.cuda.synchronize()
        waits.append(time.perf_counter() - t0)
    steps = max(args.steps, 1000)
    lib.flk_kernel_timing_enable(1)
    t0 = time.perf_counter()
    for _ in range(steps):
        kernel.mmv(Xg, Cg, vg, out=out)
    host = time.perf_counter() - t0
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    tot_ms, launches = ctypes.c_double(), ctypes.c_int64()
    _backend.raise_for_status(lib.flk_kernel_timing_read(ctypes.byref(tot_ms), ctypes.byref(launches)), "flk_kernel_timing_read")
    lib.flk_kernel_timing_enable(0)
    kern_ms = tot_ms.value / max(launches.value, 1)
    flop = N * M * (2 * d + 4 + 2 * T)
    peak = FP64_PEAK_TFLOPS if tdt == torch.float64 else FP32_PEAK_TFLOPS
    res = {
        "metric": f"fmmv kernel-entries/sec (N*M*T/s) {'fp64' if tdt == torch.float64 else 'fp32'}, 1 MI355X",
        "value": N * M * T / (elapsed / steps), "unit": "kernel entries/s", "n_gpus": 1, "steps": steps,
        "warmup": max(args.warmup, 20), "ms_per_step": elapsed / steps * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f64" if tdt == torch.float64 else "f32", "data": "synthetic",
        "config": {"workload": f"C1: gaussian fmmv K v, N={N}, d={d}, M={M}, T={T}, sigma=2, "
                               f"{'fp64' if tdt == torch.float64 else 'fp32'}, inputs resident in HBM, packing included in "
                               "every call, calls issued back to back"},
        "latency_us_per_waited_call": {"median": float(np.median(waits)) * 1e6, "min": min(waits) * 1e6},
        "host_us_per_call": host / steps * 1e6,
        "roofline": {"bound": "mfma", "achieved": flop / (kern_ms * 1e-3) / 1e12 if kern_ms > 0 else 0.0, "peak": peak,
                     "unit": "TFLOP/s", "frac": flop / (kern_ms * 1e-3) / 1e12 / peak if kern_ms > 0 else 0.0,
                     "traffic": None, "kernel": product_kernel_name(d, T, "f64" if tdt == torch.float64 else "f32"),
                     "launches_per_step": launches.value / steps, "avg_launch_ms": kern_ms, "flop_per_launch": flop,
                     "note": "launch-bound: 79 000 tiles of 16 x 16 fill the chip for a few block steps only"},
    }
    ctx = (X, C, v, out.cpu())
    if not args.no_cpu_baseline and not defer_cpu:
        c1_cpu_leg(res, ctx)
    return res, ctx


def c1_cpu_leg(res, ctx):
    """The whole of configuration 1 on the CPU path: 3 warm-ups + 5 repetitions, and the GPU result against it."""
    from oracle import mmv_ref                      # checker only; never on the product path
    X, C, v, got = ctx
    N, M, T = X.shape[0], C.shape[0], v.shape[1]
    times, ref, warmed = cpu_timed(lambda: mmv_ref.fmmv_ref(X, C, v, 2.0), lambda: mmv_ref.fmmv_ref(X, C, v, 2.0), 30.0)
    med = times[len(times) // 2]
    res["cpu_baseline"] = {"value": N * M * T / med, "unit": "kernel entries/s",
                           "cores": torch.get_num_threads(), "kind": "port", "host_cpus": os.cpu_count(),
                           "sample": f"the whole of C1, {warmed} warm-ups + {len(times)} repetitions: median "
                                     f"{med * 1e3:.2f} ms, min {times[0] * 1e3:.2f} ms",
                           "value_at_min_time": N * M * T / times[0], "parity_rows": N,
                           "rel_err_gpu_vs_cpu": _rel(got, ref)}


def make_c5(N, Nts, seed=1005, d=28):
    """Train/test rows and +-1 labels y = sign(sin(x.a) + 0.3 eps), a ~ N(0, I/d); draw order X, Xts, a, eps, eps_ts."""
    rng = np.random.default_rng(seed)
    X = rng.standard_normal((N, d)).astype(np.float32)
    Xts = rng.standard_normal((Nts, d)).astype(np.float32)
    a = rng.standard_normal(d) / np.sqrt(d)
    y = np.sign(np.sin(X @ a) + 0.3 * rng.standard_normal(N)).astype(np.float32)
    yts = np.sign(np.sin(Xts @ a) + 0.3 * rng.standard_normal(Nts)).astype(np.float32)
    return tuple(torch.from_numpy(t) for t in (X, y.reshape(-1, 1), Xts, yts.reshape(-1, 1)))


def run_c5(args, lib, defer_cpu=False):
    """End-to-end fit + predict; returns the JSON record."""
    from falkon_amd import Falkon, FalkonOptions, GaussianKernel, _backend
    dev = torch.device("cuda:0")
    N, M, d, sigma, lam, iters = args.c5_n, args.c5_m, 28, 3.8, 1e-6, 20
    Nts = N // 10
    X, Y, Xts, Yts = make_c5(N, Nts)
    Xg, Yg, Xtsg = X.to(dev), Y.to(dev), Xts.to(dev)
    n_dmmv = iters + iters // FalkonOptions().cg_full_gradient_every     # one per iteration + the full residuals
    fit_s, pre_s, pred_s, kern_ms, launches = [], [], [], 0.0, 0
    mse = err = None
    split = args.cross_term == "bf16x3"
    opt = FalkonOptions(bf16x3_cross_term=split, cg_capture_graph=args.cg_graph)
    for it in range(args.warmup + args.steps):
        timed = it >= args.warmup
        model = Falkon(GaussianKernel(sigma, opt=opt), lam, M=M, maxiter=iters, seed=12, options=opt)
        torch.cuda.synchronize()
        if timed:
            lib.flk_kernel_timing_enable(1)
        t0 = time.perf_counter()
        model.fit(Xg, Yg)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        if timed:
            tot_ms, cnt = ctypes.c_double(), ctypes.c_int64()
            _backend.raise_for_status(lib.flk_kernel_timing_read(ctypes.byref(tot_ms), ctypes.byref(cnt)),
                                      "flk_kernel_timing_read")
            lib.flk_kernel_timing_enable(0)
            kern_ms += tot_ms.value
            launches += cnt.value
        pred = model.predict(Xtsg)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        if timed:
            fit_s.append(t1 - t0)
            pre_s.append(model.fit_times_[0])          # centres + K(C,C) + both Cholesky factorisations
            pred_s.append(t2 - t1)
        mse = float(((pred.cpu() - Yts) ** 2).mean())
        err = float((torch.sign(pred.cpu()) != Yts).float().mean())
        note(f"  C5 fit {it + 1}: {t1 - t0:.2f} s, predict {t2 - t1:.4f} s")
        del model, pred
    fit, pre, prd = float(np.mean(fit_s)), float(np.mean(pre_s)), float(np.mean(pred_s))
    cg = fit - pre
    # the same preconditioner with the diagonal blocks of its factorisations left to the library routine
    # (FalkonOptions(pc_tile_factorisation=False)), built twice, the second build timed
    from falkon_amd.preconditioner import FalkonPreconditioner
    opt_lib = FalkonOptions(bf16x3_cross_term=split, pc_tile_factorisation=False)
    pre_lib = None
    for _ in range(0 if args.no_cpu_baseline else 2):      # (a baseline leg: skipped with the CPU legs)
        pc = FalkonPreconditioner(lam, GaussianKernel(sigma, opt=opt_lib), opt_lib)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        pc.init(Xg[:M])
        torch.cuda.synchronize()
        pre_lib = time.perf_counter() - t0
        del pc
    if pre_lib is not None:
        note(f"  C5 preconditioner with the library's factorisation of the diagonal blocks: {pre_lib:.2f} s")
    flop_per_launch = N * M * (2 * d + 4 + 2)
    kern_avg = kern_ms / max(launches, 1)
    achieved = flop_per_launch / (kern_avg * 1e-3) / 1e12
    # (the counters were taken at the full size only)
    c5_traffic, c5_traffic_src = measured_traffic("C5", "f32") if (N, M) == (2_000_000, 50_000) and not split else (None, None)
    res = {
        "metric": "dfmmv kernel-entries/sec (N*M*T/s) fp32 inside Falkon.fit, 1 MI355X",
        "value": N * M * n_dmmv / cg, "unit": "kernel entries/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": (fit + prd) * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32" if not split else "f32 (cross term: bf16x3 split, fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": f"C5: Falkon.fit + predict, N={N}, d={d}, M={M} uniform centres, sigma=3.8, "
                               f"penalty=1e-6, {iters} CG iterations ({n_dmmv} dfmmv + 1 fmmv), test rows {Nts}, "
                               f"fp32{' with the bf16x3 cross term' if split else ''}, data resident in HBM"},
        "fit_s": fit, "preconditioner_s": pre, "cg_s": cg, "predict_s": prd, "test_mse": mse, "test_error_rate": err,
        "preconditioner": "K(C,C) by this library, two blocked Cholesky factorisations and T T^T on library GEMMs, "
                          "their diagonal tiles by flk_potrf_tile",
        "preconditioner_s_with_library_factorisation_of_diagonal_blocks": pre_lib,
        "cg_graph": bool(args.cg_graph), "product_kernel_s_per_fit": kern_ms * 1e-3 / max(args.steps, 1),
        "cg_s_over_product_kernel_s": cg / (kern_ms * 1e-3 / max(args.steps, 1)) if kern_ms > 0 else None,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / FP32_PEAK_TFLOPS, "traffic": c5_traffic, "traffic_source": c5_traffic_src,
                     "kernel": "mmv_small_f32_kernel",
                     "launches_per_step": launches / max(args.steps, 1), "avg_launch_ms": kern_avg,
                     "flop_per_launch": flop_per_launch},
    }
    if split:
        res["roofline"] = dict(split_roofline(N * M, d, kern_avg, flop_per_launch),
                               launches_per_step=launches / max(args.steps, 1))
    ctx = None
    if not args.no_cpu_baseline:
        # the same pipeline at a size the CPU finishes in seconds, on both sides, same centres: the GPU side here
        n2, m2 = args.cpu_rows or 200_000, 5_000
        X2, Y2, X2ts, Y2ts = make_c5(n2, n2 // 10)
        small = Falkon(GaussianKernel(sigma, opt=opt), lam, M=m2, maxiter=iters, seed=12, options=opt)
        small.fit(X2.to(dev), Y2.to(dev))
        mse_gpu = float(((small.predict(X2ts.to(dev)).cpu() - Y2ts) ** 2).mean())
        ctx = (X2, Y2, X2ts, Y2ts, small.ny_points_.cpu(), mse_gpu, sigma, lam, iters, n_dmmv)
        del small
        if not defer_cpu:
            c5_cpu_leg(res, ctx)
    return res, ctx


def c5_cpu_leg(res, ctx):
    """Preconditioner + CG + predict on the CPU (scipy LAPACK + the CPU product path) at the reduced size, and the
    test error of the GPU fit on the same rows and centres beside it."""
    from oracle import falkon_ref                  # checker only; never on the product path
    X2, Y2, X2ts, Y2ts, C2, mse_gpu, sigma, lam, iters, n_dmmv = ctx
    n2, m2 = X2.shape[0], C2.shape[0]
    t0 = time.perf_counter()
    alpha_ref = falkon_ref.falkon_fit_ref(X2, Y2, C2, sigma, lam, maxiter=iters)
    dt = time.perf_counter() - t0
    mse_cpu = float(((falkon_ref.falkon_predict_ref(X2ts, C2, alpha_ref, sigma) - Y2ts) ** 2).mean())
    res["cpu_baseline"] = {"value": n2 * m2 * n_dmmv / dt, "unit": "kernel entries/s",
                           "cores": torch.get_num_threads(), "kind": "port", "host_cpus": os.cpu_count(),
                           "sample": f"whole fit (preconditioner + {iters} CG iterations) at N={n2}, M={m2}, one run, "
                                     f"{dt:.2f} s; the rate counts the fit's {n_dmmv} dfmmv over the whole fit time",
                           "test_mse_cpu": mse_cpu, "test_mse_gpu_same_sample": mse_gpu,
                           "mse_rel_diff": abs(mse_gpu - mse_cpu) / mse_cpu,
                           "mse_within_0.1_percent": abs(mse_gpu - mse_cpu) / mse_cpu <= 1e-3}


# Rows of X the CPU path is run on per configuration (the products are linear in N), and the rows of its warm-ups.
CPU_ROWS = {"C2": (1_000_000, 200_000), "C3": (200_000, 80_000), "C4": (100_000, 25_000)}
# Nominal cost in seconds of the CPU legs of the default run, in the order they run (16 host cores).
CPU_LEGS = [("C2", 70.0), ("C3", 38.0), ("C4/dmmv/f64", 36.0), ("C4/mmv/f64", 18.0), ("C4/dmmv/f32", 18.0),
            ("C4/mmv/f32", 9.0), ("C5", 16.0), ("C1", 1.0)]


def sub_record(rec):
    """A product record as a sub-record of the `configs` map: the driver-contract keys that repeat the headline's
    are dropped."""
    for key in ("n_gpus", "higher_is_better", "scaling", "vs_baseline", "data", "ms_first_call"):
        rec.pop(key, None)
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default 50; C5, whose step is a whole fit: 2)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default 3; C5: 1)")
    ap.add_argument("--workload", default=None, choices=["C1"] + sorted(WORKLOADS) + ["C5"],
                    help="run this configuration only (default: C2 as the headline and every other configuration as a "
                         "sub-record of the `configs` map)")
    ap.add_argument("--budget-s", type=float, default=270.0,
                    help="wall-clock budget of the whole run; the CPU legs shorten their repetitions to keep it")
    ap.add_argument("--c5-n", type=int, default=2_000_000, help="training rows of the C5 workload")
    ap.add_argument("--c5-m", type=int, default=50_000, help="centres of the C5 workload")
    ap.add_argument("--dtype", default=None, choices=["f32", "f64"],
                    help="arithmetic type (default: f32, the headline; f64 for C1, which is an fp64 configuration)")
    ap.add_argument("--op", default="dmmv", choices=["dmmv", "mmv"],
                    help="dmmv = K^T(Kv+w), the headline; mmv = K v only (one launch per step)")
    ap.add_argument("--kernel", default="gaussian", choices=["gaussian", "laplacian", "matern32", "matern52"],
                    help="kernel function (the headline is the Gaussian; the flop count of the roofline stays the "
                         "Gaussian's 2d+4+2T per pair, the other kernels spend a few more VALU operations per entry)")
    ap.add_argument("--cross-term", default="f32", choices=["f32", "bf16x3"],
                    help="f32 (the headline): fp32 MFMA.  bf16x3: the opt-in mode that forms x.c on the bf16 matrix cores "
                         "from an exact three-way bfloat16 split of the fp32 rows (fp32 accuracy; fp32 data); "
                         "its roofline is priced against the bf16 MFMA peak on the flops it executes")
    ap.add_argument("--stored-blocks", action="store_true",
                    help="FalkonOptions(dmmv_stored_blocks=True): dfmmv beyond 64 features through stored blocks of K "
                         "(not the headline path, which never materialises K)")
    ap.add_argument("--cg-graph", action="store_true",
                    help="C5 only: FalkonOptions(cg_capture_graph=True), the CG iterations replayed from HIP graphs")
    ap.add_argument("--rhs", type=int, default=0, metavar="T",
                    help="right-hand sides instead of the configuration's own number (not a headline workload)")
    ap.add_argument("--features", type=int, default=0, metavar="D",
                    help="feature count instead of the configuration's own (C2, C3 or C4 with --no-cpu-baseline; not a "
                         "headline workload: the same matrices' shape at another d)")
    ap.add_argument("--no-cpu-baseline", action="store_true",
                    help="only the timed steps of one workload (C2 unless --workload names another): neither the CPU "
                         "baseline, nor the side measurements, nor the other configurations (profiling runs)")
    ap.add_argument("--cpu-rows", type=int, default=0)
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="BYTES",
                    help="only run a plain device copy of BYTES bytes five times (reference point for the "
                         "FETCH_SIZE / WRITE_SIZE counters) and exit")
    args = ap.parse_args()
    every_config = args.workload is None and not args.no_cpu_baseline and not args.copy_calibration
    if args.workload is None:
        args.workload = "C2"
    if args.dtype is None:
        args.dtype = "f64" if args.workload == "C1" else "f32"
    if args.steps is None:
        args.steps = 2 if args.workload == "C5" else 50
    if args.warmup is None:
        args.warmup = 1 if args.workload == "C5" else 3
    if args.features:
        if args.workload not in WORKLOADS or not args.no_cpu_baseline or args.features < 1:
            print("bench.py: --features needs --no-cpu-baseline and one of the workloads C2, C3, C4", file=sys.stderr)
            sys.exit(2)
        seed, N, _, M, T, has_w = WORKLOADS[args.workload]
        WORKLOADS[args.workload] = (seed, N, args.features, M, T, has_w)
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only; --gpus must be 1 "
              "(sharding would split the rows of X and end with one M x T all-reduce; it is not built)",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)

    if args.copy_calibration:
        src = torch.ones(args.copy_calibration // 4, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration_bytes": src.numel() * 4, "copies": 5}))
        return

    from falkon_amd import FalkonOptions, GaussianKernel, LaplacianKernel, MaternKernel, _backend
    lib = _backend.load()                            # raises if the HIP library is missing
    budget = Budget(args.budget_s, CPU_LEGS if every_config else [(args.workload, 1e9)])
    kopt = FalkonOptions(bf16x3_cross_term=args.cross_term == "bf16x3", dmmv_stored_blocks=args.stored_blocks)
    kernel_classes = {"gaussian": (lambda s, o: GaussianKernel(s, opt=o), "gaussian"),
                      "laplacian": (lambda s, o: LaplacianKernel(s, opt=o), "laplacian"),
                      "matern32": (lambda s, o: MaternKernel(s, 1.5, opt=o), "1.5-matern"),
                      "matern52": (lambda s, o: MaternKernel(s, 2.5, opt=o), "2.5-matern")}
    make_kernel_with, kernel_name = kernel_classes[args.kernel]
    if args.workload == "C1":
        print(json.dumps(run_c1(args, lib)[0]), flush=True)
        return
    if args.workload == "C5":
        print(json.dumps(run_c5(args, lib)[0]), flush=True)
        return
    dev = torch.device("cuda:0")
    split = args.cross_term == "bf16x3"
    if split and args.dtype != "f32":
        print("bench.py: --cross-term bf16x3 applies to fp32 data", file=sys.stderr)
        sys.exit(2)

    # ------------------------------------------------------------------ GPU phase (every timed region of the run)
    cpu_jobs = []                                    # (leg, function that runs the CPU leg and fills its record)

    def products_of(workload, legs, rhs=0, with_sides=False, cpu_for=None):
        """Timed steps of `workload` for every (op, dtype, steps, warmup) in `legs`; returns {(op, dtype): record} and
        queues the CPU legs (for the legs in `cpu_for`; default: all).  The data lives on the host for the CPU legs and
        on the device for the duration of this call."""
        _, N, d, M, T, _ = WORKLOADS[workload]
        T = rhs or T
        note(f"{workload}: generating inputs")
        X, C, sigma, v, w = make_inputs(workload, rhs)
        kernel = make_kernel_with(sigma, kopt)
        rows, warm_rows = CPU_ROWS[workload]
        rows = min(args.cpu_rows or rows, N)
        warm_rows = min(warm_rows, rows)
        on_dev, recs, parity = {}, {}, {}
        for op, dtype, steps, warmup in legs:
            tdt = torch.float32 if dtype == "f32" else torch.float64
            if dtype not in on_dev:
                on_dev[dtype] = tuple(None if a is None else a.to(dev).to(tdt) for a in (X, C, v, w))
            Xg, Cg, vg, wg = on_dev[dtype]
            out = torch.empty(M if op == "dmmv" else N, T, dtype=tdt, device=dev)
            call = (lambda: kernel.dmmv(Xg, Cg, vg, wg, out=out)) if op == "dmmv" else (lambda: kernel.mmv(Xg, Cg, vg, out=out))
            meas = measure_products(lib, call, steps, warmup)
            rec = product_record(workload, op, dtype, N, d, M, T, meas, kernel_name, split, traffic_ok=not rhs and not args.features)
            note(f"gpu {workload} {op} {dtype}: {rec['ms_per_step']:.3f} ms per step, roofline frac {rec['roofline']['frac']:.3f}")
            recs[(op, dtype)] = rec
            if args.no_cpu_baseline:
                continue
            # the GPU result on the rows the CPU path will be run on
            if rows == N:
                parity[(op, dtype)] = out.cpu()
            elif op == "dmmv":
                parity[(op, dtype)] = kernel.dmmv(Xg[:rows], Cg, vg, None if wg is None else wg[:rows]).cpu()
            else:
                parity[(op, dtype)] = out[:rows].cpu()
            if with_sides and not split and dtype == "f32" and args.kernel == "gaussian":
                # not the headline: the same step with the opt-in bf16x3 cross term (fp32 data and results, the cross
                # term on the bf16 matrix cores from an exact three-way split)
                k3 = make_kernel_with(sigma, FalkonOptions(bf16x3_cross_term=True))
                out3 = torch.empty_like(out)
                call3 = (lambda: k3.dmmv(Xg, Cg, vg, wg, out=out3)) if op == "dmmv" else (lambda: k3.mmv(Xg, Cg, vg, out=out3))
                m3 = measure_products(lib, call3, steps, max(warmup, 1))
                r3 = product_record(workload, op, "f32", N, d, M, T, m3, kernel_name, True)
                rec["opt_in_bf16x3_cross_term"] = {"value": r3["value"], "ms_per_step": r3["ms_per_step"], "steps": steps,
                                                   "roofline": r3["roofline"],
                                                   "rel_diff_from_fp32_kernels": _rel(out3, out)}
                parity[(op, "bf16x3")] = out3.cpu() if rows == N else None
        del on_dev
        torch.cuda.empty_cache()
        if args.no_cpu_baseline:
            return recs

        # ------- CPU legs of this workload (run later, after every GPU measurement of the run)
        anchors = {}

        def leg(op, dtype):
            def run():
                name = workload if every_config and workload != "C4" else (f"{workload}/{op}/{dtype}" if every_config else workload)
                tdt = torch.float32 if dtype == "f32" else torch.float64
                note(f"cpu leg {workload} {op} {dtype} on {rows} rows ({budget.elapsed():.0f} s into the run)")
                Xc, Cc, vc = X[:rows].to(tdt), C.to(tdt), v.to(tdt)
                wc = None if w is None else w[:rows].to(tdt)
                base, anchor = cpu_baseline(op, Xc, Cc, sigma, vc, wc, rows, warm_rows, parity[(op, dtype)],
                                            parity.get((op, "f64")) if dtype == "f32" else None,
                                            budget.allowance(name), anchors.get(op), kernel_name)
                anchors[op] = anchor
                recs[(op, dtype)]["cpu_baseline"] = base
                side = recs[(op, dtype)].get("opt_in_bf16x3_cross_term")
                if side is not None and parity.get((op, "bf16x3")) is not None:
                    side["rel_err_vs_cpu_f64"] = _rel(parity[(op, "bf16x3")], anchor)
            return run

        # fp64 legs first: their results are the anchors of the fp32 legs on the same rows
        for op, dtype, _, _ in sorted(legs, key=lambda l: l[1] != "f64"):
            if cpu_for is None or (op, dtype) in cpu_for:
                cpu_jobs.append(leg(op, dtype))
        return recs

    if not every_config:
        recs = products_of(args.workload, [(args.op, args.dtype, args.steps, args.warmup)], args.rhs,
                           with_sides=not args.no_cpu_baseline)
        for job in cpu_jobs:
            job()
        print(json.dumps(recs[(args.op, args.dtype)]), flush=True)
        return

    # the default run: C2 is the headline (fp32, with its fp64 twin and the bf16x3 mode beside it) ...
    c2 = products_of("C2", [("dmmv", "f32", args.steps, args.warmup), ("dmmv", "f64", max(10, args.steps // 2), 2)],
                     with_sides=True, cpu_for=[("dmmv", "f32")])
    res = c2[("dmmv", "f32")]
    side64 = sub_record(c2[("dmmv", "f64")])
    res["fp64"] = side64
    # ... and every other configuration a sub-record
    sub_steps, sub_warm = 10, 3
    c1, c1_ctx = run_c1(argparse.Namespace(**{**vars(args), "dtype": "f64"}), lib, defer_cpu=True)
    c3 = products_of("C3", [("dmmv", "f32", sub_steps, sub_warm)])
    c4 = products_of("C4", [(op, dtype, sub_steps, sub_warm) for dtype in ("f32", "f64") for op in ("mmv", "dmmv")])
    c5_args = argparse.Namespace(**{**vars(args), "steps": 2, "warmup": 1})
    note("C5: fit + predict")
    c5, c5_ctx = run_c5(c5_args, lib, defer_cpu=True)
    gpu_phase_s = budget.elapsed()
    note(f"gpu phase done after {gpu_phase_s:.0f} s")

    # ------------------------------------------------------------------ CPU phase
    # in the order of CPU_LEGS; C2: one fp32 leg over all rows, whose fp64 anchor (one more pass) also serves the
    # fp64 sub-record
    for job in cpu_jobs:
        job()
    cb = res["cpu_baseline"]
    side64["rel_err_vs_cpu_f64"] = cb.get("rel_err_gpu_f64_vs_cpu_f64")
    side64["parity_rows"] = cb["parity_rows"]
    note("cpu leg C5 (reduced pipeline)")
    c5_cpu_leg(c5, c5_ctx)
    c1_cpu_leg(c1, c1_ctx)
    res["configs"] = {
        "C1": sub_record(c1),
        "C3": {"dfmmv_f32": sub_record(c3[("dmmv", "f32")])},
        "C4": {f"{'dfmmv' if op == 'dmmv' else 'fmmv'}_{dtype}": sub_record(rec) for (op, dtype), rec in c4.items()},
        "C5": sub_record(c5),
    }
    res["run_s"] = {"gpu_phase": gpu_phase_s, "total": budget.elapsed(), "budget": args.budget_s}
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
