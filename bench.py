#!/usr/bin/env python3
"""Benchmark of the Gaussian dfmmv hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C2|C3] [--no-cpu-baseline]

A step is one ``GaussianKernel.dmmv`` call (K^T (K v + w)) on inputs that are already
resident in HBM; packing of X and C is part of every step.  The default workload is
the HIGGS-shaped configuration: N=1,000,000 x d=28 standard-normal rows, M=20,000
centres drawn from them, sigma=3.8, fp32, one right-hand side.  One JSON line goes to stdout.
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
    if d > 64:
        return "mmv_large_kernel"
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


def cpu_baseline(X, C, sigma, v, w, gpu_out_fn, rows, time_rows, reps, kernel_name="gaussian"):
    """Reference-equivalent CPU path (the oracle restatement, torch CPU ops).

    Timing: dfmmv on the first `time_rows` rows with the full M, two warm-ups and `reps` timed repetitions (min and
    median).  Parity: on the first `rows` rows (all of them for config 2) the CPU path in the data's dtype at
    max_cpu_mem = 16 GiB and at 4 GiB (the fp32 accumulation order follows the row blocks), and the same path in
    fp64 on the same inputs as the anchor -- every distance is to a CPU-computed result; the GPU's own fp64 result
    is only reported beside them."""
    from oracle import mmv_ref                      # checker only; never on the product path
    M, T = v.shape
    Xt = X[:time_rows].contiguous()
    wt = w[:time_rows].contiguous() if w is not None else None
    times = []
    for i in range(2 + reps):
        t0 = time.perf_counter()
        mmv_ref.fdmmv_ref(Xt, C, v, wt, sigma, max_cpu_mem=CPU_MEM, kernel_name=kernel_name)
        if i >= 2:
            times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    Xs = X[:rows].contiguous()
    ws = w[:rows].contiguous() if w is not None else None
    base = {"value": time_rows * M * T / med, "unit": "kernel entries/s", "cores": torch.get_num_threads(),
            "kind": "port", "host_cpus": os.cpu_count(),
            "sample": f"dfmmv on the first {time_rows} rows of X with the full M={M} (linear in N), "
                      f"max_cpu_mem=16GiB, 2 warm-ups + {reps} repetitions: median {med:.2f} s, min {times[0]:.2f} s",
            "value_at_min_time": time_rows * M * T / times[0], "parity_rows": rows}
    t0 = time.perf_counter()
    cpu64 = mmv_ref.fdmmv_ref(Xs.double(), C.double(), v.double(), ws.double() if ws is not None else None, sigma,
                              max_cpu_mem=CPU_MEM, kernel_name=kernel_name)
    f64_s = time.perf_counter() - t0
    got, got64 = gpu_out_fn(Xs, ws)
    tol32, tol64 = 1e-5, 1e-11
    e_gpu64 = _rel(got64, cpu64)
    base.update({"rel_err_gpu_f64_vs_cpu_f64": e_gpu64, "fp64_within_1e-11": e_gpu64 <= tol64})
    if X.dtype == torch.float64:
        base["parity_run_s"] = {"cpu_f64_16GiB": f64_s}
        base["parity_statement"] = f"GPU fp64 result {e_gpu64:.2e} from the fp64 CPU path (bar {tol64:g})"
        return base
    t0 = time.perf_counter()
    cpu32 = mmv_ref.fdmmv_ref(Xs, C, v, ws, sigma, max_cpu_mem=CPU_MEM, kernel_name=kernel_name)
    full_s = time.perf_counter() - t0
    cpu32_4g = mmv_ref.fdmmv_ref(Xs, C, v, ws, sigma, max_cpu_mem=4 * 2**30, kernel_name=kernel_name)
    e_gpu32, e_cpu32, e_cpu32_4g = _rel(got, cpu64), _rel(cpu32, cpu64), _rel(cpu32_4g, cpu64)
    e_pair, e_pair_4g = _rel(got, cpu32), _rel(got, cpu32_4g)
    if e_pair <= tol32:
        statement = f"GPU fp32 result within {tol32:g} of the fp32 CPU path ({e_pair:.2e})"
    else:
        statement = (f"fp32 CPU path is {e_cpu32:.2e} from its fp64 twin (CPU), the GPU fp32 result {e_gpu32:.2e}: "
                     f"the two fp32 results differ by {e_pair:.2e} > {tol32:g} because of the CPU path's own fp32 "
                     f"accumulation; the 1e-5 bar is read as 'no further from the fp64 CPU result than the fp32 CPU path'")
    base.update({"parity_run_s": {"cpu_f32_16GiB": full_s, "cpu_f64_16GiB": f64_s},
                 "value_parity_run": rows * M * T / full_s,
                 # every anchor below is computed on the CPU
                 "rel_err_gpu_f32_vs_cpu_f64": e_gpu32, "rel_err_cpu_f32_vs_cpu_f64": e_cpu32,
                 "rel_err_cpu_f32_4GiB_vs_cpu_f64": e_cpu32_4g,
                 "rel_err_gpu_f32_vs_cpu_f32": e_pair, "rel_err_gpu_f32_vs_cpu_f32_4GiB": e_pair_4g,
                 "rel_err_gpu_f32_vs_gpu_f64": _rel(got, got64),          # extra: GPU against GPU, not an anchor
                 "parity_statement": statement})
    return base


def run_c1(args, lib):
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
    if not args.no_cpu_baseline:
        from oracle import mmv_ref                      # checker only; never on the product path
        for _ in range(2):
            ref = mmv_ref.fmmv_ref(X, C, v, 2.0)
        ts = []
        for _ in range(5):
            t0 = time.perf_counter()
            ref = mmv_ref.fmmv_ref(X, C, v, 2.0)
            ts.append(time.perf_counter() - t0)
        res["cpu_baseline"] = {"value": N * M * T / float(np.median(ts)), "unit": "kernel entries/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": "the whole of C1, 2 warm-ups + 5 repetitions, median",
                               "rel_err_gpu_vs_cpu": _rel(out.cpu(), ref)}
    return res


def make_c5(N, Nts, seed=1005, d=28):
    """Train/test rows and +-1 labels y = sign(sin(x.a) + 0.3 eps), a ~ N(0, I/d); draw order X, Xts, a, eps, eps_ts."""
    rng = np.random.default_rng(seed)
    X = rng.standard_normal((N, d)).astype(np.float32)
    Xts = rng.standard_normal((Nts, d)).astype(np.float32)
    a = rng.standard_normal(d) / np.sqrt(d)
    y = np.sign(np.sin(X @ a) + 0.3 * rng.standard_normal(N)).astype(np.float32)
    yts = np.sign(np.sin(Xts @ a) + 0.3 * rng.standard_normal(Nts)).astype(np.float32)
    return tuple(torch.from_numpy(t) for t in (X, y.reshape(-1, 1), Xts, yts.reshape(-1, 1)))


def run_c5(args, lib):
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
        del model, pred
    fit, pre, prd = float(np.mean(fit_s)), float(np.mean(pre_s)), float(np.mean(pred_s))
    cg = fit - pre
    flop_per_launch = N * M * (2 * d + 4 + 2)
    kern_avg = kern_ms / max(launches, 1)
    achieved = flop_per_launch / (kern_avg * 1e-3) / 1e12
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
        "cg_graph": bool(args.cg_graph), "product_kernel_s_per_fit": kern_ms * 1e-3 / max(args.steps, 1),
        "cg_s_over_product_kernel_s": cg / (kern_ms * 1e-3 / max(args.steps, 1)) if kern_ms > 0 else None,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / FP32_PEAK_TFLOPS, "traffic": None, "kernel": "mmv_small_f32_kernel",
                     "launches_per_step": launches / max(args.steps, 1), "avg_launch_ms": kern_avg,
                     "flop_per_launch": flop_per_launch},
    }
    if split:
        res["roofline"] = dict(split_roofline(N * M, d, kern_avg, flop_per_launch),
                               launches_per_step=launches / max(args.steps, 1))
    if not args.no_cpu_baseline:
        # the same pipeline at a size the CPU finishes in seconds, on both sides, same centres
        from oracle import falkon_ref                  # checker only; never on the product path
        n2, m2 = args.cpu_rows or 200_000, 5_000
        X2, Y2, X2ts, Y2ts = make_c5(n2, n2 // 10)
        small = Falkon(GaussianKernel(sigma, opt=opt), lam, M=m2, maxiter=iters, seed=12, options=opt)
        small.fit(X2.to(dev), Y2.to(dev))
        mse_gpu = float(((small.predict(X2ts.to(dev)).cpu() - Y2ts) ** 2).mean())
        C2 = small.ny_points_.cpu()
        t0 = time.perf_counter()
        alpha_ref = falkon_ref.falkon_fit_ref(X2, Y2, C2, sigma, lam, maxiter=iters)
        dt = time.perf_counter() - t0
        mse_cpu = float(((falkon_ref.falkon_predict_ref(X2ts, C2, alpha_ref, sigma) - Y2ts) ** 2).mean())
        res["cpu_baseline"] = {"value": n2 * m2 * n_dmmv / dt, "unit": "kernel entries/s",
                               "cores": torch.get_num_threads(), "kind": "port", "host_cpus": os.cpu_count(),
                               "sample": f"whole fit (preconditioner + {iters} CG iterations) at N={n2}, M={m2}, "
                                         f"{dt:.2f} s; the rate counts the fit's {n_dmmv} dfmmv over the whole fit time",
                               "test_mse_cpu": mse_cpu, "test_mse_gpu_same_sample": mse_gpu,
                               "mse_rel_diff": abs(mse_gpu - mse_cpu) / mse_cpu}
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default 50; C5, whose step is a whole fit: 2)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default 3; C5: 1)")
    ap.add_argument("--workload", default="C2", choices=["C1"] + sorted(WORKLOADS) + ["C5"])
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
    ap.add_argument("--no-cpu-baseline", action="store_true",
                    help="only the timed steps: neither the CPU baseline nor the bf16x3 side measurement (profiling runs)")
    ap.add_argument("--cpu-rows", type=int, default=0)
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="BYTES",
                    help="only run a plain device copy of BYTES bytes five times (reference point for the "
                         "FETCH_SIZE / WRITE_SIZE counters) and exit")
    args = ap.parse_args()
    if args.dtype is None:
        args.dtype = "f64" if args.workload == "C1" else "f32"
    if args.steps is None:
        args.steps = 2 if args.workload == "C5" else 50
    if args.warmup is None:
        args.warmup = 1 if args.workload == "C5" else 3
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
    kopt = FalkonOptions(bf16x3_cross_term=args.cross_term == "bf16x3", dmmv_stored_blocks=args.stored_blocks)
    def make_kernel_with(o):
        return {"gaussian": lambda s: GaussianKernel(s, opt=o), "laplacian": lambda s: LaplacianKernel(s, opt=o),
                "matern32": lambda s: MaternKernel(s, 1.5, opt=o), "matern52": lambda s: MaternKernel(s, 2.5, opt=o)}[args.kernel]

    make_kernel, kernel_name = {"gaussian": (lambda s: GaussianKernel(s, opt=kopt), "gaussian"),
                                "laplacian": (lambda s: LaplacianKernel(s, opt=kopt), "laplacian"),
                                "matern32": (lambda s: MaternKernel(s, 1.5, opt=kopt), "1.5-matern"),
                                "matern52": (lambda s: MaternKernel(s, 2.5, opt=kopt), "2.5-matern")}[args.kernel]
    if args.workload == "C1":
        print(json.dumps(run_c1(args, lib)), flush=True)
        return
    if args.workload == "C5":
        print(json.dumps(run_c5(args, lib)), flush=True)
        return
    dev = torch.device("cuda:0")
    seed, N, d, M, T, has_w = WORKLOADS[args.workload]
    T = args.rhs or T
    split = args.cross_term == "bf16x3"
    if split and args.dtype != "f32":
        print("bench.py: --cross-term bf16x3 applies to fp32 data", file=sys.stderr)
        sys.exit(2)
    X, C, sigma, v, w = make_inputs(args.workload, args.rhs)
    tdt = torch.float32 if args.dtype == "f32" else torch.float64
    X, C, v = X.to(tdt), C.to(tdt), v.to(tdt)
    w = w.to(tdt) if w is not None else None
    peak = FP32_PEAK_TFLOPS if args.dtype == "f32" else FP64_PEAK_TFLOPS
    Xg, Cg, vg = X.to(dev), C.to(dev), v.to(dev)
    wg = w.to(dev) if w is not None else None
    kernel = make_kernel(sigma)
    out = torch.empty(M if args.op == "dmmv" else N, T, dtype=tdt, device=dev)

    def step():
        if args.op == "dmmv":
            kernel.dmmv(Xg, Cg, vg, wg, out=out)
        else:
            kernel.mmv(Xg, Cg, vg, out=out)

    first_ms = None
    for i in range(args.warmup):
        t0 = time.perf_counter()
        step()
        if i == 0:                                   # the first call of the process: cold caches, lazy module load
            torch.cuda.synchronize()
            first_ms = (time.perf_counter() - t0) * 1e3
    torch.cuda.synchronize()
    lib.flk_kernel_timing_enable(1)                  # HIP events around each product-kernel launch, on its stream
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(args.steps):
        step()
        marks[i + 1].record()                        # per-step spread only; the headline uses the host clock
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    tot_ms, launches = ctypes.c_double(), ctypes.c_int64()
    rc = lib.flk_kernel_timing_read(ctypes.byref(tot_ms), ctypes.byref(launches))
    _backend.raise_for_status(rc, "flk_kernel_timing_read")
    lib.flk_kernel_timing_enable(0)

    ms_per_step = elapsed / args.steps * 1e3
    value = N * M * T / (elapsed / args.steps)
    # one launch of the product kernel evaluates all N*M pairs once: (2d+4) flop per kernel value + 2T to contract
    flop_per_launch = N * M * (2 * d + 4 + 2 * T)
    kern_ms = tot_ms.value / max(launches.value, 1)
    achieved = flop_per_launch / (kern_ms * 1e-3) / 1e12 if kern_ms > 0 else 0.0
    traffic, traffic_src = (None, None) if args.rhs or args.op != "dmmv" or args.kernel != "gaussian" else \
        measured_traffic(args.workload, args.dtype, args.cross_term)
    res = {
        "metric": f"{'dfmmv' if args.op == 'dmmv' else 'fmmv'} kernel-entries/sec (N*M*T/s) {'fp32' if args.dtype == 'f32' else 'fp64'}, 1 MI355X",
        "value": value, "unit": "kernel entries/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype if not split else "f32 (cross term: bf16x3 split, fp32 accumulate)", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {kernel_name} {'dfmmv K^T(Kv+w)' if args.op == 'dmmv' else 'fmmv K v'}, N={N}, d={d}, M={M}, T={T}, "
                               f"{ {'C2': 'sigma=3.8', 'C3': 'per-dimension sigma', 'C4': 'sigma=10'}[args.workload] }, "
                               f"{'fp32' if args.dtype == 'f32' else 'fp64'}, "
                               f"{'cross term on the bf16 matrix cores from a 3-way bfloat16 split, ' if split else ''}"
                               f"inputs resident in HBM, packing included in every step"},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
                     "frac": achieved / peak,
                     "traffic": traffic, "traffic_source": traffic_src,
                     "kernel": product_kernel_name(d, T, args.dtype),
                     "launches_per_step": launches.value / args.steps,
                     "avg_launch_ms": kern_ms, "flop_per_launch": flop_per_launch},
        "whole_step_flop_frac": (N * M * ((2 if args.op == "dmmv" else 1) * (2 * d + 4 + 2 * T)))
                                / (elapsed / args.steps) / 1e12 / peak,
        "ms_per_step_min": per_step[0] if per_step else None,
        "ms_per_step_median": per_step[len(per_step) // 2] if per_step else None,
        "ms_first_call": first_ms,
    }
    if args.op == "dmmv":
        # the conservative count: one kernel evaluation per pair, as if K were stored between the two products
        res["single_evaluation_flop_frac"] = (N * M * (2 * d + 4 + 4 * T)) / (elapsed / args.steps) / 1e12 / peak
    if launches.value == 0:
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
            res["roofline"].update(achieved=executed / (elapsed / args.steps) / 1e12, peak=BF16_PEAK_TFLOPS,
                                   frac=executed / (elapsed / args.steps) / 1e12 / BF16_PEAK_TFLOPS,
                                   algorithmic_frac_of_fp32_peak=once)
    if split and launches.value > 0 and split_kernels_serve(d, T):
        res["roofline"] = dict(split_roofline(N * M, d, kern_ms, flop_per_launch, traffic, pairs_cols=T),
                               launches_per_step=launches.value / args.steps, traffic_source=traffic_src)
    if not split and args.dtype == "f32" and args.kernel == "gaussian" and not args.no_cpu_baseline:
        # not the headline: the same step with the opt-in bf16x3 cross term (fp32 data and results, the cross term
        # on the bf16 matrix cores from an exact three-way split), timed after the run above, and how far its
        # result is from the fp32 kernels' result
        ref_out = out.clone()
        kernel = make_kernel_with(FalkonOptions(bf16x3_cross_term=True))(sigma)
        for _ in range(max(args.warmup, 1)):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        el = time.perf_counter() - t0
        diff = float(((out.double() - ref_out.double()).norm(dim=0) / ref_out.double().norm(dim=0)).max())
        res["opt_in_bf16x3_cross_term"] = {"value": N * M * T / (el / args.steps), "ms_per_step": el / args.steps * 1e3,
                                           "rel_diff_from_fp32_kernels": diff}
        kernel = make_kernel(sigma)
    side64 = None
    if not split and args.dtype == "f32" and args.kernel == "gaussian" and args.op == "dmmv" and not args.no_cpu_baseline:
        # the fp64 half of the metric: the same step on the same inputs widened to fp64 (fewer steps: it is not
        # the headline), product-kernel time from the library's HIP events as above
        X64, C64, v64 = Xg.double(), Cg.double(), vg.double()
        w64 = wg.double() if wg is not None else None
        out64 = torch.empty(M, T, dtype=torch.float64, device=dev)
        steps64 = max(5, args.steps // 5)
        for _ in range(2):
            kernel.dmmv(X64, C64, v64, w64, out=out64)
        torch.cuda.synchronize()
        lib.flk_kernel_timing_enable(1)
        t0 = time.perf_counter()
        for _ in range(steps64):
            kernel.dmmv(X64, C64, v64, w64, out=out64)
        torch.cuda.synchronize()
        el64 = (time.perf_counter() - t0) / steps64
        tot64, n64 = ctypes.c_double(), ctypes.c_int64()
        _backend.raise_for_status(lib.flk_kernel_timing_read(ctypes.byref(tot64), ctypes.byref(n64)), "flk_kernel_timing_read")
        lib.flk_kernel_timing_enable(0)
        k64 = tot64.value / max(n64.value, 1)
        a64 = flop_per_launch / (k64 * 1e-3) / 1e12 if k64 > 0 else 0.0
        tr64, tr64_src = measured_traffic(args.workload, "f64")
        side64 = {"metric": "dfmmv kernel-entries/sec (N*M*T/s) fp64, 1 MI355X", "value": N * M * T / el64,
                  "unit": "kernel entries/s", "dtype": "f64", "steps": steps64, "warmup": 2, "ms_per_step": el64 * 1e3,
                  "roofline": {"bound": "mfma", "achieved": a64, "peak": FP64_PEAK_TFLOPS, "unit": "TFLOP/s",
                               "frac": a64 / FP64_PEAK_TFLOPS, "traffic": tr64, "traffic_source": tr64_src,
                               "kernel": product_kernel_name(d, T, "f64"), "launches_per_step": n64.value / steps64,
                               "avg_launch_ms": k64, "flop_per_launch": flop_per_launch}}
        res["fp64"] = side64
        del X64, C64, v64, w64
    if not args.no_cpu_baseline and args.op == "dmmv":
        full = args.workload == "C2" and not args.cpu_rows
        rows = args.cpu_rows or {"C2": N, "C3": 200_000, "C4": 100_000}[args.workload]
        time_rows = min(rows, {"C2": 200_000, "C3": 100_000, "C4": 50_000}[args.workload])

        def gpu_on(Xs, ws):
            if full and tdt == torch.float32 and side64 is not None:
                step()
                return out.clone(), out64                       # the timed steps' own results, all N rows
            Xd = Xs.to(dev)
            wd = ws.to(dev) if ws is not None else None
            r32 = kernel.dmmv(Xd, Cg, vg, wd)
            r64 = r32 if tdt == torch.float64 else kernel.dmmv(Xd.double(), Cg.double(), vg.double(),
                                                               wd.double() if wd is not None else None)
            return r32, r64

        res["cpu_baseline"] = cpu_baseline(X, C, sigma, v, w, gpu_on, rows, time_rows, 5 if full else 3, kernel_name)
        if side64 is not None:
            side64["rel_err_vs_cpu_f64"] = res["cpu_baseline"]["rel_err_gpu_f64_vs_cpu_f64"]
            side64["parity_rows"] = rows
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
