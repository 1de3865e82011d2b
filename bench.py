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

WORKLOADS = {
    # name: (seed, N, d, M, T, has_w)
    "C2": (1002, 1_000_000, 28, 20_000, 1, True),
    "C3": (1003, 10_000_000, 9, 50_000, 1, False),
    "C4": (1004, 500_000, 784, 10_000, 10, True),
}

# HBM bytes per launch of the product kernel, keyed by workload: rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE
# (KiB per dispatch, mean over the launches of the kernel) scaled by what the same counters read for a plain
# 1 GiB device copy (FETCH_SIZE reads half the true bytes on this box: factor 2.0; WRITE_SIZE factor 1.0).
# The summaries are under profiles/.  None where it has not been measured.
MEASURED_TRAFFIC_BYTES = {
    "C2": int((73470.7 * 2.0 + 17773.4 * 1.0) * 1024),     # 168.7 MB; algorithmic: packed X 112 MB + C + vectors
    "C4": int((2.61207e7 * 2.0) * 1024),                   # 53.5 GB (reads only; tiles are re-read from L2/MALL/HBM)
}


def make_inputs(name):
    """Synthetic inputs of the named configuration (draw order X, idx, sigma, v, w)."""
    seed, N, d, M, T, has_w = WORKLOADS[name]
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


def cpu_baseline(X, C, sigma, v, w, gpu_out_fn, rows):
    """Reference-equivalent CPU path (the oracle restatement, torch CPU ops) on the first `rows` rows."""
    from oracle import mmv_ref                      # checker only; never on the product path
    Xs = X[:rows].contiguous()
    ws = w[:rows].contiguous() if w is not None else None
    mmv_ref.fdmmv_ref(Xs[:2000], C, v, ws[:2000] if ws is not None else None, sigma, max_cpu_mem=4 * 2**30)  # warm-up
    t0 = time.perf_counter()
    exp = mmv_ref.fdmmv_ref(Xs, C, v, ws, sigma, max_cpu_mem=4 * 2**30)
    dt = time.perf_counter() - t0
    got, got64 = gpu_out_fn(Xs, ws)
    got, got64, exp = got.double().cpu(), got64.double().cpu(), exp.double()

    def rel(a, b):
        return float(((a - b).norm(dim=0) / b.norm(dim=0)).max())

    M, T = v.shape
    return {"value": rows * M * T / dt, "unit": "kernel entries/s", "cores": torch.get_num_threads(),
            "kind": "port", "host_cpus": os.cpu_count(),
            "sample": f"first {rows} rows of X with the full M={M} (dfmmv is linear in N), "
                      f"max_cpu_mem=4GiB, {dt:.2f} s",
            # fp64 anchor = the same product in fp64 on the same fp32-valued inputs (GPU fp64 kernel)
            "rel_err_gpu_f32_vs_cpu_f32": rel(got, exp), "rel_err_gpu_f32_vs_f64": rel(got, got64),
            "rel_err_cpu_f32_vs_f64": rel(exp, got64)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="C2", choices=sorted(WORKLOADS))
    ap.add_argument("--dtype", default="f32", choices=["f32", "f64"], help="arithmetic type (the headline is f32)")
    ap.add_argument("--op", default="dmmv", choices=["dmmv", "mmv"],
                    help="dmmv = K^T(Kv+w), the headline; mmv = K v only (one launch per step)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=0)
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="BYTES",
                    help="only run a plain device copy of BYTES bytes five times (reference point for the "
                         "FETCH_SIZE / WRITE_SIZE counters) and exit")
    args = ap.parse_args()
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

    from falkon_amd import GaussianKernel, _backend
    lib = _backend.load()                            # raises if the HIP library is missing
    dev = torch.device("cuda:0")
    seed, N, d, M, T, has_w = WORKLOADS[args.workload]
    X, C, sigma, v, w = make_inputs(args.workload)
    tdt = torch.float32 if args.dtype == "f32" else torch.float64
    X, C, v = X.to(tdt), C.to(tdt), v.to(tdt)
    w = w.to(tdt) if w is not None else None
    peak = FP32_PEAK_TFLOPS if args.dtype == "f32" else FP64_PEAK_TFLOPS
    Xg, Cg, vg = X.to(dev), C.to(dev), v.to(dev)
    wg = w.to(dev) if w is not None else None
    kernel = GaussianKernel(sigma)
    out = torch.empty(M if args.op == "dmmv" else N, T, dtype=tdt, device=dev)

    def step():
        if args.op == "dmmv":
            kernel.dmmv(Xg, Cg, vg, wg, out=out)
        else:
            kernel.mmv(Xg, Cg, vg, out=out)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    lib.flk_kernel_timing_enable(1)                  # HIP events around each product-kernel launch, on its stream
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    tot_ms, launches = ctypes.c_double(), ctypes.c_int64()
    rc = lib.flk_kernel_timing_read(ctypes.byref(tot_ms), ctypes.byref(launches))
    _backend.raise_for_status(rc, "flk_kernel_timing_read")
    lib.flk_kernel_timing_enable(0)

    ms_per_step = elapsed / args.steps * 1e3
    value = N * M * T / (elapsed / args.steps)
    # one launch of the product kernel evaluates all N*M pairs once: (2d+4) flop per kernel value + 2T to contract
    flop_per_launch = N * M * (2 * d + 4 + 2 * T)
    kern_ms = tot_ms.value / max(launches.value, 1)
    achieved = flop_per_launch / (kern_ms * 1e-3) / 1e12
    res = {
        "metric": f"{'dfmmv' if args.op == 'dmmv' else 'fmmv'} kernel-entries/sec (N*M*T/s) {'fp32' if args.dtype == 'f32' else 'fp64'}, 1 MI355X",
        "value": value, "unit": "kernel entries/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": f"{args.workload}: Gaussian {'dfmmv K^T(Kv+w)' if args.op == 'dmmv' else 'fmmv K v'}, N={N}, d={d}, M={M}, T={T}, "
                               f"{ {'C2': 'sigma=3.8', 'C3': 'per-dimension sigma', 'C4': 'sigma=10'}[args.workload] }, "
                               f"{'fp32' if args.dtype == 'f32' else 'fp64'}, "
                               f"inputs resident in HBM, packing included in every step"},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
                     "frac": achieved / peak,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload) if args.dtype == "f32" else None,
                     "kernel": ("mmv_large_kernel" if d > 64 else "mmv_small_%s_kernel" % args.dtype),
                     "launches_per_step": launches.value / args.steps,
                     "avg_launch_ms": kern_ms, "flop_per_launch": flop_per_launch},
        "whole_step_flop_frac": (N * M * ((2 if args.op == "dmmv" else 1) * (2 * d + 4 + 2 * T)))
                                / (elapsed / args.steps) / 1e12 / peak,
    }
    if not args.no_cpu_baseline and args.op == "dmmv":
        rows = args.cpu_rows or {"C2": N, "C3": 400_000, "C4": 100_000}[args.workload]

        def gpu_on(Xs, ws):
            Xd = Xs.to(dev)
            wd = ws.to(dev) if ws is not None else None
            r32 = kernel.dmmv(Xd, Cg, vg, wd)
            r64 = r32 if tdt == torch.float64 else kernel.dmmv(Xd.double(), Cg.double(), vg.double(),
                                                               wd.double() if wd is not None else None)
            return r32, r64

        res["cpu_baseline"] = cpu_baseline(X, C, sigma, v, w, gpu_on, rows)
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
