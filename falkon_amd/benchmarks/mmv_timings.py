"""Timing sweep of ``GaussianKernel.mmv`` over N and over D, on one MI355X.

The sweep is the reference's own benchmark of this path (falkon/benchmarks/timing_benchmarks/mmv_timings.py:53-127):
fp32, ``GaussianKernel(3.0)``, M = 20 000 centres, T = 10 right-hand sides; N from 1 000 to 1e8 at D = 10, and D from 10
to 10 000 at N = 20 000.  As there, the matrices are standard normal, live in HOST memory, the output is allocated by
the call, and a repetition is timed from the call to the end of ``torch.cuda.synchronize()`` (best of ``--reps``): the
figures include the upload of X1, X2 and v and the download of the result.  ``--resident`` adds the same calls with
the inputs already on the GPU.

    python -m falkon_amd.benchmarks.mmv_timings [--max-n 100000000] [--max-d 10000] [--reps 5] [--resident]

prints one JSON line per experiment: ``{"exp": ..., "N": ..., "D": ..., "M": ..., "T": ..., "seconds": ...,
"entries_per_s": N*M*T/seconds}``.
"""
import argparse
import json
import time

import torch

from .. import FalkonOptions, GaussianKernel

N_SWEEP = [1_000, 5_000, 20_000, 50_000, 100_000, 200_000, 400_000, 600_000, 1_000_000, 2_000_000, 10_000_000,
           50_000_000, 100_000_000]
D_SWEEP = [10, 50, 100, 250, 500, 750, 1_000, 1_250, 1_500, 2_000, 2_500, 3_000, 4_000, 5_000, 7_000, 10_000]
DEFAULT_N, DEFAULT_M, DEFAULT_D, DEFAULT_T = 20_000, 20_000, 10, 10


def _data(n, m, d, t, generator):
    return (torch.randn(n, d, dtype=torch.float32, generator=generator),
            torch.randn(m, d, dtype=torch.float32, generator=generator),
            torch.randn(m, t, dtype=torch.float32, generator=generator))


def _best_of(fn, reps):
    best = float("inf")
    for _ in range(reps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        best = min(best, time.perf_counter() - t0)
    return best


def run(max_n, max_d, reps, resident, bf16x3):
    kernel = GaussianKernel(3.0, opt=FalkonOptions(bf16x3_cross_term=bf16x3))
    gen = torch.Generator().manual_seed(0)
    cases = [("varying N", n, DEFAULT_D) for n in N_SWEEP if n <= max_n]
    cases += [("varying D", DEFAULT_N, d) for d in D_SWEEP if d <= max_d]
    for exp, n, d in cases:
        X1, X2, v = _data(n, DEFAULT_M, d, DEFAULT_T, gen)
        kernel.mmv(X1, X2, v)                                   # first call: library load, allocator warm-up
        rec = {"exp": exp + (" (bf16x3 cross term)" if bf16x3 else ""), "N": n, "D": d, "M": DEFAULT_M, "T": DEFAULT_T,
               "seconds": _best_of(lambda: kernel.mmv(X1, X2, v), reps)}
        rec["entries_per_s"] = n * DEFAULT_M * DEFAULT_T / rec["seconds"]
        if resident:
            Xg, Cg, vg = X1.cuda(), X2.cuda(), v.cuda()
            rec["seconds_resident"] = _best_of(lambda: kernel.mmv(Xg, Cg, vg), reps)
            del Xg, Cg, vg
        print(json.dumps(rec), flush=True)
        del X1, X2, v
        torch.cuda.empty_cache()


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--max-n", type=int, default=N_SWEEP[-1])
    ap.add_argument("--max-d", type=int, default=D_SWEEP[-1])
    ap.add_argument("--reps", type=int, default=5)
    ap.add_argument("--resident", action="store_true", help="also time the calls with the inputs on the GPU")
    ap.add_argument("--bf16x3", action="store_true", help="FalkonOptions(bf16x3_cross_term=True)")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("mmv_timings: no GPU visible")
    run(args.max_n, args.max_d, args.reps, args.resident, args.bf16x3)


if __name__ == "__main__":
    main()
