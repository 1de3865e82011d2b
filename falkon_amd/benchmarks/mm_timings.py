"""Timing of the explicit kernel matrix ``GaussianKernel(5.0)(A, A)`` on one MI355X.

The reference's benchmark of this call (falkon/benchmarks/timing_benchmarks/mm_timings.py:19-48): A is
50 000 x 256, fp32, standard normal, in pinned HOST memory; the 50 000 x 50 000 result (10 GB) is allocated by the
call, in host memory as the data is, so a repetition (call to the end of ``torch.cuda.synchronize()``, best of
``--reps``) includes the download of K; once with ``no_single_kernel=True`` (kernel values computed in fp64 and
rounded once, the reference's default for the preconditioner) and once in plain fp32.  ``--resident`` adds the same
calls with A on the GPU (the result then stays on the GPU).

    python -m falkon_amd.benchmarks.mm_timings [--n 50000] [--d 256] [--reps 5] [--resident]

prints one JSON line per setting.
"""
import argparse
import json
import time

import torch

from .. import FalkonOptions, GaussianKernel


def _best_of(fn, reps):
    best = float("inf")
    for _ in range(reps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = fn()
        torch.cuda.synchronize()
        best = min(best, time.perf_counter() - t0)
        del out
    return best


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--n", type=int, default=50_000)
    ap.add_argument("--d", type=int, default=256)
    ap.add_argument("--reps", type=int, default=5)
    ap.add_argument("--resident", action="store_true", help="also time the call with A (and the result) on the GPU")
    ap.add_argument("--bf16x3", action="store_true",
                    help="FalkonOptions(bf16x3_cross_term=True): serves the fp32 evaluation beyond 64 features")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("mm_timings: no GPU visible")
    A = torch.randn(args.n, args.d, dtype=torch.float32, generator=torch.Generator().manual_seed(0)).pin_memory()
    for no_single_kernel in (True, False):
        kernel = GaussianKernel(5.0, opt=FalkonOptions(no_single_kernel=no_single_kernel,
                                                       bf16x3_cross_term=args.bf16x3))
        kernel(A[:1000], A[:1000])                           # first call: library load
        rec = {"exp": "kernel matrix" + (" (bf16x3 cross term)" if args.bf16x3 else ""), "N": args.n, "D": args.d, "no_single_kernel": no_single_kernel,
               "seconds": _best_of(lambda: kernel(A, A), args.reps)}
        if args.resident:
            Ag = A.cuda()
            rec["seconds_resident"] = _best_of(lambda: kernel(Ag, Ag), args.reps)
            del Ag
        print(json.dumps(rec), flush=True)
        torch.cuda.empty_cache()


if __name__ == "__main__":
    main()
