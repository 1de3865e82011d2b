"""Writes tests/golden/gaussian_products.npz: small input/expected-output vectors for fmmv / fdmmv.

The reference repository holds no golden files for this path (its tests regenerate inputs from seeds
and compare with a naive kernel).  These vectors are therefore produced by THIS repository's
brute-force witness (oracle/brute.py: closed form, fp64 difference form), on the reference's own
test fixture (falkon/tests/test_kernels.py:32-71: n=20, m=5, d=3, t=2, seeds 92..95) for a scalar and
a per-dimension sigma.  They freeze the numbers so that a later change to the oracle or the kernels
that moves them is noticed.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import brute, inputs  # noqa: E402


def main():
    A, B, v, w = inputs.reference_test_mats(20, 5, 3, 2, np.float64)
    out = {"A": A.numpy(), "B": B.numpy(), "v": v.numpy(), "w": w.numpy()}
    for name, sigma in (("iso", torch.tensor([3.0])), ("diag", torch.tensor([0.7, 2.0, 5.0]))):
        out[f"sigma_{name}"] = sigma.numpy()
        out[f"K_{name}"] = brute.gaussian_brute(A, B, sigma)
        out[f"mmv_{name}"] = brute.mmv_brute(A, B, sigma, v)
        out[f"dmmv_{name}"] = brute.dmmv_brute(A, B, sigma, v, w)
        out[f"dmmv_now_{name}"] = brute.dmmv_brute(A, B, sigma, v, None)
    np.savez(os.path.join(os.path.dirname(os.path.abspath(__file__)), "gaussian_products.npz"), **out)


if __name__ == "__main__":
    main()
