"""Committed vectors (tests/golden/gaussian_products.npz, written by tests/golden/make_golden.py)."""
import os

import numpy as np
import pytest
import torch

from falkon_amd import GaussianKernel
from oracle import brute_c, gaussian_ref, mmv_ref

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gaussian_products.npz"))


@pytest.mark.parametrize("name", ["iso", "diag"])
def test_oracle_matches_golden(name):
    A, B, v, w = (torch.from_numpy(G[k]) for k in ("A", "B", "v", "w"))
    sigma = torch.from_numpy(G[f"sigma_{name}"])
    np.testing.assert_allclose(gaussian_ref.rbf_core_ref(A, B, None, sigma).numpy(), G[f"K_{name}"], rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(mmv_ref.fmmv_ref(A, B, v, sigma).numpy(), G[f"mmv_{name}"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(mmv_ref.fdmmv_ref(A, B, v, w, sigma).numpy(), G[f"dmmv_{name}"], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(mmv_ref.fdmmv_ref(A, B, v, None, sigma).numpy(), G[f"dmmv_now_{name}"], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(brute_c.dmmv_brute_c(A, B, sigma, v, w), G[f"dmmv_{name}"], rtol=1e-13, atol=1e-13)
    # the stored K has the textbook properties: entries in (0, 1], matches exp(-d^2/2) of one pair
    K = G[f"K_{name}"]
    s = G[f"sigma_{name}"] if G[f"sigma_{name}"].size > 1 else np.full(3, G[f"sigma_{name}"][0])
    assert 0 < K.min() and K.max() <= 1
    assert abs(K[3, 2] - np.exp(-0.5 * (((G["A"][3] - G["B"][2]) / s) ** 2).sum())) < 1e-15


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["iso", "diag"])
@pytest.mark.parametrize("dtype,tol", [(torch.float64, 1e-11), (torch.float32, 1e-5)])
def test_gpu_matches_golden(dev, name, dtype, tol):
    A, B, v, w = (torch.from_numpy(G[k]).to(dtype).to(dev) for k in ("A", "B", "v", "w"))
    k = GaussianKernel(torch.from_numpy(G[f"sigma_{name}"]))
    np.testing.assert_allclose(k.mmv(A, B, v).double().cpu().numpy(), G[f"mmv_{name}"], rtol=tol, atol=tol)
    np.testing.assert_allclose(k.dmmv(A, B, v, w).double().cpu().numpy(), G[f"dmmv_{name}"], rtol=tol * 10, atol=tol * 10)
    np.testing.assert_allclose(k.dmmv(A, B, v, None).double().cpu().numpy(), G[f"dmmv_now_{name}"], rtol=tol * 10, atol=tol * 10)
