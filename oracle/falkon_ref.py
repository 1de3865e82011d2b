"""Reference-equivalent CPU restatement of the callers of the hot path (test infrastructure only).

``falkon_fit_ref`` follows ``Falkon.fit`` (falkon/models/falkon.py:205-298) for dense host data:
preconditioner ``T = chol(K_MM + eps*M*I)``, ``A = chol(T T^T / M + lambda*I)``
(falkon/preconditioner/flk_preconditioner.py:94-155, K_MM computed in fp64 and stored in the data
dtype, falkon/mmv_ops/fmm.py:619-622), then the preconditioned conjugate gradient of
falkon/optim/conjgrad.py:53-185,242-306 whose products are the CPU oracle's ``fmmv_ref`` /
``fdmmv_ref``.  Linear algebra is scipy LAPACK, as on the reference's CPU path
(falkon/preconditioner/pc_utils.py:61-80, falkon/la_helpers/cpu_trsm.py).
"""
from typing import Optional

import numpy as np
import scipy.linalg as sla
import torch

from .gaussian_ref import rbf_core_ref, validate_sigma_ref
from .mmv_ref import fdmmv_ref, fmmv_ref

PC_EPS = {torch.float32: 1e-5, torch.float64: 1e-13}      # falkon/options.py:257-258
CG_EPS = {torch.float32: 1e-7, torch.float64: 1e-15}      # falkon/options.py:223-224


class PrecondRef:
    def __init__(self, centers: torch.Tensor, sigma, penalty: float):
        dt = centers.dtype
        M = centers.shape[0]
        K = rbf_core_ref(centers.double(), centers.double(), None, sigma).to(dt).numpy()
        K[np.diag_indices(M)] += PC_EPS[dt] * M
        self.T = sla.cholesky(K, lower=False)                     # K = T^T T
        G = (self.T @ self.T.T) / M
        G[np.diag_indices(M)] += penalty
        self.A = sla.cholesky(G, lower=False)                     # G = A^T A
        self.dt = dt

    def _solve(self, R, v, trans):
        return torch.from_numpy(sla.solve_triangular(R, v.numpy(), lower=False, trans=trans))

    def invA(self, v): return self._solve(self.A, v, 0)
    def invAt(self, v): return self._solve(self.A, v, 1)
    def invT(self, v): return self._solve(self.T, v, 0)
    def invTt(self, v): return self._solve(self.T, v, 1)
    def apply(self, v): return self.invT(self.invA(v))
    def apply_t(self, v): return self.invAt(self.invTt(v))


def falkon_fit_ref(X: torch.Tensor, Y: torch.Tensor, centers: torch.Tensor, sigma, penalty: float, maxiter: int,
                   cg_tolerance: float = 1e-7, full_gradient_every: int = 10,
                   max_cpu_mem: float = 4 * 2**30) -> torch.Tensor:
    """Returns alpha (M x T).  ``centers`` are given (selection is a separate, trivially seeded step)."""
    sigma = validate_sigma_ref(sigma)
    if Y.dim() == 1:
        Y = Y.unsqueeze(1)
    n = Y.shape[0]
    prec = PrecondRef(centers, sigma, penalty)
    eps = CG_EPS[X.dtype]

    def falkon_mmv(sol):
        v = prec.invA(sol)
        v_t = prec.invT(v)
        cc = fdmmv_ref(X, centers, v_t, None, sigma, max_cpu_mem=max_cpu_mem)
        return prec.invAt(prec.invTt(cc / n) + penalty * v)

    B = prec.apply_t(fmmv_ref(centers, X, Y / n, sigma, max_cpu_mem=max_cpu_mem))
    R = B.clone()
    beta = torch.zeros_like(B)
    P = R.clone()
    rs_old = R.square().sum(0)
    for it in range(maxiter):
        AP = falkon_mmv(P)
        alpha = rs_old / ((P * AP).sum(0) + eps)
        beta += P * alpha
        if (it + 1) % full_gradient_every == 0:
            R = B - falkon_mmv(beta)
        else:
            R -= AP * alpha
        rs_new = R.square().sum(0)
        if bool((rs_new < cg_tolerance**2).all()):
            break
        P = P * (rs_new / (rs_old + eps)) + R
        rs_old = rs_new
    return prec.apply(beta)


def falkon_predict_ref(X: torch.Tensor, centers: torch.Tensor, alpha: torch.Tensor, sigma,
                       max_cpu_mem: float = 4 * 2**30) -> torch.Tensor:
    """falkon/models/falkon.py:300-312: one kernel-vector product."""
    return fmmv_ref(X, centers, alpha, validate_sigma_ref(sigma), max_cpu_mem=max_cpu_mem)


def nystrom_krr_direct(X, Y, centers, sigma, penalty, kernel_name: str = "gaussian") -> np.ndarray:
    """The linear system Falkon solves, in closed form and fp64:
    alpha = (K_nm^T K_nm + lambda n K_mm)^-1 K_nm^T y  (falkon/tests/test_conjgrad.py:100-118)."""
    from .gaussian_ref import core_ref_for
    s = validate_sigma_ref(sigma)
    core = core_ref_for(kernel_name)
    Knm = core(X.double(), centers.double(), None, s).numpy()
    Kmm = core(centers.double(), centers.double(), None, s).numpy()
    Yn = Y.double().numpy().reshape(X.shape[0], -1)
    return np.linalg.solve(Knm.T @ Knm + penalty * X.shape[0] * Kmm, Knm.T @ Yn)
