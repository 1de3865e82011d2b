"""Differentiable model-selection objectives for Nystroem kernel ridge regression.

The exact objectives of the reference (falkon/hopt/objectives/exact_objectives/{holdout,gcv,loocv,sgpr,compreg,
new_compreg}.py; base class falkon/hopt/objectives/objectives.py:11-66, transform transforms.py:6-38), restated on one
shared factorisation.  They are ``torch.nn.Module``s whose parameters are the kernel's differentiable parameters
(lengthscales; the kernel is a sub-module), optionally the centres and the penalty; ``forward(X, Y)`` returns the objective, whose gradient flows
through ``kernel(centres, X)`` and ``kernel(centres, centres)``: kernel matrices and their backward passes from the
MI355X kernels (falkon_amd/mmv_ops/fmm.py, fmmv_grad.py).

With v = penalty * n, K_mm = L L^T, A = L^-1 K_mn / sqrt(v), B = A A^T + I = L_B L_B^T and C = L_B^-1 A (m x n):
the hat matrix of the Nystroem estimator is H = C^T C, its coefficients are alpha = L^-T L_B^-T (C Y) / sqrt(v), and

    tr(H) = |C|_F^2,   diag(H) = column sums of C^2,   H Y = C^T (C Y),   Y^T (I - H) Y = |Y|^2 - |C Y|^2,
    1/2 log det(B) = sum(log(diag(L_B))),   tr(K_nn - Q_nn) = tr(K_nn) - v * tr(A A^T)   (Q_nn the Nystroem kernel).

``StochasticNystromCompReg`` (at the end) is the matrix-free counterpart of ``NystromCompReg``: trace estimators and
the Falkon solver on top of ``kernel.mmv`` and its backward pass.
"""
from typing import Dict, Optional

import torch
import torch.nn.functional as F

from ..kernels.diff_kernel import DiffKernel

__all__ = ("PositiveTransform", "HyperoptObjective", "HoldOut", "GCV", "LOOCV", "SGPR", "CompReg", "NystromCompReg",
           "StochasticNystromCompReg")


class PositiveTransform:
    """x -> softplus(x) + lower_bound, with a numerically careful inverse (falkon/hopt/objectives/transforms.py:6-38)."""

    def __init__(self, lower_bound: float = 0.0):
        self.lower_bound = lower_bound

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        return F.softplus(x) + self.lower_bound

    def inv(self, y: torch.Tensor) -> torch.Tensor:
        z = y - self.lower_bound
        # softplus^-1(z) = z + log(1 - exp(-z)); log(z) for tiny z and z itself for large z avoid the cancellation
        eps = torch.finfo(z.dtype).eps
        small, large = z < eps ** 0.5, z > -2 * torch.log(torch.tensor(eps, dtype=z.dtype))
        safe = torch.where(small | large, torch.ones_like(z), z)
        mid = safe + torch.log(-torch.expm1(-safe))
        return torch.where(small, torch.log(z), torch.where(large, z, mid))


class _Identity:
    def __call__(self, x):
        return x

    def inv(self, y):
        return y


def _jittered_cholesky(mat: torch.Tensor) -> torch.Tensor:
    """Lower Cholesky factor of ``mat + eps I`` for the smallest eps of a fixed ladder that makes it succeed
    (falkon/hopt/objectives/exact_objectives/utils.py:18-28)."""
    eye = torch.eye(mat.shape[0], device=mat.device, dtype=mat.dtype)
    for eps in (1e-8, 1e-6, 1e-5, 1e-4, 1e-3, 1e-2, 1e-1, 1e0):
        L, info = torch.linalg.cholesky_ex(mat + eye * eps)
        if int(info) == 0:
            return L
    raise RuntimeError("Cholesky failed even with a jitter of 1.0 on the diagonal")


class _Factors:
    """The shared factorisation (see the module docstring) for training data X, Y and variance v."""

    def __init__(self, kernel, centres, X, Y, variance):
        self.variance, self.root = variance, torch.sqrt(variance)
        kmn, kmm = kernel(centres, X), kernel(centres, centres)
        self.L = _jittered_cholesky(kmm)
        self.A = torch.linalg.solve_triangular(self.L, kmn, upper=False) / self.root
        self.AAT = self.A @ self.A.T
        self.LB = _jittered_cholesky(self.AAT + torch.eye(self.AAT.shape[0], device=X.device, dtype=X.dtype))
        self.C = torch.linalg.solve_triangular(self.LB, self.A, upper=False)
        self.CY = self.C @ Y

    def trace_hat(self):
        return self.C.square().sum()

    def residual_energy(self, Y):
        return Y.square().sum() - self.CY.square().sum()

    def fitted(self):
        return self.C.T @ self.CY

    def coefficients(self):
        inner = torch.linalg.solve_triangular(self.LB.T, self.CY, upper=True)
        return torch.linalg.solve_triangular(self.L.T, inner, upper=True) / self.root


class HyperoptObjective(torch.nn.Module):
    def __init__(self, kernel, centers_init: torch.Tensor, penalty_init: torch.Tensor, opt_centers: bool,
                 opt_penalty: bool, centers_transform=None, pen_transform=None):
        super().__init__()
        if not isinstance(kernel, DiffKernel):
            raise TypeError("Kernel must inherit from `DiffKernel` for hyperparameter optimization.")
        self.kernel = kernel
        self.centers_transform = centers_transform or _Identity()
        self.penalty_transform = pen_transform or PositiveTransform(1e-8)
        centers_init = self.centers_transform.inv(centers_init)
        penalty_init = self.penalty_transform.inv(penalty_init)
        for name, value, optimise in (("centers_", centers_init, opt_centers), ("penalty_", penalty_init, opt_penalty)):
            if optimise:
                self.register_parameter(name, torch.nn.Parameter(value))
            else:
                self.register_buffer(name, value)
        self.x_train = self.y_train = None
        self.losses: Optional[Dict[str, torch.Tensor]] = None

    @property
    def penalty(self):
        return self.penalty_transform(self.penalty_)

    @property
    def centers(self):
        return self.centers_transform(self.centers_)

    def _variance(self, n: int):
        return self.penalty * n

    def _factors(self, X, Y) -> _Factors:
        return _Factors(self.kernel, self.centers, X, Y, self._variance(X.shape[0]))

    def _remember(self, X, Y, **losses):
        self.x_train, self.y_train = X.detach(), Y.detach()
        self.losses = {k: v.detach() for k, v in losses.items()}

    def predict(self, X):
        if self.x_train is None or self.y_train is None:
            raise RuntimeError("Call forward at least once before calling predict.")
        with torch.no_grad():
            return self.kernel(X, self.centers) @ self._factors(self.x_train, self.y_train).coefficients()

    def __repr__(self):
        return (f"{type(self).__name__}(kernel={self.kernel}, penalty={float(self.penalty.detach()):.3e}, "
                f"num_centers={self.centers.shape[0]})")


class HoldOut(HyperoptObjective):
    """Mean squared error on a held-out part of the data of the estimator fitted on the rest (holdout.py:37-58)."""

    def __init__(self, kernel, centers_init, penalty_init, opt_centers, opt_penalty, val_pct: float,
                 per_iter_split: bool, centers_transform=None, pen_transform=None):
        super().__init__(kernel, centers_init, penalty_init, opt_centers, opt_penalty, centers_transform, pen_transform)
        self.val_pct, self.per_iter_split = val_pct, per_iter_split
        self.tr_indices = self.val_indices = None

    def forward(self, X, Y):
        if self.tr_indices is None or self.per_iter_split:
            order = torch.randperm(X.shape[0], device=X.device)
            num_val = int(X.shape[0] * self.val_pct)
            self.val_indices, self.tr_indices = order[:num_val], order[num_val:]
        alpha = self._factors(X[self.tr_indices], Y[self.tr_indices]).coefficients()
        loss = torch.mean((Y[self.val_indices] - self.kernel(X[self.val_indices], self.centers) @ alpha) ** 2)
        self._remember(X, Y, **{"hold-out": loss})
        return loss


class GCV(HyperoptObjective):
    """Generalised cross validation: mean squared residual over (1 - tr(H) / n)^2 (gcv.py:33-45)."""

    def forward(self, X, Y):
        f = self._factors(X, Y)
        loss = torch.mean((Y - f.fitted()) ** 2) / (1 - f.trace_hat() / X.shape[0]) ** 2
        self._remember(X, Y, GCV=loss)
        return loss


class LOOCV(HyperoptObjective):
    """Leave-one-out error in closed form, ((y_i - (H y)_i) / (1 - H_ii))^2 averaged, with v = penalty (n - 1)
    (loocv.py:33-46,61-75)."""

    def _variance(self, n: int):
        return self.penalty * (n - 1)

    def forward(self, X, Y):
        f = self._factors(X, Y)
        leverage = f.C.square().sum(0).reshape(-1, 1)
        loss = torch.mean(((Y - f.fitted()) / (1 - leverage)) ** 2)
        self._remember(X, Y, LOOCV=loss)
        return loss


class SGPR(HyperoptObjective):
    """Negative variational lower bound of the sparse Gaussian process with noise variance v (sgpr.py:31-45)."""

    def forward(self, X, Y):
        n = X.shape[0]
        f = self._factors(X, Y)
        log_det = torch.log(torch.diagonal(f.LB)).sum() + 0.5 * n * torch.log(f.variance)
        data_fit = 0.5 * f.residual_energy(Y) / f.variance
        trace = 0.5 * (self.kernel(X, X, diag=True).sum() / f.variance - torch.trace(f.AAT))
        self._remember(X, Y, log_det=log_det, data_fit=data_fit, trace=trace)
        return log_det + data_fit + trace


class CompReg(HyperoptObjective):
    """Effective dimension plus data fit: tr(H) + Y^T (I - H) Y (compreg.py:30-39)."""

    def forward(self, X, Y):
        f = self._factors(X, Y)
        deff, data_fit = f.trace_hat(), f.residual_energy(Y)
        self._remember(X, Y, **{"d_eff": deff, "data_fit": data_fit})
        return deff + data_fit


class NystromCompReg(HyperoptObjective):
    """CompReg plus the Nystroem approximation's trace penalty, tr(K_nn - Q_nn) * datafit / (v n)
    (new_compreg.py:31-44)."""

    def forward(self, X, Y):
        f = self._factors(X, Y)
        deff, data_fit = f.trace_hat(), f.residual_energy(Y)
        gap = self.kernel(X, X, diag=True).sum() - f.variance * torch.trace(f.AAT)
        trace = gap * data_fit / (f.variance * X.shape[0])
        self._remember(X, Y, **{"d_eff": deff, "data_fit": data_fit, "trace": trace})
        return deff + data_fit + trace


class StochasticNystromCompReg(HyperoptObjective):
    r"""``NystromCompReg`` without any n x m matrix: traces by Hutchinson's estimator, linear systems by the Falkon solver,
    every kernel product a ``kernel.mmv`` (the reference's objective of the same name,
    falkon/hopt/objectives/stoch_objectives/stoch_new_compreg.py:21-505, which hand-writes the backward pass).

    With S = (K_mn K_nm + v K_mm)^-1, random vectors Z (n x t, standard normal) and ZY = [Z, Y]:

        tr(H) ~ 1/t sum_j z_j^T K_nm S K_mn z_j,      Y^T (I - H) Y = |Y|^2 - Y^T K_nm S K_mn Y,
        tr(Q_nn) ~ 1/t sum_j |L^-1 K_mn z_j|^2         (K_mm = L L^T).

    The quadratic forms ``b^T S b`` (b = K_mn z, depending on the hyperparameters through K_mn and S) are differentiated
    without differentiating the solver: with u = S b from the Falkon solver held fixed,
    ``2 u^T b - u^T (K_mn K_nm + v K_mm) u`` has the value and the gradient of ``b^T S b`` at the current
    hyperparameters, and its pieces are kernel-vector products whose backward pass is the MI355X one
    (falkon_amd/mmv_ops/fmmv_grad.py).  The solver runs ``flk_maxiter`` iterations to ``flk_opt.cg_tolerance``."""

    def __init__(self, kernel, centers_init, penalty_init, opt_centers: bool, opt_penalty: bool, flk_opt=None,
                 flk_maxiter: int = 10, num_trace_est: int = 20, centers_transform=None, pen_transform=None):
        super().__init__(kernel, centers_init, penalty_init, opt_centers, opt_penalty, centers_transform, pen_transform)
        from ..options import FalkonOptions
        self.flk_opt = flk_opt or FalkonOptions()
        self.flk_maxiter, self.num_trace_est = flk_maxiter, num_trace_est
        self.trace_vectors: Optional[torch.Tensor] = None    # fixed Z (n x t) instead of a fresh draw per call

    def _solve(self, X, centres, rhs, penalty: float) -> torch.Tensor:
        """(K_mn K_nm + penalty n K_mm)^-1 K_mn rhs with the preconditioned CG of the estimator."""
        from ..optim import FalkonConjugateGradient
        from ..preconditioner import FalkonPreconditioner
        kernel = self.kernel.detach()                          # the solver is not differentiated
        with torch.inference_mode():
            precond = FalkonPreconditioner(penalty, kernel, self.flk_opt)
            precond.init(centres)
            solver = FalkonConjugateGradient(kernel, precond, self.flk_opt)
            coeff = precond.apply(solver.solve(X, centres, rhs, penalty, None, self.flk_maxiter))
        return coeff.clone()                                   # an ordinary tensor, usable in the graph below

    def forward(self, X, Y):
        n, t = X.shape[0], self.num_trace_est
        Z = self.trace_vectors if self.trace_vectors is not None else torch.randn(n, t, dtype=X.dtype, device=X.device)
        t = Z.shape[1]
        ZY = torch.cat([Z, Y], dim=1)
        centres, variance = self.centers, self.penalty * n
        U = self._solve(X.detach(), centres.detach(), ZY, float(self.penalty.detach()))
        B = self.kernel.mmv(centres, X, ZY)                    # K_mn [Z, Y], differentiable
        KU = self.kernel.mmv(X, centres, U)                    # K_nm U
        kmm = self.kernel(centres, centres)
        quad = 2 * (U * B).sum(0) - KU.square().sum(0) - variance * (U * (kmm @ U)).sum(0)
        deff = quad[:t].sum() / t
        data_fit = Y.square().sum() - quad[t:].sum()
        half = torch.linalg.solve_triangular(_jittered_cholesky(kmm), B[:, :t], upper=False)
        gap = self.kernel(X, X, diag=True).sum() - half.square().sum() / t
        trace = gap * data_fit / (variance * n)
        self._remember(X, Y, **{"d_eff": deff, "data_fit": data_fit, "trace": trace})
        return deff + data_fit + trace

    def predict(self, X):
        if self.x_train is None or self.y_train is None:
            raise RuntimeError("Call forward at least once before calling predict.")
        with torch.no_grad():
            alpha = self._solve(self.x_train, self.centers.detach(), self.y_train, float(self.penalty.detach()))
            return self.kernel.detach().mmv(X, self.centers.detach(), alpha)
