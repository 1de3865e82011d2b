"""Falkon's two-Cholesky Nystroem preconditioner on torch-ROCm linear algebra.

Same algebra as falkon/preconditioner/flk_preconditioner.py:94-300: with K_MM the kernel matrix of
the centres, ``T = chol(K_MM + eps*M*I)`` (upper, K = T^T T) and ``A = chol(T T^T / M + lambda*I)``
(upper); the preconditioner is ``B = 1/sqrt(n) T^-1 A^-1``.  The reference runs this on its own
out-of-core Cholesky/LAUUM; here the factorisations are ``torch.linalg.cholesky`` and the solves
``torch.linalg.solve_triangular`` on the GPU (the caller side of the hot path, not accelerated).
"""
from typing import Optional

import torch

from .options import FalkonOptions

__all__ = ("FalkonPreconditioner",)


class FalkonPreconditioner:
    def __init__(self, penalty: float, kernel, opt: Optional[FalkonOptions] = None):
        self.params = opt if opt is not None else FalkonOptions()
        self._lambda = penalty
        self.kernel = kernel
        self.LT: Optional[torch.Tensor] = None   # lower factor of K_MM + eps*M*I  (T = LT^T)
        self.LA: Optional[torch.Tensor] = None   # lower factor of T T^T / M + lambda*I  (A = LA^T)

    def init(self, X: torch.Tensor, weight_vec: Optional[torch.Tensor] = None) -> None:
        if weight_vec is not None:
            raise NotImplementedError("weighted least squares is not part of this build")
        M = X.shape[0]
        with torch.inference_mode():
            C = self.kernel(X, X, opt=self.params)                     # fp64-computed when no_single_kernel
            eps = self.params.pc_epsilon(C.dtype)
            C.diagonal().add_(eps * M)
            LT = torch.linalg.cholesky(C)
            del C
            G = LT.T @ LT                                               # T T^T
            G.mul_(1.0 / M)
            G.diagonal().add_(self._lambda)
            self.LA = torch.linalg.cholesky(G)
            self.LT = LT

    def _check(self):
        if self.LT is None or self.LA is None:
            raise RuntimeError("FALKON preconditioner is not initialized. Please run `init` before any other "
                               "method on the preconditioner.")

    def to(self, device):
        if self.LT is not None:
            self.LT, self.LA = self.LT.to(device), self.LA.to(device)
        return self

    def invA(self, v):
        self._check()
        return torch.linalg.solve_triangular(self.LA.T, v, upper=True)

    def invAt(self, v):
        self._check()
        return torch.linalg.solve_triangular(self.LA, v, upper=False)

    def invT(self, v):
        self._check()
        return torch.linalg.solve_triangular(self.LT.T, v, upper=True)

    def invTt(self, v):
        self._check()
        return torch.linalg.solve_triangular(self.LT, v, upper=False)

    def apply(self, v):
        """T^-1 A^-1 v: preconditioned solution -> kernel coefficients."""
        return self.invT(self.invA(v))

    def apply_t(self, v):
        """A^-T T^-T v."""
        return self.invAt(self.invTt(v))
