"""Conjugate gradient solvers: the callers of ``dmmv`` (falkon/optim/conjgrad.py:42-306)."""
import functools
import time
from typing import Callable, Optional

import torch

from .options import ConjugateGradientOptions, FalkonOptions

__all__ = ("ConjugateGradient", "FalkonConjugateGradient", "StopOptimizationException")


class StopOptimizationException(Exception):
    def __init__(self, message):
        super().__init__()
        self.message = message


class ConjugateGradient:
    """Multi right-hand-side CG on ``A X = B`` with ``A`` given as a product callback
    (falkon/optim/conjgrad.py:53-185; differential convergence is not carried over)."""

    def __init__(self, opt: Optional[ConjugateGradientOptions] = None):
        self.params = opt or ConjugateGradientOptions()
        self.num_iter = None

    def solve(self, X0: Optional[torch.Tensor], B: torch.Tensor, mmv: Callable[[torch.Tensor], torch.Tensor],
              max_iter: int, callback: Optional[Callable[[int, torch.Tensor, float], None]] = None) -> torch.Tensor:
        t0 = time.time()
        if X0 is None:
            R = B.clone()
            X = torch.zeros_like(B)
        else:
            R = B - mmv(X0)
            X = X0
        eps = self.params.cg_epsilon(X.dtype)
        full_grad_every = self.params.cg_full_gradient_every or max_iter * 2
        tol = self.params.cg_tolerance ** 2
        P = R.clone()
        rs_old = R.square().sum(dim=0)
        e_train = time.time() - t0
        for self.num_iter in range(max_iter):
            t0 = time.time()
            AP = mmv(P)
            alpha = rs_old / (torch.sum(P * AP, dim=0).add_(eps))
            X.addcmul_(P, alpha.reshape(1, -1))
            if (self.num_iter + 1) % full_grad_every == 0:
                if X.is_cuda:
                    torch.cuda.synchronize()
                R = B - mmv(X)
            else:
                R.addcmul_(AP, alpha.reshape(1, -1), value=-1.0)
            rs_new = R.square().sum(dim=0)
            if torch.all(rs_new < tol):
                break
            P = P.mul_((rs_new / rs_old.add_(eps)).reshape(1, -1)).add_(R)
            rs_old = rs_new
            e_train += time.time() - t0
            if callback is not None:
                try:
                    callback(self.num_iter + 1, X, e_train)
                except StopOptimizationException as e:
                    print(f"Optimization stopped from callback: {e.message}")
                    break
        return X


class FalkonConjugateGradient:
    r"""Preconditioned CG on ``B^T (K_nm^T K_nm + lambda n K_mm) B beta = B^T K_nm^T y / n`` with
    ``B = 1/sqrt(n) T^-1 A^-1`` (falkon/optim/conjgrad.py:187-306).  One ``kernel.dmmv`` per iteration."""

    def __init__(self, kernel, preconditioner, opt: FalkonOptions, weight_fn=None):
        if weight_fn is not None:
            raise NotImplementedError("weighted least squares is not part of this build")
        self.kernel, self.preconditioner, self.params = kernel, preconditioner, opt
        self.optimizer = ConjugateGradient(ConjugateGradientOptions(
            cg_epsilon_32=opt.cg_epsilon_32, cg_epsilon_64=opt.cg_epsilon_64, cg_tolerance=opt.cg_tolerance,
            cg_full_gradient_every=opt.cg_full_gradient_every,
            cg_differential_convergence=opt.cg_differential_convergence))

    def falkon_mmv(self, sol, penalty, X, M, n: int):
        prec = self.preconditioner
        v = prec.invA(sol)
        v_t = prec.invT(v)
        cc = self.kernel.dmmv(X, M, v_t, None, opt=self.params)      # K_nm^T (K_nm v_t): the hot call
        cc_ = prec.invTt(cc.div_(n)).add_(v.mul_(penalty))
        return prec.invAt(cc_)

    def solve(self, X, M, Y, _lambda, initial_solution, max_iter, callback=None):
        if not torch.is_inference_mode_enabled():
            raise RuntimeError("FalkonConjugateGradient.solve must run under torch.inference_mode()")
        n = Y.size(0)
        y_over_n = Y / n
        B = self.kernel.mmv(M, X, y_over_n, opt=self.params)          # K_nm^T y / n
        B = self.preconditioner.apply_t(B)
        mmv = functools.partial(self.falkon_mmv, penalty=_lambda, X=X, M=M, n=n)
        return self.optimizer.solve(initial_solution, B, mmv, max_iter, callback)
