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
    """Conjugate gradient on ``A X = B`` for several right-hand sides at once (one column each, with its own
    step lengths), ``A`` given as a product callback.  Same iteration, constants and stopping rule as
    falkon/optim/conjgrad.py:53-185: ``eps`` guards the two divisions, the residual is recomputed from scratch
    every ``cg_full_gradient_every`` iterations, and the solve stops once every column has
    ``|r|^2 < cg_tolerance^2``.  Differential convergence is not carried over."""

    def __init__(self, opt: Optional[ConjugateGradientOptions] = None):
        self.params = opt if opt is not None else ConjugateGradientOptions()
        self.num_iter = None

    def solve(self, X0: Optional[torch.Tensor], B: torch.Tensor, mmv: Callable[[torch.Tensor], torch.Tensor],
              max_iter: int, callback: Optional[Callable[[int, torch.Tensor, float], None]] = None) -> torch.Tensor:
        started = time.time()
        if X0 is None:
            sol, resid = torch.zeros_like(B), B.clone()
        else:
            sol, resid = X0, B - mmv(X0)
        eps = self.params.cg_epsilon(sol.dtype)
        refresh = self.params.cg_full_gradient_every or 2 * max_iter
        stop_below = self.params.cg_tolerance ** 2
        direction = resid.clone()
        rr = (resid * resid).sum(0)                       # squared residual norm of every column
        elapsed = time.time() - started
        for it in range(max_iter):
            self.num_iter = it
            started = time.time()
            a_dir = mmv(direction)
            step = rr / ((direction * a_dir).sum(0) + eps)
            sol += direction * step
            if (it + 1) % refresh:
                resid -= a_dir * step
            else:
                if sol.is_cuda:
                    torch.cuda.synchronize()
                resid = B - mmv(sol)
            rr_next = (resid * resid).sum(0)
            if bool((rr_next < stop_below).all()):
                break
            direction *= rr_next / (rr + eps)
            direction += resid
            rr = rr_next
            elapsed += time.time() - started
            if callback is not None:
                try:
                    callback(it + 1, sol, elapsed)
                except StopOptimizationException as stop:
                    print(f"Optimization stopped from callback: {stop.message}")
                    break
        return sol


class FalkonConjugateGradient:
    r"""Preconditioned CG on ``B^T (K_nm^T K_nm + lambda n K_mm) B beta = B^T K_nm^T y / n`` with
    ``B = 1/sqrt(n) T^-1 A^-1`` (falkon/optim/conjgrad.py:187-306).  One ``kernel.dmmv`` per iteration; with a
    ``weight_fn`` (weighted least squares, ``K_nm^T W K_nm`` and ``K_nm^T W y``) two ``kernel.mmv`` with the weights
    applied in between (conjgrad.py:258-272,291-300)."""

    def __init__(self, kernel, preconditioner, opt: FalkonOptions, weight_fn=None, stored_knm=None):
        """``stored_knm``: K(X, M) kept in memory for the solve (what the reference's ``PrecomputedKernel`` is for,
        falkon/kernels/precomputed_kernel.py, falkon/models/model_utils.py:155-190): the products of every iteration
        are then library GEMMs on it instead of kernel evaluations."""
        self.kernel, self.preconditioner, self.params, self.weight_fn = kernel, preconditioner, opt, weight_fn
        self.stored_knm = stored_knm
        cg_fields = ("cg_epsilon_32", "cg_epsilon_64", "cg_tolerance", "cg_full_gradient_every",
                     "cg_differential_convergence")
        self.optimizer = ConjugateGradient(ConjugateGradientOptions(**{f: getattr(opt, f) for f in cg_fields}))

    def falkon_mmv(self, sol, penalty, X, M, n: int):
        """``A^-T (T^-T K_nm^T K_nm T^-1 / n + penalty I) A^-1 sol``: the operator of the preconditioned system
        (falkon/optim/conjgrad.py:262-285)."""
        pc = self.preconditioner
        inner = pc.invA(sol)
        if self.stored_knm is not None:
            gram = self.stored_knm.T @ (self.stored_knm @ pc.invT(inner))
        else:
            gram = self.kernel.dmmv(X, M, pc.invT(inner), None, opt=self.params)  # K_nm^T K_nm (.): the hot call
        return pc.invAt(pc.invTt(gram / n) + penalty * inner)

    def weighted_falkon_mmv(self, sol, penalty, X, M, y_weights, n: int):
        """The same operator with ``K_nm^T W K_nm`` in the middle (falkon/optim/conjgrad.py:258-272)."""
        pc = self.preconditioner
        inner = pc.invA(sol)
        if self.stored_knm is not None:
            gram = self.stored_knm.T @ (self.stored_knm @ pc.invT(inner)).mul_(y_weights)
        else:
            weighted = self.kernel.mmv(X, M, pc.invT(inner), None, opt=self.params).mul_(y_weights)
            gram = self.kernel.mmv(M, X, weighted, None, opt=self.params)
        return pc.invAt(pc.invTt(gram / n) + penalty * inner)

    @property
    def is_weighted(self) -> bool:
        return self.weight_fn is not None

    def solve(self, X, M, Y, _lambda, initial_solution, max_iter, callback=None):
        if not torch.is_inference_mode_enabled():
            # the reference fails here too, with torch's own message about inference tensors (the products run under
            # inference mode and the solver updates their results in place; falkon/tests/test_conjgrad.py:133-143)
            raise RuntimeError("FalkonConjugateGradient.solve was called outside InferenceMode: "
                               "wrap the call in `with torch.inference_mode():`")
        n = Y.shape[0]
        y_over_n = Y / n
        if self.is_weighted:
            y_weights = self.weight_fn(Y, X, torch.arange(n))
            y_over_n.mul_(y_weights)
            operator = functools.partial(self.weighted_falkon_mmv, penalty=_lambda, X=X, M=M, y_weights=y_weights, n=n)
        else:
            operator = functools.partial(self.falkon_mmv, penalty=_lambda, X=X, M=M, n=n)
        kty = self.stored_knm.T @ y_over_n if self.stored_knm is not None else self.kernel.mmv(M, X, y_over_n, opt=self.params)
        rhs = self.preconditioner.apply_t(kty)                                                # B^T K_nm^T (W) y / n
        return self.optimizer.solve(initial_solution, rhs, operator, max_iter, callback)
