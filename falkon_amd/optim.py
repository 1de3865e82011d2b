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
    every ``cg_full_gradient_every`` iterations, the solve stops once every column has
    ``|r|^2 < cg_tolerance^2``, and with ``cg_differential_convergence`` a column that has converged is frozen at
    its value while the others go on (:113-161).

    GPU tensors take the device-resident iteration (``flk_cg_update``): one launch does the vector work of an
    iteration, step lengths and convergence flags stay on the device, and the host looks at the flags only every
    ``CHECK_EVERY`` iterations (every iteration when a callback wants the solution), so iterations are enqueued
    without waiting for each other.  Once every column has converged the remaining launches of that window leave the
    solution untouched: the result is the one the reference's ``break`` gives.  With ``cg_capture_graph`` every kind
    of iteration is captured once into a HIP graph (operator and update together) and replayed; the row-block plan
    and workspace sizes of the operator are those of the capture, an operator that cannot be captured makes the
    solve continue eagerly with a warning, and host-resident operands switch replay off.  Differential convergence
    freezes a converged column but still passes it through the operator: unlike the reference, which shrinks its
    matrices (:113-161), it saves no operator work here.  Host tensors run the same iteration in torch ops."""

    CHECK_EVERY = 5

    def __init__(self, opt: Optional[ConjugateGradientOptions] = None):
        self.params = opt if opt is not None else ConjugateGradientOptions()
        self.num_iter = None
        self.capture_ok = True      # set to False by a caller whose operator touches host-resident data

    def solve(self, X0: Optional[torch.Tensor], B: torch.Tensor, mmv: Callable[[torch.Tensor], torch.Tensor],
              max_iter: int, callback: Optional[Callable[[int, torch.Tensor, float], None]] = None) -> torch.Tensor:
        if B.is_cuda and B.dim() == 2 and B.dtype in (torch.float32, torch.float64) and B.numel() > 0:
            return self._solve_on_device(X0, B, mmv, max_iter, callback)
        return self._solve_in_torch_ops(X0, B, mmv, max_iter, callback)

    # ------------------------------------------------------------------ GPU tensors
    def _solve_on_device(self, X0, B, mmv, max_iter, callback) -> torch.Tensor:
        from . import _backend
        from .mmv_ops.fmmv import _current, _stream_handle
        lib = _backend.load()
        started = time.time()
        dev, (m, t) = B.device, B.shape
        # work buffers take B's strides, so B has to be dense: row-major or column-major as it is, anything else (a
        # slice with a leading dimension, an expanded view whose columns alias each other) as a row-major copy
        if not (B.is_contiguous() or B.T.is_contiguous()):
            B = B.contiguous()
        strides = B.stride()

        def like_b(src=None):
            buf = torch.empty_strided((m, t), strides, dtype=B.dtype, device=dev)
            return buf if src is None else buf.copy_(src)

        def same_layout(x):
            return x if (x.stride() == strides and x.dtype == B.dtype) else like_b(x)

        if X0 is None:
            sol, resid = like_b().zero_(), like_b(B)
        else:
            sol, resid = same_layout(X0), like_b(B - mmv(X0))
        direction = like_b(resid)
        rsold = (resid * resid).sum(0).contiguous()
        state = torch.zeros(int(lib.flk_cg_state_ints(t)), dtype=torch.int32, device=dev)
        code = _backend.FLK_F32 if B.dtype == torch.float32 else _backend.FLK_F64
        eps = float(self.params.cg_epsilon(B.dtype))
        tol2 = float(self.params.cg_tolerance) ** 2
        refresh = self.params.cg_full_gradient_every or 2 * max_iter
        differential = int(bool(self.params.cg_differential_convergence) and t > 1)
        rs, cs = strides

        def update(mode, q, it):
            q = same_layout(q)
            with _current(dev):
                rc = lib.flk_cg_update(mode, sol.data_ptr(), resid.data_ptr(), direction.data_ptr(), q.data_ptr(),
                                       B.data_ptr(), m, t, rs, cs, rsold.data_ptr(), state.data_ptr(), it, eps, tol2,
                                       differential, code, _stream_handle(dev))
            _backend.raise_for_status(rc, "flk_cg_update")

        def iteration(it):
            if (it + 1) % refresh:
                update(0, mmv(direction), it)
            else:                                   # step, then the residual from scratch: R = B - A X
                update(1, mmv(direction), it)
                update(2, mmv(sol), it)

        graphs, pool = {}, None
        # replay needs an operator that only enqueues device work on device-resident data (a host-resident operand
        # would put pageable uploads into the capture): the caller says so through `capture_ok`
        use_graph = bool(getattr(self.params, "cg_capture_graph", False)) and self.capture_ok
        every = 1 if callback is not None else self.CHECK_EVERY
        elapsed = time.time() - started
        applied = 0
        for it in range(max_iter):
            started = time.time()
            if use_graph and it > 0:                # the first iteration runs eagerly (library set-up, lazy loads)
                key = (bool((it + 1) % refresh), it & 1)
                if key not in graphs:
                    g = torch.cuda.CUDAGraph()
                    pool = torch.cuda.graph_pool_handle() if pool is None else pool
                    try:
                        with torch.cuda.graph(g, pool=pool):
                            iteration(it)
                        graphs[key] = g
                    except Exception as exc:            # noqa: BLE001 -- an operator that cannot be captured
                        # (it waits for the device, or allocates outside the pool): the capture has ended with the
                        # context manager; nothing of this iteration has run, so the solve goes on eagerly from here
                        import warnings
                        warnings.warn(f"cg_capture_graph: the iteration could not be captured ({exc!r}); "
                                      "continuing without graph replay")
                        use_graph = False
                        graphs.pop(key, None)
                if use_graph:
                    graphs[key].replay()
                else:
                    iteration(it)
            else:
                iteration(it)
            applied = it + 1
            stop = False
            if (it + 1) % every == 0 or it + 1 == max_iter:
                flags = state.cpu()                 # waits for the iterations enqueued so far
                applied = int(flags[1])
                stop = bool(flags[2 + (it & 1) * t: 2 + (it & 1) * t + t].all())
            if stop:
                break
            elapsed += time.time() - started
            if callback is not None:
                try:
                    callback(it + 1, sol, elapsed)
                except StopOptimizationException as stop_exc:
                    print(f"Optimization stopped from callback: {stop_exc.message}")
                    break
        self.num_iter = max(applied - 1, 0) if max_iter > 0 else None
        if X0 is not None and sol is not X0:
            X0.copy_(sol)
            return X0
        return sol

    # ------------------------------------------------------------------ host tensors
    def _solve_in_torch_ops(self, X0, B, mmv, max_iter, callback) -> torch.Tensor:
        started = time.time()
        if X0 is None:
            sol, resid = torch.zeros_like(B), B.clone()
        else:
            sol, resid = X0, B - mmv(X0)
        eps = self.params.cg_epsilon(sol.dtype)
        refresh = self.params.cg_full_gradient_every or 2 * max_iter
        stop_below = self.params.cg_tolerance ** 2
        differential = bool(self.params.cg_differential_convergence) and sol.dim() == 2 and sol.shape[1] > 1
        frozen = torch.zeros(sol.shape[1], dtype=torch.bool, device=sol.device) if differential else None
        direction = resid.clone()
        rr = (resid * resid).sum(0)                       # squared residual norm of every column
        elapsed = time.time() - started
        for it in range(max_iter):
            self.num_iter = it
            started = time.time()
            a_dir = mmv(direction)
            step = rr / ((direction * a_dir).sum(0) + eps)
            if differential:
                step = torch.where(frozen, torch.zeros_like(step), step)      # frozen columns no longer move
            sol += direction * step
            if (it + 1) % refresh:
                resid -= a_dir * step
            else:
                if sol.is_cuda:
                    torch.cuda.synchronize()
                fresh = B - mmv(sol)
                resid = torch.where(frozen, resid, fresh) if differential else fresh
            rr_next = (resid * resid).sum(0)
            converged = rr_next < stop_below
            if differential:
                frozen |= converged
                converged = frozen
            if bool(converged.all()):
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
        self._packed = None          # X and the centres packed once for the solve (PackedProducts), where that applies
        cg_fields = ("cg_epsilon_32", "cg_epsilon_64", "cg_tolerance", "cg_full_gradient_every",
                     "cg_differential_convergence", "cg_capture_graph")
        self.optimizer = ConjugateGradient(ConjugateGradientOptions(**{f: getattr(opt, f) for f in cg_fields}))

    def falkon_mmv(self, sol, penalty, X, M, n: int):
        """``A^-T (T^-T K_nm^T K_nm T^-1 / n + penalty I) A^-1 sol``: the operator of the preconditioned system
        (falkon/optim/conjgrad.py:262-285)."""
        pc = self.preconditioner
        inner = pc.invA(sol)
        if self.stored_knm is not None:
            gram = self.stored_knm.T @ (self.stored_knm @ pc.invT(inner))
        elif self._packed is not None:
            gram = self._packed.dmmv(pc.invT(inner))                              # the same product on operands packed once
        else:
            gram = self.kernel.dmmv(X, M, pc.invT(inner), None, opt=self.params)  # K_nm^T K_nm (.): the hot call
        return pc.invAt(pc.invTt(gram / n) + penalty * inner)

    def weighted_falkon_mmv(self, sol, penalty, X, M, y_weights, n: int):
        """The same operator with ``K_nm^T W K_nm`` in the middle (falkon/optim/conjgrad.py:258-272)."""
        pc = self.preconditioner
        inner = pc.invA(sol)
        if self.stored_knm is not None:
            gram = self.stored_knm.T @ (self.stored_knm @ pc.invT(inner)).mul_(y_weights)
        elif self._packed is not None:
            gram = self._packed.mmv_t(self._packed.mmv(pc.invT(inner)).mul_(y_weights))
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
        self.optimizer.capture_ok = bool(X.is_cuda and M.is_cuda and Y.is_cuda)
        self._packed = None
        if self.stored_knm is None and getattr(self.params, "cg_pack_once", True) and Y.is_cuda:
            from .mmv_ops.fmmv import PackedProducts
            self._packed = PackedProducts.create(X, M, self.kernel, self.params, columns=Y.shape[1])
            if self._packed is not None and (Y.device != X.device or Y.dtype != X.dtype):
                self._packed = None
        try:
            if self.stored_knm is not None:
                kty = self.stored_knm.T @ y_over_n
            elif self._packed is not None:
                kty = self._packed.mmv_t(y_over_n)
            else:
                kty = self.kernel.mmv(M, X, y_over_n, opt=self.params)
            rhs = self.preconditioner.apply_t(kty)                                            # B^T K_nm^T (W) y / n
            return self.optimizer.solve(initial_solution, rhs, operator, max_iter, callback)
        finally:
            self._packed = None                                                               # frees the packed copies
