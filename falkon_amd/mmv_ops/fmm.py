"""Explicit kernel matrix K(X1, X2): the K(C, C) the preconditioner factorises once per fit, and
``kernel(X1, X2)``.

Drop-in for falkon/mmv_ops/fmm.py:298-388,576-640,699-708 in the dense, non-differentiable case of the radial
kernels (Gaussian, Laplacian, Matern):
``flk_gauss_fmm`` packs both operands and writes the matrix in one launch (cross term on MFMA, exp2 on
the accumulators).  With ``opt.no_single_kernel`` fp32 inputs are evaluated in fp64 and rounded once
when stored (falkon/mmv_ops/fmm.py:619-622).  Rows of X1 are split only when the result is wanted on
the host or the operands do not fit.  The diagonal (``diag=True``) is O(N d) and stays on stock torch
ops through the kernel's ``compute``.
"""
from typing import Optional

import torch

from .. import _backend
from ..options import BaseOptions
from ..utils.helpers import sizeof_dtype
from .fmmv import (_DTYPE_CODE, _arith_code, _check_dtype, _compute_device, _current, _kernel_fn, _mat, _on,
                   _rows_that_fit, _stream_handle)
from .utils import check_contiguity, create_output_mat, usable_gpu_memory

__all__ = ("fmm", "gauss_fmm_native")


def gauss_fmm_native(X1, X2, sigma_dev, out, compute_f64: bool, kernel_fn: int = _backend.FLK_GAUSSIAN,
                     code: Optional[int] = None) -> None:
    """out[n,m] = K(X1, X2) through ``flk_kernel_fmm``.  All tensors on one GPU, 2-D, same dtype; ``code`` is the
    library's dtype code (the data's dtype, or the bf16x3 mode of fp32)."""
    lib = _backend.load()
    code = _DTYPE_CODE[X1.dtype] if code is None else code
    n, d = X1.shape
    m = X2.shape[0]
    ws_bytes = lib.flk_gauss_fmm_workspace_bytes(n, m, d, code, int(compute_f64))
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=X1.device)
    p1, _, r1, c1 = _mat(X1)
    p2, _, r2, c2 = _mat(X2)
    po, _, ro, co = _mat(out)
    with _current(X1.device):
        rc = lib.flk_kernel_fmm(kernel_fn, p1, n, r1, c1, p2, m, r2, c2, d, sigma_dev.data_ptr(), sigma_dev.numel(),
                                po, ro, co, code, int(compute_f64), ws.data_ptr(), ws_bytes,
                                _stream_handle(X1.device))
    _backend.raise_for_status(rc, "flk_kernel_fmm")


class _KernelMmFn(torch.autograd.Function):
    """The kernel matrix with its backward pass (the reference's KernelMmFnFull, falkon/mmv_ops/fmm.py:441-696)."""

    @staticmethod
    def forward(ctx, kernel, opt, out, X1, X2, *kernel_params):
        kernel_fn = _kernel_fn(kernel)
        res = _fmm_run(kernel, kernel_fn, opt, out, X1, X2, cached_sigma=False)
        if out is not None:
            ctx.mark_dirty(out)
        ctx.save_for_backward(X1, X2, *kernel_params)
        ctx.kernel_fn, ctx.opt = kernel_fn, opt
        return res

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_out):
        from .fmmv_grad import fmm_backward
        X1, X2, sigma = ctx.saved_tensors
        grads = fmm_backward(ctx.kernel_fn, X1, X2, sigma, grad_out, ctx.needs_input_grad[3:6], ctx.opt)
        grads = [None if g is None else g.reshape(t.shape).to(device=t.device, dtype=t.dtype)
                 for g, t in zip(grads, (X1, X2, sigma))]
        return (None, None, None, *grads)


def fmm(kernel, opt: Optional[BaseOptions], out: Optional[torch.Tensor], diag: bool, X1: torch.Tensor,
        X2: torch.Tensor, kwargs_m1=None, kwargs_m2=None) -> torch.Tensor:
    """``K(X1, X2)`` (N x M) or its diagonal (falkon/mmv_ops/fmm.py:699-717); differentiable with respect to X1, X2
    and the kernel's lengthscale when any of them requires a gradient."""
    opt = opt if opt is not None else BaseOptions()
    check_contiguity((X1, "X1"), (X2, "X2"), (out, "out"))
    kernel_params = list(kernel.diff_params.values())
    differentiable = any(t.requires_grad for t in [X1, X2] + kernel_params)
    if diag:
        dev = _compute_device(opt, (X1.device, X2.device))
        if differentiable:
            # the diagonal is O(N d): stock torch ops under autograd
            res = kernel.compute_diff(X1.to(dev), X2.to(dev), diag=True).to(X1.device)
            return res if out is None else out.copy_(res.reshape(out.shape))
        with torch.inference_mode():
            res = kernel.compute(X1.to(dev), X2.to(dev), None, diag=True)
            if out is None:
                return res.to(X1.device)
            return out.copy_(res.reshape(out.shape))
    kernel_fn = _kernel_fn(kernel)
    if differentiable:
        return _KernelMmFn.apply(kernel, opt, out, X1, X2, *kernel_params)
    return _fmm_run(kernel, kernel_fn, opt, out, X1, X2, cached_sigma=True)


def _fmm_run(kernel, kernel_fn: int, opt: BaseOptions, out, X1, X2, cached_sigma: bool) -> torch.Tensor:
    data_devs = (X1.device, X2.device)
    dev = _compute_device(opt, data_devs)
    N, D = X1.shape
    M = X2.shape[0]
    _check_dtype(X1.dtype)
    out = create_output_mat(out, data_devs, shape=(N, M), dtype=X1.dtype, other_mat=X1)
    if N == 0 or M == 0:
        return out
    with torch.inference_mode():
        lib = _backend.load()
        code, sz = _arith_code(X1.dtype, opt), sizeof_dtype(X1.dtype)      # (the bf16x3 mode of fp32 where it applies)
        compute_f64 = X1.dtype == torch.float32 and bool(opt.no_single_kernel)
        sigma_dev = kernel._sigma_on(dev, X1.dtype, cached=cached_sigma)
        x1_in, out_in = X1.device == dev, out.device == dev
        fixed = 0 if X2.device == dev else M * D * sz

        def need(rows: int) -> float:
            stage = (0 if x1_in else rows * D * sz) + (0 if out_in else rows * M * sz)
            return lib.flk_gauss_fmm_workspace_bytes(rows, M, D, code, int(compute_f64)) + stage + fixed

        usable = usable_gpu_memory(dev, opt.max_gpu_mem, opt.memory_slack, enough=need(N))
        blk = _rows_that_fit(N, need, usable)
        X2d = _on(X2, dev)
        for i in range(0, N, blk):
            li = min(blk, N - i)
            X1d = _on(X1[i:i + li], dev)
            outd = out[i:i + li] if out_in else torch.empty((li, M), dtype=out.dtype, device=dev)
            gauss_fmm_native(X1d, X2d, sigma_dev, outd, compute_f64, kernel_fn, code)
            if not out_in:
                out[i:i + li].copy_(outd)
    return out
