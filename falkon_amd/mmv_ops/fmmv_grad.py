"""Backward passes of the kernel-vector product and of the kernel matrix for the radial kernels, on the MI355X.

The reference differentiates ``K(X1, X2) @ v`` by re-running every block of the product under autograd
(falkon/mmv_ops/fmmv.py:405-485, backward at :935-957): per block it stores K, the graph of the kernel's core
function and the gradients of the expanded squared distance.  Here the gradients are written out in closed form and
reduced to products the library's kernels already compute, so that the backward pass too never stores K.

With u_ij = sum_k ((x_ik - c_jk) / sigma_k)^2, K_ij = f(u_ij) and G = dL/d(out) (N x T):

    W_ij      = f'(u_ij) * sum_t G_it v_jt
    dL/dv     = K^T G                                             (a kernel-vector product with the kernel itself)
    dL/dx_ik  =  2/sigma_k^2 * ( x_ik * sum_j W_ij - sum_j W_ij c_jk )
    dL/dc_jk  =  2/sigma_k^2 * ( c_jk * sum_i W_ij - sum_i W_ij x_ik )
    dL/dsigma_k = -( sum_i x_ik dL/dx_ik + sum_j c_jk dL/dc_jk ) / sigma_k     (K depends on x / sigma only)

``sum_j W_ij [c_j, 1]`` is ``sum_t G[:, t] * (K' @ (v[:, t] * [C, 1]))``: a kernel-vector product with the derivative
kernel K' = f'(u) and d + 1 right-hand sides per column of v, and likewise on the other side.  f' is, up to a
factor, a kernel of the library (see ``_DERIVATIVE``).  All formulas are invariant under a common translation of X1
and X2; the data is centred on the mean of X2 first, which keeps the differences above from cancelling.

The Laplacian's derivative weight exp(-D)/D is unbounded where two points (nearly) coincide, as centres drawn from
the data do: there the pair's true contribution W_ij (x_i - c_j) is zero, but W_ij itself is 1/(the rounding noise of
D), and in fp32 the two sums it enters no longer cancel (an error of order sqrt(eps) per such pair, which the
reference's fp32 autograd shows as well).  The Laplacian's backward pass therefore runs in fp64 whatever the data's
dtype: the noise of D drops to 1e-8 and the cancellation keeps eight digits.
"""
import math
from typing import Optional, Sequence, Tuple

import torch

from .. import _backend
from ..options import BaseOptions
from .fmmv import _compute_device, _on, gauss_fmmv_native
from .fmm import gauss_fmm_native

__all__ = ("fmmv_backward", "fmm_backward", "derivative_kernel")

# f'(u) = coef * kernel'(X1, X2; factor * sigma), u the squared scaled distance:
#   Gaussian   f = exp(-u/2):                 f' = -1/2 f
#   Laplacian  f = exp(-sqrt(u)):             f' = -1/2 exp(-D)/D, 0 where the reference clamps u (distance_kernel.py:100)
#   Matern 3/2 f = (1+s) exp(-s), s=sqrt(3u): f' = -3/2 exp(-s)          = -3/2 Laplacian with sigma / sqrt(3)
#   Matern 5/2 f = (1+s+s^2/3) exp(-s), s=sqrt(5u): f' = -5/6 (1+s) exp(-s) = -5/6 Matern 3/2 with sigma * sqrt(3/5)
_DERIVATIVE = {
    _backend.FLK_GAUSSIAN: (_backend.FLK_GAUSSIAN, 1.0, -0.5),
    _backend.FLK_LAPLACIAN: (_backend.FLK_LAPLACIAN_DU, 1.0, -0.5),
    _backend.FLK_MATERN32: (_backend.FLK_LAPLACIAN, 1.0 / math.sqrt(3.0), -1.5),
    _backend.FLK_MATERN52: (_backend.FLK_MATERN32, math.sqrt(3.0 / 5.0), -5.0 / 6.0),
}

# right-hand sides handed to one kernel-vector product of the backward pass
_MAX_COLUMNS = 256


def derivative_kernel(kernel_fn: int) -> Tuple[int, float, float]:
    """(library kernel, factor on sigma, coefficient) such that f'(u) = coefficient * kernel(factor * sigma)."""
    return _DERIVATIVE[kernel_fn]


def _unit_strided(t: torch.Tensor) -> torch.Tensor:
    return t if (t.dim() == 2 and 1 in t.stride() and 0 not in t.stride()) else t.contiguous()


def _weighted_moments(Xa, Xb, ga, vb, sigma_dev, kernel_fn: int) -> torch.Tensor:
    """R[i] = sum_j kernel(Xa_i, Xb_j) * (sum_t ga[i, t] vb[j, t]) * [Xb_j, 1]: na x (d + 1), K never stored."""
    na, d = Xa.shape
    nb, T = vb.shape
    ext = torch.cat([Xb, torch.ones((nb, 1), dtype=Xb.dtype, device=Xb.device)], dim=1)
    acc = torch.zeros((na, d + 1), dtype=Xa.dtype, device=Xa.device)
    if na == 0 or nb == 0:
        return acc
    per_call = max(1, min(T, _MAX_COLUMNS // (d + 1)))
    for t0 in range(0, T, per_call):
        k = min(per_call, T - t0)
        rhs = (vb[:, t0:t0 + k, None] * ext[:, None, :]).reshape(nb, k * (d + 1))
        res = torch.empty((na, k * (d + 1)), dtype=Xa.dtype, device=Xa.device)
        gauss_fmmv_native(Xa, Xb, sigma_dev, rhs, res, kernel_fn)
        acc += (res.view(na, k, d + 1) * ga[:, t0:t0 + k, None]).sum(dim=1)
    return acc


def _sigma_grad(sig: torch.Tensor, Xa, ga_x, Xb, gb_x) -> torch.Tensor:
    """dL/dsigma_k = -(sum_i x_ik dL/dx_ik + sum_j c_jk dL/dc_jk) / sigma_k; summed over k for a single sigma."""
    per_dim = -((Xa * ga_x).sum(0) + (Xb * gb_x).sum(0)) / sig
    return per_dim if sig.numel() > 1 else per_dim.sum().reshape(1)


def _work_dtype(kernel_fn: int, dtype: torch.dtype) -> torch.dtype:
    """The arithmetic of the backward pass: the data's dtype, except fp64 for the Laplacian (unbounded weight)."""
    return torch.float64 if _DERIVATIVE[kernel_fn][0] == _backend.FLK_LAPLACIAN_DU else dtype


def _centre(X1: torch.Tensor, X2: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    if X2.shape[0] == 0:
        return X1, X2
    mu = X2.mean(dim=0, keepdim=True)
    return (X1 - mu).contiguous(), (X2 - mu).contiguous()


def fmmv_backward(kernel_fn: int, X1: torch.Tensor, X2: torch.Tensor, v: torch.Tensor, sigma: torch.Tensor,
                  G: torch.Tensor, needs: Sequence[bool], opt: Optional[BaseOptions] = None):
    """Gradients of ``sum(G * (K(X1, X2) @ v))`` with respect to (X1, X2, v, sigma), None where ``needs`` is False.

    ``sigma`` has 1 or d elements; every tensor may live on the host or on the GPU, the results are on the compute
    device.  The whole problem is kept resident (no splitting over rows as in the forward pass)."""
    opt = opt if opt is not None else BaseOptions()
    need_x1, need_x2, need_v, need_sigma = needs
    dev = _compute_device(opt, (X1.device, X2.device, v.device, G.device))
    dtype = X1.dtype
    with torch.no_grad():
        X1d, X2d, vd = (_unit_strided(_on(t.detach(), dev)) for t in (X1, X2, v))
        Gd = _unit_strided(_on(G.detach(), dev).to(dtype))
        g_x1 = g_x2 = g_v = g_sigma = None
        if need_v:
            g_v = torch.empty(vd.shape, dtype=dtype, device=dev)
            if X1d.shape[0] == 0 or X2d.shape[0] == 0:
                g_v.zero_()
            else:
                sig = sigma.detach().reshape(-1).to(device=dev, dtype=dtype).contiguous()
                gauss_fmmv_native(X2d, X1d, sig, Gd, g_v, kernel_fn)
        if need_x1 or need_x2 or need_sigma:
            d_fn, factor, coef = _DERIVATIVE[kernel_fn]
            work = _work_dtype(kernel_fn, dtype)
            X1d, X2d, vd, Gd = (t.to(work) for t in (X1d, X2d, vd, Gd))
            sig = sigma.detach().reshape(-1).to(device=dev, dtype=work).contiguous()
            d_sig = (sig * factor).contiguous()
            Xc1, Xc2 = _centre(X1d, X2d)
            scale = (2.0 * coef) / (sig * sig)
            d = X1d.shape[1]
            if need_x1 or need_sigma:
                mom = _weighted_moments(Xc1, Xc2, Gd, vd, d_sig, d_fn)
                g_x1 = (Xc1 * mom[:, d:] - mom[:, :d]) * scale
            if need_x2 or need_sigma:
                mom = _weighted_moments(Xc2, Xc1, vd, Gd, d_sig, d_fn)
                g_x2 = (Xc2 * mom[:, d:] - mom[:, :d]) * scale
            if need_sigma:
                g_sigma = _sigma_grad(sig, Xc1, g_x1, Xc2, g_x2)
            g_x1 = g_x1 if need_x1 else None
            g_x2 = g_x2 if need_x2 else None
    return g_x1, g_x2, g_v, g_sigma


def fmm_backward(kernel_fn: int, X1: torch.Tensor, X2: torch.Tensor, sigma: torch.Tensor, G: torch.Tensor,
                 needs: Sequence[bool], opt: Optional[BaseOptions] = None):
    """Gradients of ``sum(G * K(X1, X2))`` with respect to (X1, X2, sigma): W = f'(u) * G is stored (N x M, as G is),
    the contractions ``W @ X2`` and ``W.T @ X1`` are library GEMMs (the reference re-runs every block
    under autograd instead, falkon/mmv_ops/fmm.py:391-438,648-696)."""
    opt = opt if opt is not None else BaseOptions()
    need_x1, need_x2, need_sigma = needs
    dev = _compute_device(opt, (X1.device, X2.device, G.device))
    dtype = _work_dtype(kernel_fn, X1.dtype)
    with torch.no_grad():
        X1d, X2d = (_unit_strided(_on(t.detach(), dev)).to(dtype) for t in (X1, X2))
        sig = sigma.detach().reshape(-1).to(device=dev, dtype=dtype).contiguous()
        d_fn, factor, coef = _DERIVATIVE[kernel_fn]
        Xc1, Xc2 = _centre(X1d, X2d)
        W = torch.empty((X1d.shape[0], X2d.shape[0]), dtype=dtype, device=dev)
        if W.numel() > 0:
            gauss_fmm_native(Xc1, Xc2, (sig * factor).contiguous(), W, False, d_fn)
        W.mul_(_on(G.detach(), dev).to(dtype))
        scale = (2.0 * coef) / (sig * sig)
        g_x1 = g_x2 = g_sigma = None
        if need_x1 or need_sigma:
            g_x1 = (Xc1 * W.sum(dim=1, keepdim=True) - W @ Xc2) * scale
        if need_x2 or need_sigma:
            g_x2 = (Xc2 * W.sum(dim=0).unsqueeze(1) - W.T @ Xc1) * scale
        if need_sigma:
            g_sigma = _sigma_grad(sig, Xc1, g_x1, Xc2, g_x2)
        g_x1 = g_x1 if need_x1 else None
        g_x2 = g_x2 if need_x2 else None
    return g_x1, g_x2, g_sigma
