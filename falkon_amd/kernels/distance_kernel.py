"""Gaussian kernel object (falkon/kernels/distance_kernel.py:20-38,314-432).

``mmv`` / ``dmmv`` and the kernel matrix ``kernel(X1, X2)`` run the MI355X kernels of
``libfalkon_amd``.  ``compute`` (the explicit kernel block the reference's ``rbf_core``
produces) is kept with stock torch ops for the kernel diagonal and for callers that hand it
their own blocks; it is not on the kernel-vector path.
"""
from typing import Dict, Optional, Union

import torch

from ..options import FalkonOptions
from .diff_kernel import DiffKernel

__all__ = ("GaussianKernel", "validate_sigma")


def validate_sigma(sigma: Union[float, torch.Tensor]) -> torch.Tensor:
    """float -> 1-element fp64 tensor; 1-element tensor kept as is; vector or (d,1) matrix ->
    flat per-dimension lengthscales; anything else ValueError (distance_kernel.py:20-38)."""
    if not isinstance(sigma, torch.Tensor):
        try:
            value = float(sigma)
        except TypeError:
            raise TypeError("Sigma must be a scalar or a tensor.") from None
        return torch.tensor([value], dtype=torch.float64)
    if sigma.numel() == 1:
        return sigma
    is_vector = sigma.dim() == 1 or (sigma.dim() == 2 and sigma.shape[1] == 1)
    if not is_vector:
        raise ValueError("sigma must be a scalar or a vector.")
    return sigma.reshape(-1)


def _rbf_block(mat1, mat2, out: Optional[torch.Tensor], diag: bool, sigma: torch.Tensor) -> torch.Tensor:
    """exp(-1/2 |mat1/sigma - mat2/sigma|^2) as a stored block, with stock torch ops."""
    sigma = sigma.to(device=mat1.device, dtype=mat1.dtype)
    a, b = mat1 / sigma, mat2 / sigma
    if diag:
        res = (a - b).square().sum(-1).mul_(-0.5).exp_()
        return res if out is None else out.copy_(res)
    na, nb = a.square().sum(-1, keepdim=True), b.square().sum(-1, keepdim=True)
    if out is None:
        out = torch.addmm(na, a, b.T, alpha=-2, beta=1)
    else:
        out = torch.addmm(na, a, b.T, alpha=-2, beta=1, out=out)
    out.add_(nb.T).clamp_min_(1e-20).mul_(-0.5).exp_()
    return out


class GaussianKernel(DiffKernel):
    r"""k(x, x') = exp(-|x - x'|^2 / (2 sigma^2)); ``sigma`` a scalar or one lengthscale per dimension."""

    kernel_name = "gaussian"
    core_fn = _rbf_block

    def __init__(self, sigma: Union[float, torch.Tensor], opt: Optional[FalkonOptions] = None):
        sigma = validate_sigma(sigma)
        super().__init__(self.kernel_name, opt, core_fn=GaussianKernel.core_fn, sigma=sigma)
        self._sigma_cache = {}

    def _sigma_on(self, device: torch.device, dtype: torch.dtype) -> torch.Tensor:
        """sigma on the data's device and dtype (distance_kernel.py:148), cached until sigma changes."""
        sigma = self.sigma
        key = (device, dtype)
        tag = (sigma.data_ptr(), sigma._version, sigma.numel())
        hit = self._sigma_cache.get(key)
        if hit is None or hit[0] != tag:
            hit = (tag, sigma.detach().reshape(-1).to(device=device, dtype=dtype).contiguous())
            self._sigma_cache[key] = hit
        return hit[1]

    def extra_mem(self, is_differentiable, is_sparse, dtype, density1=None, density2=None) -> Dict[str, float]:
        # the fused kernels need no per-entry scratch; the packed operands are sized by the library itself
        return {}

    def detach(self) -> "GaussianKernel":
        return GaussianKernel(self.sigma.detach(), opt=self.params)

    def __repr__(self):
        return f"GaussianKernel(sigma={self.sigma})"

    def __str__(self):
        return f"Gaussian kernel<{self.sigma}>"
