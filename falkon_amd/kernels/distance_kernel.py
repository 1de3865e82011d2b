"""Distance kernels: Gaussian, Laplacian, Matern (falkon/kernels/distance_kernel.py:20-38,314-648).

``mmv`` / ``dmmv`` and the kernel matrix ``kernel(X1, X2)`` run the MI355X kernels of
``libfalkon_amd``.  ``compute`` (the explicit kernel block the reference's ``rbf_core``
produces) is kept with stock torch ops for the kernel diagonal and for callers that hand it
their own blocks; it is not on the kernel-vector path.
"""
from typing import Dict, Optional, Union

import torch

from ..options import FalkonOptions
from .diff_kernel import DiffKernel

__all__ = ("GaussianKernel", "LaplacianKernel", "MaternKernel", "validate_sigma")


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


_SQRT3, _SQRT5 = 3.0 ** 0.5, 5.0 ** 0.5


def _radial_block(mat1, mat2, out: Optional[torch.Tensor], diag: bool, sigma: torch.Tensor,
                  nu: float = float("inf")) -> torch.Tensor:
    """A stored block of a radial kernel with stock torch ops: f(D), D = |mat1/sigma - mat2/sigma|, with
    f = exp(-D^2/2) (nu = inf), exp(-D) (1/2), (1 + s) exp(-s) with s = sqrt(3) D (3/2),
    (1 + s + s^2/3) exp(-s) with s = sqrt(5) D (5/2).  Off the kernel-vector path (diagonals, callers' own blocks)."""
    sigma = sigma.to(device=mat1.device, dtype=mat1.dtype)
    a, b = mat1 / sigma, mat2 / sigma
    # no in-place updates: the block may be differentiated (diagonals under autograd)
    if diag:
        d2 = (a - b).square().sum(-1)
        if nu != float("inf") and d2.requires_grad:
            d2 = d2.clamp_min(1e-20)                                # keeps the square root's gradient finite
    else:
        d2 = torch.addmm(a.square().sum(-1, keepdim=True), a, b.T, alpha=-2, beta=1)
        d2 = (d2 + b.square().sum(-1, keepdim=True).T).clamp_min(1e-20)
    if nu == float("inf"):
        res = torch.exp(-0.5 * d2)
    else:
        s = d2.sqrt() * {0.5: 1.0, 1.5: _SQRT3, 2.5: _SQRT5}[nu]
        decay = torch.exp(-s)
        res = decay if nu == 0.5 else decay * (1 + s if nu == 1.5 else 1 + s + s * s / 3)
    return res if out is None else out.copy_(res.reshape(out.shape))


class _RadialKernel(DiffKernel):
    """Shared part of the distance kernels: ``sigma`` (scalar or one lengthscale per dimension) as a registered
    parameter, its cached copy on the data's device, and no per-entry scratch memory."""

    def __init__(self, name: str, sigma, opt: Optional[FalkonOptions], **other_params):
        super().__init__(name, opt, core_fn=_radial_block, sigma=validate_sigma(sigma), **other_params)
        self._sigma_cache = {}

    def _sigma_on(self, device: torch.device, dtype: torch.dtype, cached: bool = True) -> torch.Tensor:
        """sigma on the data's device and dtype (distance_kernel.py:148).  A host-resident sigma (the usual case) is
        uploaded once per (device, dtype) and again whenever its VALUES differ from the snapshot taken at the upload:
        the comparison is of 1 or d host numbers, and unlike the tensor's version counter it also sees writes through
        ``sigma.data``.  A sigma that already lives on the GPU is used (or converted) as it is on every call."""
        sigma = self.sigma.detach().reshape(-1)
        if not cached or sigma.device.type != "cpu":
            return sigma.to(device=device, dtype=dtype).contiguous()
        key = (device, dtype)
        hit = self._sigma_cache.get(key)
        if hit is None or hit[0].shape != sigma.shape or not torch.equal(hit[0], sigma):
            hit = (sigma.clone(), sigma.to(device=device, dtype=dtype).contiguous())
            self._sigma_cache[key] = hit
        return hit[1]

    def extra_mem(self, is_differentiable, is_sparse, dtype, density1=None, density2=None) -> Dict[str, float]:
        # the fused kernels need no per-entry scratch; the packed operands are sized by the library itself
        return {}


class GaussianKernel(_RadialKernel):
    r"""k(x, x') = exp(-|x - x'|^2 / (2 sigma^2)); ``sigma`` a scalar or one lengthscale per dimension."""

    kernel_name = "gaussian"

    def __init__(self, sigma: Union[float, torch.Tensor], opt: Optional[FalkonOptions] = None):
        super().__init__(self.kernel_name, sigma, opt)

    def detach(self) -> "GaussianKernel":
        return GaussianKernel(self.sigma.detach(), opt=self.params)

    def __repr__(self):
        return f"GaussianKernel(sigma={self.sigma})"

    def __str__(self):
        return f"Gaussian kernel<{self.sigma}>"


class LaplacianKernel(_RadialKernel):
    r"""k(x, x') = exp(-|x - x'| / sigma) (falkon/kernels/distance_kernel.py:435-507)."""

    kernel_name = "laplacian"

    def __init__(self, sigma: Union[float, torch.Tensor], opt: Optional[FalkonOptions] = None):
        super().__init__(self.kernel_name, sigma, opt, nu=0.5)

    def detach(self) -> "LaplacianKernel":
        return LaplacianKernel(self.sigma.detach(), opt=self.params)

    def __repr__(self):
        return f"LaplacianKernel(sigma={self.sigma})"

    def __str__(self):
        return f"Laplacian kernel<{self.sigma}>"


class MaternKernel(_RadialKernel):
    r"""Matern kernel for the smoothness values with a closed form, nu in {0.5, 1.5, 2.5, inf}
    (falkon/kernels/distance_kernel.py:510-648): nu = 0.5 is the Laplacian, nu = inf the Gaussian."""

    _valid_nu_values = frozenset({0.5, 1.5, 2.5, float("inf")})

    def __init__(self, sigma: Union[float, torch.Tensor], nu: Union[float, torch.Tensor],
                 opt: Optional[FalkonOptions] = None):
        nu = self.validate_nu(nu)
        self.kernel_name = f"{nu:.1f}-matern"
        super().__init__(self.kernel_name, sigma, opt, nu=nu)

    @staticmethod
    def validate_nu(nu: Union[torch.Tensor, float]) -> float:
        """A float or a tensor without gradient, rounded to two digits, one of the four closed-form values."""
        if isinstance(nu, torch.Tensor):
            if nu.requires_grad:
                raise ValueError("The nu parameter of the Matern kernel is not differentiable, "
                                 "and must not require gradients.")
            if nu.numel() != 1:
                raise ValueError(f"nu={nu} is not convertible to a scalar.")
            value = float(nu.item())
        elif isinstance(nu, float):
            value = nu
        else:
            raise TypeError(f"nu must be a float or a tensor, not a {type(nu)}")
        value = round(value, ndigits=2)
        if value not in MaternKernel._valid_nu_values:
            raise ValueError(f"The given value of nu = {value} can only take values {MaternKernel._valid_nu_values}.")
        return value

    def detach(self) -> "MaternKernel":
        return MaternKernel(self.sigma.detach(), self.nondiff_params["nu"], opt=self.params)

    def __repr__(self):
        return f"MaternKernel(sigma={self.sigma}, nu={self.nondiff_params['nu']:.1f})"

    def __str__(self):
        return f"Matern kernel<{self.sigma}, {self.nondiff_params['nu']:.1f}>"
