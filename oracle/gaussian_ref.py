"""Per-block arithmetic of the reference's distance kernels (Gaussian, Laplacian, Matern), restated in torch CPU ops.

Test infrastructure only (see ``oracle/__init__.py``).
"""
from typing import Optional, Union

import torch


def validate_sigma_ref(sigma: Union[float, torch.Tensor]) -> torch.Tensor:
    """Follows falkon/kernels/distance_kernel.py:20-38.

    float -> 1-element fp64 tensor; 1-element tensor kept; 1-D or (d,1) tensor
    flattened (per-dimension lengthscales); anything else is a ValueError.
    """
    if isinstance(sigma, torch.Tensor):
        if sigma.numel() == 1:
            return sigma
        if sigma.dim() == 1 or sigma.shape[1] == 1:
            return sigma.reshape(-1)
        raise ValueError("sigma must be a scalar or a vector.")
    try:
        return torch.tensor([float(sigma)], dtype=torch.float64)
    except TypeError:
        raise TypeError("Sigma must be a scalar or a tensor.") from None


def square_norm_ref(x: torch.Tensor, dim: int = -1, keepdim: bool = True) -> torch.Tensor:
    """Row-wise sum of squares in the input dtype.

    Follows falkon/la_helpers/wrapper.py:128-129 ->
    falkon/c_ext/ops/cpu/cpu_square_norm.cpp:14-60 (a TensorIterator reduction of
    x*x accumulated in the input dtype).  Equal to ``torch.norm(x, dim)**2`` up to
    summation order (falkon/tests/test_matrix_ops.py:72-76).
    """
    return (x * x).sum(dim=dim, keepdim=keepdim)


def sq_dist_ref(mat1, mat2, norm_mat1, norm_mat2, out: Optional[torch.Tensor]) -> torch.Tensor:
    """Follows falkon/kernels/distance_kernel.py:88-101 (2-D branch).

    One ``addmm(alpha=-2, beta=1)`` that broadcasts the row norms, then the
    column norms are added and the result clamped at 1e-20.
    """
    if out is None:
        out = torch.addmm(norm_mat1, mat1, mat2.transpose(-2, -1), alpha=-2, beta=1)
    else:
        out = torch.addmm(norm_mat1, mat1, mat2.transpose(-2, -1), alpha=-2, beta=1, out=out)
    out.add_(norm_mat2.transpose(-2, -1))
    out.clamp_min_(1e-20)
    return out


def rbf_core_ref(mat1: torch.Tensor, mat2: torch.Tensor, out: Optional[torch.Tensor], sigma: torch.Tensor) -> torch.Tensor:
    """Follows falkon/kernels/distance_kernel.py:140-159 (``diag=False``).

    sigma is cast to the data dtype first, both operands are divided by it, the
    squared distance is formed through the expanded norm, then ``*(-0.5)`` and
    ``exp`` in place.  A sigma whose length is neither 1 nor d fails in the
    division with torch's broadcast RuntimeError, as in the reference
    (falkon/tests/test_kernels.py:338-358).
    """
    sigma = sigma.to(device=mat1.device, dtype=mat1.dtype)
    mat1_div_sig = mat1 / sigma
    mat2_div_sig = mat2 / sigma
    norm_sq_mat1 = square_norm_ref(mat1_div_sig, -1, True)
    norm_sq_mat2 = square_norm_ref(mat2_div_sig, -1, True)
    out = sq_dist_ref(mat1_div_sig, mat2_div_sig, norm_sq_mat1, norm_sq_mat2, out)
    out.mul_(-0.5)
    out.exp_()
    return out


def laplacian_core_ref(mat1: torch.Tensor, mat2: torch.Tensor, out: Optional[torch.Tensor], sigma: torch.Tensor) -> torch.Tensor:
    """Follows falkon/kernels/distance_kernel.py:182-205 (``diag=False``): the clamped squared distance of the
    scaled operands (expanded norm), then ``sqrt_``, negate, ``exp_``."""
    sigma = sigma.to(device=mat1.device, dtype=mat1.dtype)
    mat1_div_sig = mat1 / sigma
    mat2_div_sig = mat2 / sigma
    out = sq_dist_ref(mat1_div_sig, mat2_div_sig, square_norm_ref(mat1_div_sig), square_norm_ref(mat2_div_sig), out)
    out.sqrt_()
    out.neg_()
    out.exp_()
    return out


def matern_core_ref(mat1: torch.Tensor, mat2: torch.Tensor, out: Optional[torch.Tensor], sigma: torch.Tensor,
                    nu: float) -> torch.Tensor:
    """Follows falkon/kernels/distance_kernel.py:225-269 (``diag=False``): nu = 0.5 and inf delegate to the
    Laplacian and Gaussian cores; 1.5: ``D*sqrt(3)``, ``exp(-.)`` on a copy, ``(. + 1) * exp``; 2.5:
    ``sqrt(D2)*sqrt(5)`` on a copy, ``D2 * 5/3 + . + 1``, times ``exp(-.)``."""
    if nu == 0.5:
        return laplacian_core_ref(mat1, mat2, out, sigma)
    if nu == float("inf"):
        return rbf_core_ref(mat1, mat2, out, sigma)
    sigma = sigma.to(device=mat1.device, dtype=mat1.dtype)
    mat1_div_sig = mat1 / sigma
    mat2_div_sig = mat2 / sigma
    out = sq_dist_ref(mat1_div_sig, mat2_div_sig, square_norm_ref(mat1_div_sig), square_norm_ref(mat2_div_sig), out)
    if nu == 1.5:
        out.sqrt_()
        out.mul_(3.0 ** 0.5)
        out_neg = torch.neg(out)
        out_neg.exp_()
        out.add_(1.0).mul_(out_neg)
    elif nu == 2.5:
        out_sqrt = torch.sqrt(out)
        out_sqrt.mul_(5.0 ** 0.5)
        out.mul_(5.0 / 3.0).add_(out_sqrt).add_(1.0)
        out_sqrt.neg_().exp_()
        out.mul_(out_sqrt)
    else:
        raise ValueError(f"nu = {nu} has no closed form")
    return out


def core_ref_for(kernel_name: str):
    """The per-block function for a kernel name as the reference spells it ("gaussian", "laplacian",
    "1.5-matern", ...), with the signature of ``rbf_core_ref``."""
    if kernel_name == "gaussian":
        return rbf_core_ref
    if kernel_name == "laplacian":
        return laplacian_core_ref
    if kernel_name.endswith("-matern"):
        nu = float(kernel_name.split("-")[0])
        return lambda mat1, mat2, out, sigma: matern_core_ref(mat1, mat2, out, sigma, nu)
    raise ValueError(kernel_name)
