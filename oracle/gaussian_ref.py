"""Per-block Gaussian kernel arithmetic of the reference, restated in torch CPU ops.

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
