"""Gradients of the kernel-vector product and of the kernel matrix as the reference computes them: torch autograd
through the kernel's core function on CPU.

Test infrastructure only (see ``oracle/__init__.py``).

The reference's backward pass re-runs the product block by block under autograd and asks for
``torch.autograd.grad(K_block @ v_block, inputs, grad_outputs=G_block)`` (falkon/mmv_ops/fmmv.py:405-485), summing
the blocks; the kernel matrix goes through ``sum(K_block * G_block)`` (falkon/mmv_ops/fmm.py:391-438,648-696).
The graph that gets differentiated is that of the core functions (falkon/kernels/distance_kernel.py:140-159,
182-205, 225-269): operands divided by sigma, squared distance through the expanded norm (:88-101), clamped at
1e-20, then the radial function.  ``radial_kernel_autograd`` restates that graph without the in-place updates
(which only save memory); blocks add up to the unblocked result, so one block is used.

Pinned (tests/test_oracle.py) against autograd through the difference form ``sum_k ((x_k - c_k)/sigma_k)^2`` in
fp64 and against central finite differences.
"""
from typing import Optional, Sequence, Tuple

import torch

_SCALE = {"1.5-matern": 3.0 ** 0.5, "2.5-matern": 5.0 ** 0.5}


def radial_kernel_autograd(X1: torch.Tensor, X2: torch.Tensor, sigma: torch.Tensor, kernel_name: str) -> torch.Tensor:
    """K(X1, X2) as a differentiable torch expression with the reference's arithmetic (expanded norm, clamp)."""
    sigma = sigma.to(device=X1.device, dtype=X1.dtype)
    a, b = X1 / sigma, X2 / sigma
    d2 = torch.addmm((a * a).sum(-1, keepdim=True), a, b.T, alpha=-2, beta=1) + (b * b).sum(-1, keepdim=True).T
    d2 = d2.clamp_min(1e-20)
    if kernel_name in ("gaussian", "inf-matern"):
        return torch.exp(-0.5 * d2)
    if kernel_name in ("laplacian", "0.5-matern"):
        return torch.exp(-torch.sqrt(d2))
    s = torch.sqrt(d2) * _SCALE[kernel_name]
    if kernel_name == "1.5-matern":
        return (s + 1.0) * torch.exp(-s)
    return (d2 * (5.0 / 3.0) + s + 1.0) * torch.exp(-s)          # 2.5-matern: s^2/3 = 5/3 D^2


def radial_kernel_difference_form(X1, X2, sigma, kernel_name: str) -> torch.Tensor:
    """The same kernels from the definition, D = |(x - c)/sigma| formed entry by entry (no expanded norm, no clamp
    except under the square root of exactly coincident points): the check of ``radial_kernel_autograd``."""
    sigma = sigma.to(device=X1.device, dtype=X1.dtype)
    diff = (X1[:, None, :] - X2[None, :, :]) / sigma
    d2 = (diff * diff).sum(-1)
    if kernel_name in ("gaussian", "inf-matern"):
        return torch.exp(-0.5 * d2)
    dist = torch.sqrt(d2.clamp_min(1e-300))
    if kernel_name in ("laplacian", "0.5-matern"):
        return torch.exp(-dist)
    s = dist * _SCALE[kernel_name]
    if kernel_name == "1.5-matern":
        return (1 + s) * torch.exp(-s)
    return (1 + s + s * s / 3) * torch.exp(-s)


def _leaves(tensors, needs):
    return [t.detach().clone().requires_grad_(bool(n)) for t, n in zip(tensors, needs)]


def fmmv_grads_ref(X1, X2, v, sigma, G, kernel_name: str = "gaussian",
                   needs: Sequence[bool] = (True, True, True, True), kernel_fn=radial_kernel_autograd
                   ) -> Tuple[Optional[torch.Tensor], ...]:
    """(dL/dX1, dL/dX2, dL/dv, dL/dsigma) for L = sum(G * (K(X1, X2) @ v)); None where ``needs`` is False."""
    x1, x2, vv, sg = _leaves((X1, X2, v, sigma), needs)
    out = kernel_fn(x1, x2, sg, kernel_name) @ vv
    wanted = [t for t in (x1, x2, vv, sg) if t.requires_grad]
    got = iter(torch.autograd.grad(out, wanted, grad_outputs=G.to(out.dtype)))
    return tuple(next(got) if t.requires_grad else None for t in (x1, x2, vv, sg))


def fmm_grads_ref(X1, X2, sigma, G, kernel_name: str = "gaussian", needs: Sequence[bool] = (True, True, True),
                  kernel_fn=radial_kernel_autograd) -> Tuple[Optional[torch.Tensor], ...]:
    """(dL/dX1, dL/dX2, dL/dsigma) for L = sum(G * K(X1, X2))."""
    x1, x2, sg = _leaves((X1, X2, sigma), needs)
    out = kernel_fn(x1, x2, sg, kernel_name)
    wanted = [t for t in (x1, x2, sg) if t.requires_grad]
    got = iter(torch.autograd.grad(out, wanted, grad_outputs=G.to(out.dtype)))
    return tuple(next(got) if t.requires_grad else None for t in (x1, x2, sg))
