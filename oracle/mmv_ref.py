"""Blocked CPU drivers of the reference's ``fmmv`` / ``fdmmv``, restated in torch CPU ops.

Test infrastructure only (see ``oracle/__init__.py``).  This is the path the
reference takes for ``FalkonOptions(use_cpu=True, keops_active="no")`` with
dense, non-differentiable inputs that all live on the host:
``fmmv`` -> ``KernelMmvFnFull.run_cpu_cpu`` -> ``mmv_run_starter`` -> ``mmv_run_thread``
and ``fdmmv`` -> ``dmmv_run_starter(device_id=-1)`` -> ``dmmv_run_thread``.
"""
import math
from typing import Optional, Tuple

import torch

from .gaussian_ref import core_ref_for, rbf_core_ref, validate_sigma_ref

# falkon/mmv_ops/utils.py:44 -- head-room the reference reserves for addmm work buffers
EXTRA_MM_RAM_BYTES = 8519680


def sizeof_dtype_ref(dtype: torch.dtype) -> int:
    """falkon/utils/helpers.py:225-238."""
    if dtype == torch.float64:
        return 8
    if dtype == torch.float32:
        return 4
    raise TypeError(f"Dtype {dtype} not valid")


# ---------------------------------------------------------------------------
# stride helpers (falkon/utils/tensor_helpers.py:149-213)
# ---------------------------------------------------------------------------
def is_f_contig_strict_ref(t: torch.Tensor) -> bool:
    """``is_f_contig(t, strict=True)`` of falkon/utils/tensor_helpers.py:149-198."""
    st, sz = t.stride(), t.shape
    if len(sz) == 0:
        return True
    if len(sz) == 1:
        return st[0] == 1
    if sz[-2] == 1:
        return st[-2] == 1
    if sz[-1] == 1:
        return st[-2] == 1 and st[-1] >= sz[-2]
    return st[-2] == 1 and st[-1] >= st[-2]


def is_contig_ref(t: torch.Tensor) -> bool:
    """falkon/utils/tensor_helpers.py:210-213: some stride equals one."""
    return any(s == 1 for s in t.stride())


def _alloc_like_order(shape, other: torch.Tensor, dtype) -> torch.Tensor:
    """falkon/utils/tensor_helpers.py:128-140 (``create_same_stride``)."""
    if is_f_contig_strict_ref(other):
        return torch.empty_strided(shape, (1, shape[0]), dtype=dtype)
    if is_contig_ref(other):
        return torch.empty(shape, dtype=dtype)
    raise ValueError("Desired stride is not contiguous, cannot create.")


def _carve(flat: torch.Tensor, shape, other: torch.Tensor, offset: int) -> Tuple[torch.Tensor, int]:
    """falkon/mmv_ops/utils.py:108-112 + tensor_helpers.py:63-73 (``_extract_flat``)."""
    if is_f_contig_strict_ref(other):
        strides = (1, shape[0])
    elif is_contig_ref(other):
        strides = (shape[1], 1)
    else:
        raise ValueError("Desired stride is not contiguous, cannot extract.")
    return flat.as_strided(shape, strides, offset), offset + shape[0] * shape[1]


# ---------------------------------------------------------------------------
# block-size solvers (falkon/utils/helpers.py:24-31,74-85,149-195)
# ---------------------------------------------------------------------------
def _pos_root(a: float, b: float, c: float) -> float:
    """Larger root of a x^2 + b x + c (helpers.py:24-27); +inf when a == 0."""
    if a == 0:
        return float("inf")
    return (-b + math.sqrt(b * b - 4 * a * c)) / (2 * a)


def select_dim_over_n_ref(max_n, m, d, coef_nm, coef_nd, coef_md, coef_n, coef_m, coef_d, rest, max_mem) -> int:
    """helpers.py:74-85: largest n with n*(m*coef_nm + d*coef_nd + coef_n) + rest' <= max_mem."""
    per_row = m * coef_nm + d * coef_nd + coef_n
    fixed = rest + coef_md * m * d + coef_m * m + coef_d * d
    n = int(min((max_mem - fixed) / per_row, max_n))
    if n <= 0:
        raise MemoryError("Available memory %.2fMB is not enough." % (max_mem / 2**20))
    return n


def select_dim_over_nd_ref(max_n, max_d, coef_nd, coef_n, coef_d, rest, max_mem) -> Tuple[int, int]:
    """helpers.py:149-185: grow n and d together, then spend what is left on the other one."""
    if coef_nd == 0 and (coef_n == 0 or coef_d == 0):
        if coef_d == coef_n:
            n, d = max_n, max_d
        elif coef_n == 0:
            n, d = max_n, (max_mem - rest) / coef_d
        else:
            n, d = (max_mem - rest) / coef_n, max_d
    else:
        if coef_nd == 0:
            x = -(rest - max_mem) / (coef_n + coef_d)
        else:
            try:
                x = _pos_root(coef_nd, coef_n + coef_d, rest - max_mem)
            except ValueError:
                x = -1
        n = math.floor(min(max_n, x))
        d = math.floor(min(max_d, x))
        if d == max_d and n < max_n:
            n = (max_mem - rest - coef_d * d) / (coef_nd * d + coef_n)
        elif d < max_d and n == max_n:
            d = (max_mem - rest - coef_n * n) / (coef_nd * n + coef_d)
    n, d = int(min(max_n, n)), int(min(max_d, d))
    if n <= 0 or d <= 0:
        raise MemoryError(f"Available memory {max_mem / 2**20:.2f}MB is not enough.")
    return n, d


def gaussian_extra_mem_ref(dtype: torch.dtype) -> dict:
    """falkon/kernels/distance_kernel.py:41-85, dense non-differentiable Gaussian case."""
    return {"0": EXTRA_MM_RAM_BYTES / sizeof_dtype_ref(dtype), "nd": 1, "md": 1, "m": 1, "n": 1, "nm": 0}


def mmv_blk_sizes_ref(n, d, m, t, avail_elems: float, dtype) -> Tuple[int, int, int]:
    """falkon/mmv_ops/fmmv.py:60-114 with every operand in-core, dense, no grad."""
    extra = gaussian_extra_mem_ref(dtype)
    blk_n, blk_m = select_dim_over_nd_ref(
        max_n=n, max_d=m, coef_nd=1 + extra["nm"], coef_n=extra["n"] + extra["nd"] * d,
        coef_d=extra["m"] + extra["md"] * d, rest=extra["0"], max_mem=avail_elems)
    return blk_n, blk_m, blk_n * blk_m


def dmmv_blk_sizes_ref(n, d, m, t, avail_elems: float, dtype) -> Tuple[int, int]:
    """falkon/mmv_ops/fmmv.py:488-544 with every operand in-core, dense."""
    extra = gaussian_extra_mem_ref(dtype)
    blk_n = select_dim_over_n_ref(
        max_n=n, m=m, d=d, coef_nm=1 + extra["nm"], coef_nd=extra["nd"], coef_md=extra["md"],
        coef_n=1 * t + extra["n"], coef_m=0 * t + extra["m"], coef_d=0, rest=extra["0"], max_mem=avail_elems)
    return blk_n, blk_n * (m + t)


# ---------------------------------------------------------------------------
# drivers
# ---------------------------------------------------------------------------
def _check_inputs(X1, X2, v, w, out, out_rows):
    """Argument checks of falkon/kernels/kernel.py:44-105 + mmv_ops/utils.py:36-39."""
    if X1.dim() != 2:
        raise ValueError("Matrix X1 must be 2D.")
    if X2.dim() != 2:
        raise ValueError("Matrix X2 must be 2D.")
    if v is not None and v.dim() == 1:
        v = v.reshape(-1, 1)
    if w is not None and w.dim() == 1:
        w = w.reshape(-1, 1)
    T = v.shape[1] if v is not None else w.shape[1]
    if v is not None and v.shape != (X2.shape[0], T):
        raise ValueError("Dimensions of matrix v are incorrect")
    if w is not None and w.shape != (X1.shape[0], T):
        raise ValueError("Dimensions of matrix w are incorrect")
    if out is not None and tuple(out.shape) != (out_rows, T):
        raise ValueError("Output dimension is incorrect.")
    dts = {a.dtype for a in (X1, X2, v, w, out) if a is not None}
    if len(dts) != 1:
        raise TypeError("Data types of input matrices must be equal.")
    for a, name in ((X1, "X1"), (X2, "X2"), (v, "v"), (out, "out")):
        if a is not None and not is_contig_ref(a):
            raise ValueError(f"Tensor '{name}' must be memory contiguous")
    return v, w


def fmmv_ref(X1, X2, v, sigma, out: Optional[torch.Tensor] = None, max_cpu_mem: float = float("inf"),
             kernel_name: str = "gaussian") -> torch.Tensor:
    """out[N,T] = K(X1,X2) @ v, blocked over rows of X1 and of X2.

    Follows falkon/mmv_ops/fmmv.py:887-932 (output creation), :117-185 (block
    sizes from the ``max_cpu_mem`` budget) and :309-402 (the loop: zero the
    output rows, then for every column block ``K = compute(X1_i, X2_j)`` and
    ``out_i.addmm_(K, v_j)``).
    """
    sigma = validate_sigma_ref(sigma)
    core = core_ref_for(kernel_name)        # the kernel's per-block function (the block loop is shared)
    v, _ = _check_inputs(X1, X2, v, None, out, X1.shape[0])
    N, D = X1.shape
    M, T = v.shape
    if out is None:
        out = _alloc_like_order((N, T), X1, v.dtype)
    avail = max_cpu_mem / sizeof_dtype_ref(X1.dtype)
    blk_n, blk_m, need = mmv_blk_sizes_ref(N, D, M, T, avail, X1.dtype)
    flat = torch.empty(need, dtype=X1.dtype)
    ker_buf, _ = _carve(flat, (blk_n, blk_m), out, 0)
    with torch.inference_mode():
        for i in range(0, N, blk_n):
            li = min(blk_n, N - i)
            x_i = X1[i:i + li, :]
            o_i = out[i:i + li]
            o_i.fill_(0.0)
            for j in range(0, M, blk_m):
                lj = min(blk_m, M - j)
                k_ij = ker_buf[:li, :lj].fill_(0.0)
                k_ij = core(x_i, X2[j:j + lj, :], k_ij, sigma)
                o_i.addmm_(k_ij, v[j:j + lj, :])
    return out


def fdmmv_ref(X1, X2, v, w, sigma, out: Optional[torch.Tensor] = None, max_cpu_mem: float = float("inf"),
              kernel_name: str = "gaussian") -> torch.Tensor:
    """out[M,T] = K(X1,X2).T @ (K(X1,X2) @ v + w), blocked over rows of X1.

    Follows falkon/mmv_ops/fmmv.py:1033-1061 (checks, output creation, CPU
    branch), :547-606 (block size) and :683-767 (the loop: per row block the K
    block is materialised once, ``u = w_i`` (or zeros), ``u.addmm_(K, v)``,
    ``out.addmm_(K.T, u)``).  ``v`` is required, ``w`` may be None (the
    reference reads ``v.shape`` unconditionally, fmmv.py:1041).
    """
    sigma = validate_sigma_ref(sigma)
    core = core_ref_for(kernel_name)
    v, w = _check_inputs(X1, X2, v, w, out, X2.shape[0])
    N, D = X1.shape
    M, T = v.shape
    if out is None:
        out = _alloc_like_order((M, T), X1, v.dtype)
    avail = max_cpu_mem / sizeof_dtype_ref(X1.dtype)
    blk_n, need = dmmv_blk_sizes_ref(N, D, M, T, avail, X1.dtype)
    flat = torch.empty(need, dtype=X1.dtype)
    ker_buf, off = _carve(flat, (blk_n, M), out, 0)
    u_buf, off = _carve(flat, (blk_n, T), v if w is None else w, off)
    with torch.inference_mode():
        out.fill_(0.0)
        for i in range(0, N, blk_n):
            li = min(blk_n, N - i)
            x_i = X1[i:i + li, :]
            if w is not None:
                u_i = u_buf[:li, :].copy_(w[i:i + li, :])
            else:
                u_i = u_buf[:li, :].fill_(0.0)
            k_i = ker_buf[:li, :].fill_(0.0)
            k_i = core(x_i, X2, k_i, sigma)
            u_i.addmm_(k_i, v)
            out.addmm_(k_i.T, u_i)
    return out
