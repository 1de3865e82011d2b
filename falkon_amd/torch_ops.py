"""``torch.ops.falkon.*`` entries for the MI355X kernel-vector products.

The reference reaches its native code through ``torch.ops.falkon.<name>`` (schema in
falkon/c_ext/ops/square_norm.cpp:23-26, lazy lookup in falkon/c_ext/__init__.py:13-21).  Importing this module
registers the two products of this build the same way, for callers that dispatch through ``torch.ops``:

    torch.ops.falkon.kernel_fmmv(X1, X2, sigma, v, out, kernel_fn=0, bf16x3=False)        out <- K(X1, X2) @ v
    torch.ops.falkon.kernel_fdmmv(X1, X2, sigma, v, w, out, kernel_fn=0, bf16x3=False)    out <- K^T (K v + w)

All tensors are 2-D (``sigma`` 1-D with 1 or d entries), on one GPU, of one dtype; ``out`` is overwritten in place;
``kernel_fn`` is the library's kernel code (0 Gaussian, 1 Laplacian, 2 Matern 3/2, 3 Matern 5/2).  The ops enqueue on
the current stream and do not synchronise.  They are thin: argument checks beyond what the C ABI does itself live in
``falkon_amd.kernels`` / ``falkon_amd.mmv_ops.fmmv``.
"""
from typing import Optional

import torch

from . import _backend
from .mmv_ops.fmmv import gauss_fdmmv_native, gauss_fmmv_native

__all__ = ("kernel_fmmv", "kernel_fdmmv")


def _code(X1: torch.Tensor, bf16x3: bool) -> int:
    if X1.dtype == torch.float32:
        return _backend.FLK_F32_BF16X3 if bf16x3 else _backend.FLK_F32
    if X1.dtype == torch.float64:
        return _backend.FLK_F64
    raise TypeError(f"falkon kernel products take float32 or float64 tensors, not {X1.dtype}")


def _check(X1, *others):
    if X1.device.type != "cuda":
        raise RuntimeError("falkon kernel products run on the GPU only: tensors must be on a ROCm device")
    for t in others:
        if t is not None and (t.device != X1.device or t.dtype != X1.dtype):
            raise TypeError("all tensors of a falkon kernel product must share one device and one dtype")


@torch.library.custom_op("falkon::kernel_fmmv", mutates_args=("out",))
def kernel_fmmv(X1: torch.Tensor, X2: torch.Tensor, sigma: torch.Tensor, v: torch.Tensor, out: torch.Tensor,
                kernel_fn: int = 0, bf16x3: bool = False) -> None:
    _check(X1, X2, sigma, v, out)
    gauss_fmmv_native(X1, X2, sigma.reshape(-1).contiguous(), v, out, kernel_fn, _code(X1, bf16x3))


@torch.library.custom_op("falkon::kernel_fdmmv", mutates_args=("out",))
def kernel_fdmmv(X1: torch.Tensor, X2: torch.Tensor, sigma: torch.Tensor, v: torch.Tensor, w: Optional[torch.Tensor],
                 out: torch.Tensor, kernel_fn: int = 0, bf16x3: bool = False) -> None:
    _check(X1, X2, sigma, v, w, out)
    gauss_fdmmv_native(X1, X2, sigma.reshape(-1).contiguous(), v, w, out, kernel_fn, _code(X1, bf16x3))
