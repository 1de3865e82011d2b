"""Explicit kernel matrix K(X1, X2), needed once per fit for the preconditioner's K_MM.

Not on the kernel-vector hot path: the blocks are produced by the kernel's ``compute`` with stock
torch-ROCm ops, as the reference's GPU path does (falkon/mmv_ops/fmm.py:298-388).  With
``opt.no_single_kernel`` fp32 inputs are computed in fp64 and stored in fp32
(falkon/mmv_ops/fmm.py:619-622).
"""
from typing import Optional

import torch

from ..options import BaseOptions
from .utils import check_contiguity, create_output_mat, usable_gpu_memory

__all__ = ("fmm",)


def fmm(kernel, opt: Optional[BaseOptions], out: Optional[torch.Tensor], diag: bool, X1: torch.Tensor,
        X2: torch.Tensor, kwargs_m1=None, kwargs_m2=None) -> torch.Tensor:
    opt = opt if opt is not None else BaseOptions()
    check_contiguity((X1, "X1"), (X2, "X2"), (out, "out"))
    if opt.use_cpu or not torch.cuda.is_available():
        raise RuntimeError("falkon_amd computes kernel matrices on the GPU only")
    data_devs = (X1.device, X2.device)
    cuda_devs = [d for d in data_devs if d.type == "cuda"]
    dev = cuda_devs[0] if cuda_devs else torch.device("cuda", torch.cuda.current_device())
    N, M = X1.shape[0], X2.shape[0]
    with torch.inference_mode():
        if diag:
            res = kernel.compute(X1.to(dev), X2.to(dev), None, diag=True)
            if out is None:
                return res.to(X1.device)
            return out.copy_(res.reshape(out.shape))
        out = create_output_mat(out, data_devs, shape=(N, M), dtype=X1.dtype, other_mat=X1)
        upcast = X1.dtype == torch.float32 and opt.no_single_kernel
        work_dt = torch.float64 if upcast else X1.dtype
        X2d = X2.to(device=dev, dtype=work_dt)
        usable = usable_gpu_memory(dev, opt.max_gpu_mem, opt.memory_slack)
        per_row = (M * 3 + X1.shape[1] * 2) * (8 if work_dt == torch.float64 else 4)
        blk = int(max(1, min(N, usable // max(per_row, 1))))
        for i in range(0, N, blk):
            li = min(blk, N - i)
            x1 = X1[i:i + li].to(device=dev, dtype=work_dt)
            if out.device == dev and not upcast:
                kernel.compute(x1, X2d, out[i:i + li], diag=False)
            else:
                out[i:i + li].copy_(kernel.compute(x1, X2d, None, diag=False))
    return out
