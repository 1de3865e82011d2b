"""Kernel base class: the plugin API whose ``mmv`` / ``dmmv`` this build sits behind.

Same public surface as falkon/kernels/kernel.py:14-577: argument validation, per-call option
override by ``dataclasses.replace``, and the ``_decide_*_impl`` hooks that pick the backend
callable.  The hooks return this build's ``fmmv`` / ``fdmmv`` (MI355X only).
"""
import dataclasses
from abc import ABC, abstractmethod
from typing import Dict, Optional

import torch

from ..mmv_ops.fmm import fmm
from ..mmv_ops.fmmv import fdmmv, fmmv
from ..options import FalkonOptions
from ..utils.helpers import check_same_device, check_same_dtype

__all__ = ("Kernel",)


class Kernel(torch.nn.Module, ABC):
    def __init__(self, name: str, opt: Optional[FalkonOptions]):
        super().__init__()
        self.name = name
        self.params: FalkonOptions = opt if opt is not None else FalkonOptions()

    # -- validation: the checks, exception types and order of falkon/kernels/kernel.py:44-127 -------------
    @staticmethod
    def _need_matrix(name: str, t: torch.Tensor) -> None:
        if t.dim() != 2:
            raise ValueError(f"Matrix {name} must be 2D.")

    @staticmethod
    def _as_columns(name: str, t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        """A 1-D right-hand side becomes one column; anything but 1-D / 2-D is refused."""
        if t is None:
            return None
        if t.dim() == 1:
            t = t.reshape((-1, 1))
        if t.dim() != 2:
            raise ValueError(f"{name} must be a vector or a 2D matrix. Found {t.dim()}D.")
        return t

    @staticmethod
    def _need_shape(what: str, t: Optional[torch.Tensor], rows: int, cols: int) -> None:
        if t is not None and tuple(t.shape) != (rows, cols):
            raise ValueError(f"{what}: Expected ({rows}, {cols}) found {tuple(t.shape)}")

    @staticmethod
    def _need_one_dtype(*tensors) -> None:
        if not check_same_dtype(*tensors):
            raise TypeError("Data types of input matrices must be equal.")

    @staticmethod
    def _check_dmmv_dimensions(X1, X2, v, w, out):
        if v is None and w is None:
            raise ValueError("One of v and w must be specified to run fdMMV.")
        Kernel._need_matrix("X1", X1)
        Kernel._need_matrix("X2", X2)
        v, w = Kernel._as_columns("v", v), Kernel._as_columns("w", w)
        n, m = X1.shape[0], X2.shape[0]
        t = (v if v is not None else w).shape[1]
        Kernel._need_shape("Output dimension is incorrect", out, m, t)
        Kernel._need_shape("Dimensions of matrix v are incorrect", v, m, t)
        Kernel._need_shape("Dimensions of matrix w are incorrect", w, n, t)
        Kernel._need_one_dtype(X1, X2, v, w, out)
        return X1, X2, v, w, out

    @staticmethod
    def _check_mmv_dimensions(X1, X2, v, out):
        Kernel._need_matrix("X1", X1)
        Kernel._need_matrix("X2", X2)
        v = Kernel._as_columns("v", v)
        t = v.shape[1]
        Kernel._need_shape("Output dimension is incorrect", out, X1.shape[0], t)
        Kernel._need_shape("Dimensions of matrix v are incorrect", v, X2.shape[0], t)
        Kernel._need_one_dtype(X1, X2, v, out)
        return X1, X2, v, out

    @staticmethod
    def _check_mm_dimensions(X1, X2, diag, out):
        Kernel._need_matrix("X1", X1)
        Kernel._need_matrix("X2", X2)
        n, m = X1.shape[0], X2.shape[0]
        if diag:
            if n != m:
                raise ValueError(f"Cannot compute the kernel diagonal between matrices with {n} and {m} samples.")
            if out is not None and out.numel() != n:
                raise ValueError(f"Output dimension is incorrect. Expected ({n}) found {tuple(out.shape)}.")
        else:
            Kernel._need_shape("Output dimension is incorrect", out, n, m)
        Kernel._need_one_dtype(X1, X2, out)
        return X1, X2, out

    @staticmethod
    def _check_device_properties(*tensors, fn_name: str, opt):
        if not check_same_device(*tensors):
            raise RuntimeError(f"All input arguments to {fn_name} must be on the same device")

    def _merged(self, opt: Optional[FalkonOptions]) -> FalkonOptions:
        """Per-call options override the kernel's own (falkon/kernels/kernel.py:283-285)."""
        if opt is None:
            return self.params
        return dataclasses.replace(self.params, **dataclasses.asdict(opt))

    # -- kernel matrix (falkon/kernels/kernel.py:135-224) ----------------------------------------
    def __call__(self, X1, X2, diag: bool = False, out=None, opt: Optional[FalkonOptions] = None,
                 kwargs_m1: Optional[Dict[str, torch.Tensor]] = None, kwargs_m2: Optional[Dict[str, torch.Tensor]] = None):
        """The kernel matrix ``K(X1, X2)`` (N x M), or its diagonal when ``diag``."""
        X1, X2, out = self._check_mm_dimensions(X1, X2, diag, out)
        self._check_device_properties(X1, X2, out, fn_name="kernel", opt=opt)
        params = self._merged(opt)
        mm_impl = self._decide_mm_impl(X1, X2, diag, params)
        return mm_impl(kernel=self, opt=params, out=out, diag=diag, X1=X1, X2=X2, kwargs_m1=kwargs_m1,
                       kwargs_m2=kwargs_m2)

    def _decide_mm_impl(self, X1, X2, diag: bool, opt: FalkonOptions):
        return fmm

    # -- products (falkon/kernels/kernel.py:226-459) --------------------------------------------
    def mmv(self, X1, X2, v, out=None, opt: Optional[FalkonOptions] = None,
            kwargs_m1: Optional[Dict[str, torch.Tensor]] = None, kwargs_m2: Optional[Dict[str, torch.Tensor]] = None):
        """``K(X1, X2) @ v``: X1 (N x D), X2 (M x D), v (M x T) or (M,), result (N x T)."""
        X1, X2, v, out = self._check_mmv_dimensions(X1, X2, v, out)
        params = self._merged(opt)
        mmv_impl = self._decide_mmv_impl(X1, X2, v, params)
        return mmv_impl(X1=X1, X2=X2, v=v, kernel=self, out=out, opt=params, kwargs_m1=kwargs_m1, kwargs_m2=kwargs_m2)

    def _decide_mmv_impl(self, X1, X2, v, opt: FalkonOptions):
        return fmmv

    def dmmv(self, X1, X2, v, w, out=None, opt: Optional[FalkonOptions] = None,
             kwargs_m1: Optional[Dict[str, torch.Tensor]] = None, kwargs_m2: Optional[Dict[str, torch.Tensor]] = None):
        """``K(X1, X2).T @ (K(X1, X2) @ v + w)``: v (M x T), w (N x T) or None, result (M x T)."""
        X1, X2, v, w, out = self._check_dmmv_dimensions(X1, X2, v, w, out)
        params = self._merged(opt)
        dmmv_impl = self._decide_dmmv_impl(X1, X2, v, w, params)
        return dmmv_impl(X1=X1, X2=X2, v=v, w=w, kernel=self, out=out, differentiable=False, opt=params,
                         kwargs_m1=kwargs_m1, kwargs_m2=kwargs_m2)

    def _decide_dmmv_impl(self, X1, X2, v, w, opt: FalkonOptions):
        return fdmmv

    @abstractmethod
    def compute(self, X1: torch.Tensor, X2: torch.Tensor, out: torch.Tensor, diag: bool, **kwargs) -> torch.Tensor:
        """Fill ``out`` with the kernel matrix of ``X1`` and ``X2`` (falkon/kernels/kernel.py:461-497)."""

    def extra_mem(self, is_differentiable, is_sparse, dtype, density1=None, density2=None) -> Dict[str, float]:
        return {}

    def __str__(self):
        return f"<{self.name} kernel>"
