"""Kernels whose hyper-parameters are registered torch parameters (falkon/kernels/diff_kernel.py:13-145)."""
import abc
from typing import Any, Dict, Optional

import torch
from torch import nn

from ..options import FalkonOptions
from .kernel import Kernel

__all__ = ("DiffKernel",)


class DiffKernel(Kernel, abc.ABC):
    def __init__(self, name, options, core_fn, **kernel_params):
        super().__init__(name=name, opt=options)
        self.core_fn = core_fn
        self._other_params = {}
        for k, v in kernel_params.items():
            if isinstance(v, torch.Tensor):
                self.register_parameter(k, nn.Parameter(v, requires_grad=v.requires_grad))
            else:
                self._other_params[k] = v
                setattr(self, k, v)

    @property
    def diff_params(self) -> Dict[str, torch.Tensor]:
        return dict(self.named_parameters())

    @property
    def nondiff_params(self) -> Dict[str, Any]:
        return self._other_params

    def compute(self, X1, X2, out, diag: bool, **kwargs):
        return self.core_fn(X1, X2, out=out, diag=diag, **kwargs, **self.diff_params, **self._other_params)

    def compute_diff(self, X1, X2, diag: bool, **kwargs):
        return self.core_fn(X1, X2, out=None, diag=diag, **kwargs, **self.diff_params, **self._other_params)

    @abc.abstractmethod
    def detach(self) -> "Kernel":
        """A copy of the kernel whose parameters are detached from any autograd graph."""

    def dmmv(self, X1, X2, v, w, out=None, opt: Optional[FalkonOptions] = None):
        """Same as :meth:`Kernel.dmmv`, but tells the backend whether any input wants gradients
        (falkon/kernels/diff_kernel.py:127-145); the backend is called positionally, as there."""
        X1, X2, v, w, out = self._check_dmmv_dimensions(X1, X2, v, w, out)
        params = self._merged(opt)
        dmmv_impl = self._decide_dmmv_impl(X1, X2, v, w, params)
        diff = any(t.requires_grad for t in [X1, X2, v, w] + list(self.diff_params.values()) if t is not None)
        return dmmv_impl(X1, X2, v, w, self, out, diff, params)
