"""Kernels whose hyper-parameters are registered torch parameters (falkon/kernels/diff_kernel.py:13-145)."""
import abc
from typing import Any, Dict, Optional

import torch
from torch import nn

from ..options import FalkonOptions
from .kernel import Kernel

__all__ = ("DiffKernel",)


class DiffKernel(Kernel, abc.ABC):
    """Tensor-valued hyper-parameters become ``nn.Parameter`` s of the module (so they show up in
    ``named_parameters`` and can carry gradients), everything else is kept as a plain attribute; both kinds
    are handed to ``core_fn`` by keyword."""

    def __init__(self, name, options, core_fn, **kernel_params):
        super().__init__(name=name, opt=options)
        self.core_fn = core_fn
        tensors = {key: val for key, val in kernel_params.items() if isinstance(val, torch.Tensor)}
        self._other_params = {key: val for key, val in kernel_params.items() if key not in tensors}
        for key, val in tensors.items():
            self.register_parameter(key, nn.Parameter(val, requires_grad=val.requires_grad))
        for key, val in self._other_params.items():
            setattr(self, key, val)

    @property
    def diff_params(self) -> Dict[str, torch.Tensor]:
        return {key: par for key, par in self.named_parameters()}

    @property
    def nondiff_params(self) -> Dict[str, Any]:
        return self._other_params

    def _core(self, X1, X2, out, diag: bool, extra: Dict[str, Any]):
        return self.core_fn(X1, X2, out=out, diag=diag, **extra, **self.diff_params, **self._other_params)

    def compute(self, X1, X2, out, diag: bool, **kwargs):
        return self._core(X1, X2, out, diag, kwargs)

    def compute_diff(self, X1, X2, diag: bool, **kwargs):
        return self._core(X1, X2, None, diag, kwargs)

    @abc.abstractmethod
    def detach(self) -> "Kernel":
        """A copy of the kernel whose parameters are detached from any autograd graph."""

    def dmmv(self, X1, X2, v, w, out=None, opt: Optional[FalkonOptions] = None):
        """Same as :meth:`Kernel.dmmv`, but tells the backend whether any input wants gradients
        (falkon/kernels/diff_kernel.py:127-145); the backend is called positionally, as there."""
        X1, X2, v, w, out = self._check_dmmv_dimensions(X1, X2, v, w, out)
        params = self._merged(opt)
        backend = self._decide_dmmv_impl(X1, X2, v, w, params)
        operands = [t for t in (X1, X2, v, w) if t is not None] + list(self.diff_params.values())
        wants_grad = any(t.requires_grad for t in operands)
        return backend(X1, X2, v, w, self, out, wants_grad, params)
