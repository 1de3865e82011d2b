"""Generalised self-concordant losses for ``LogisticFalkon`` (falkon/gsc_losses.py:14-435).

A loss is a function l(true, pred) with its first and second derivative in ``pred``, plus the two kernel products
Newton's method needs, both of which are two ``kernel.mmv`` calls on the MI355X path:

    knmp_grad(X, Xc, Y, u)    = K(Xc, X) l'(Y, K(X, Xc) u) / n        (and the function values K(X, Xc) u)
    knmp_hess(X, Xc, Y, f, u) = K(Xc, X) (l''(Y, f) * K(X, Xc) u) / n

The derivatives are written with ``sigmoid`` / ``softplus`` (no overflow for large |pred|).
"""
import dataclasses
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from .options import FalkonOptions

__all__ = ("Loss", "LogisticLoss", "WeightedCrossEntropyLoss")


class Loss:
    def __init__(self, name: str, kernel, opt: Optional[FalkonOptions] = None):
        self.name, self.kernel, self.params = name, kernel, opt or FalkonOptions()

    def _update_opt(self, opt: Optional[FalkonOptions]) -> FalkonOptions:
        return self.params if opt is None else dataclasses.replace(self.params, **dataclasses.asdict(opt))

    def __call__(self, y1: torch.Tensor, y2: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def df(self, y1: torch.Tensor, y2: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def ddf(self, y1: torch.Tensor, y2: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def knmp_grad(self, X, Xc, Y, u, opt: Optional[FalkonOptions] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        """(K(Xc, X) l'(Y, f) / n, f) with f = K(X, Xc) u (falkon/gsc_losses.py:96-139)."""
        opt = self._update_opt(opt)
        func_val = self.kernel.mmv(X, Xc, u, opt=opt)
        out = self.kernel.mmv(Xc, X, self.df(Y, func_val), opt=opt)
        return out.mul_(1.0 / X.shape[0]), func_val

    def knmp_hess(self, X, Xc, Y, f, u, opt: Optional[FalkonOptions] = None) -> torch.Tensor:
        """K(Xc, X) (l''(Y, f) * K(X, Xc) u) / n (falkon/gsc_losses.py:141-190)."""
        opt = self._update_opt(opt)
        inner = self.kernel.mmv(X, Xc, u, opt=opt).mul_(self.ddf(Y, f))
        return self.kernel.mmv(Xc, X, inner, opt=opt).mul_(1.0 / X.shape[0])

    def __str__(self):
        return self.name


class LogisticLoss(Loss):
    """l(y, p) = log(1 + exp(-y p)) for labels y in {-1, +1} (falkon/gsc_losses.py:196-292)."""

    def __init__(self, kernel, opt: Optional[FalkonOptions] = None):
        super().__init__("LogisticLoss", kernel, opt)

    def __call__(self, y1, y2):
        return F.softplus(-y1 * y2)

    def df(self, y1, y2):
        return -y1 * torch.sigmoid(-y1 * y2)

    def ddf(self, y1, y2):
        s = torch.sigmoid(y1 * y2)
        return y1 * y1 * s * (1 - s)

    def __repr__(self):
        return f"LogisticLoss(kernel={self.kernel})"


class WeightedCrossEntropyLoss(Loss):
    """l(t, p) = t log(1 + exp(-p)) + w (1 - t) log(1 + exp(p)) for labels t in {0, 1}, w the weight of the
    negative class (falkon/gsc_losses.py:295-435)."""

    def __init__(self, kernel, neg_weight: float, opt: Optional[FalkonOptions] = None):
        super().__init__("WeightedCrossEntropy", kernel, opt)
        self.neg_weight = neg_weight

    def __call__(self, true, pred):
        return true * F.softplus(-pred) + self.neg_weight * (1 - true) * F.softplus(pred)

    def df(self, true, pred):
        s = torch.sigmoid(pred)
        return self.neg_weight * (1 - true) * s - true * (1 - s)

    def ddf(self, true, pred):
        s = torch.sigmoid(pred)
        return (true + self.neg_weight * (1 - true)) * s * (1 - s)

    def __repr__(self):
        return f"WeightedCrossEntropy(kernel={self.kernel})"
