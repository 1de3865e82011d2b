"""Nystroem centre selection (falkon/center_selection.py:17-281): uniform without replacement, or fixed."""
import warnings
from abc import ABC, abstractmethod
from typing import Optional

import numpy as np
import torch

from .utils.tensor_helpers import create_same_stride

__all__ = ("CenterSelector", "UniformSelector", "FixedSelector")


class CenterSelector(ABC):
    def __init__(self, random_gen):
        self.random_gen = random_gen if isinstance(random_gen, np.random.Generator) else np.random.default_rng(random_gen)

    @abstractmethod
    def select_indices(self, X, Y):
        pass

    def select(self, X, Y):
        res = self.select_indices(X, Y)
        return res[0] if len(res) == 2 else (res[0], res[1])


class UniformSelector(CenterSelector):
    """``idx = rng.choice(N, M, replace=False)`` then a row gather that keeps device and memory order
    (falkon/center_selection.py:187-248)."""

    def __init__(self, random_gen, num_centers: int):
        self.num_centers = num_centers
        super().__init__(random_gen)

    def select_indices(self, X: torch.Tensor, Y: Optional[torch.Tensor]):
        N, M = X.shape[0], self.num_centers
        if M > N:
            warnings.warn(f"Number of centers M greater than the number of data-points. Setting `num_centers` to {N}",
                          stacklevel=2)
            M = N
        idx = self.random_gen.choice(N, size=M, replace=False).astype(np.int64)
        th_idx = torch.from_numpy(idx).to(X.device)
        Xc = create_same_stride((M, X.shape[1]), X, X.dtype, X.device)
        torch.index_select(X, 0, th_idx, out=Xc)
        if Y is None:
            return Xc, th_idx
        Yc = create_same_stride((M, Y.shape[1]), Y, Y.dtype, Y.device)
        torch.index_select(Y, 0, th_idx.to(Y.device), out=Yc)
        return Xc, Yc, th_idx


class FixedSelector(CenterSelector):
    """Centres given up front (falkon/center_selection.py:57-163)."""

    def __init__(self, centers, y_centers=None, idx_centers=None):
        super().__init__(0)
        self.centers, self.y_centers, self.idx_centers = centers, y_centers, idx_centers

    def _with_targets(self, want_targets: bool, *tail):
        """(centres[, their targets], *tail); asking for targets that were never supplied is an error."""
        if not want_targets:
            return (self.centers, *tail)
        if self.y_centers is None:
            raise RuntimeError("FixedSelector has no y-centers available, but `Y` is not None.")
        return (self.centers, self.y_centers, *tail)

    def select(self, X, Y):
        picked = self._with_targets(Y is not None)
        return picked[0] if len(picked) == 1 else picked

    def select_indices(self, X, Y):
        if self.idx_centers is None:
            raise RuntimeError("`select_indices` method called but no indices were provided.")
        return self._with_targets(Y is not None, self.idx_centers)
