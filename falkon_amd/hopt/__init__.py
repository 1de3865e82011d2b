"""Hyperparameter optimisation objectives on the MI355X kernels (the exact objectives of falkon/hopt/objectives)."""
from .objectives import (GCV, LOOCV, SGPR, CompReg, HoldOut, HyperoptObjective, NystromCompReg,  # noqa: F401
                         PositiveTransform, StochasticNystromCompReg)
