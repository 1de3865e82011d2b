"""Option dataclasses with the reference's field names and defaults.

Mirrors falkon/options.py:164-303 (``BaseOptions``, ``KeopsOptions``,
``ConjugateGradientOptions``, ``PreconditionerOptions``, ``CholeskyOptions``,
``FalkonOptions``) so that code written against ``falkon.FalkonOptions`` keeps
working.  On the kernel-vector path this build reads ``use_cpu``,
``max_gpu_mem`` and ``memory_slack``; the other fields are carried for the callers.
"""
from dataclasses import dataclass

import numpy as np
import torch

__all__ = ("BaseOptions", "KeopsOptions", "ConjugateGradientOptions", "PreconditionerOptions",
           "CholeskyOptions", "FalkonOptions")


@dataclass
class BaseOptions:
    debug: bool = False
    use_cpu: bool = False
    max_gpu_mem: float = np.inf
    max_cpu_mem: float = np.inf
    compute_arch_speed: bool = False
    no_single_kernel: bool = True
    min_cuda_pc_size_32: int = 10000
    min_cuda_pc_size_64: int = 30000
    min_cuda_iter_size_32: int = 10_000 * 10 * 3_000
    min_cuda_iter_size_64: int = 30_000 * 10 * 3_000
    never_store_kernel: bool = False
    store_kernel_d_threshold: int = 1200
    num_fmm_streams: int = 2
    memory_slack: float = 0.9


@dataclass
class KeopsOptions:
    keops_acc_dtype: str = "auto"
    keops_sum_scheme: str = "auto"
    keops_active: str = "auto"
    keops_memory_slack: float = 0.7


@dataclass
class ConjugateGradientOptions:
    cg_epsilon_32: float = 1e-7
    cg_epsilon_64: float = 1e-15
    cg_tolerance: float = 1e-7
    cg_full_gradient_every: int = 10
    cg_differential_convergence: bool = False

    def cg_epsilon(self, dtype):
        if dtype == torch.float32:
            return self.cg_epsilon_32
        if dtype == torch.float64:
            return self.cg_epsilon_64
        raise TypeError(f"Data-type {str(dtype)} invalid")


@dataclass
class PreconditionerOptions:
    pc_epsilon_32: float = 1e-5
    pc_epsilon_64: float = 1e-13
    cpu_preconditioner: bool = False

    def pc_epsilon(self, dtype):
        if dtype == torch.float32:
            return self.pc_epsilon_32
        if dtype == torch.float64:
            return self.pc_epsilon_64
        raise TypeError(f"Data-type {str(dtype)} invalid")


@dataclass
class CholeskyOptions:
    chol_force_in_core: bool = False
    chol_force_ooc: bool = False
    chol_par_blk_multiplier: int = 2


@dataclass
class FalkonOptions(BaseOptions, ConjugateGradientOptions, PreconditionerOptions, CholeskyOptions, KeopsOptions):
    """Global options, same fields as falkon/options.py:293-303."""
    pass
