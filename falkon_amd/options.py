"""Option dataclasses with the reference's field names and defaults.

Mirrors falkon/options.py:164-303 (``BaseOptions``, ``KeopsOptions``,
``ConjugateGradientOptions``, ``PreconditionerOptions``, ``CholeskyOptions``,
``FalkonOptions``) so that code written against ``falkon.FalkonOptions`` keeps
working.  The comment after each field says what this build does with it.
"""
from dataclasses import dataclass

import numpy as np
import torch

__all__ = ("BaseOptions", "KeopsOptions", "ConjugateGradientOptions", "PreconditionerOptions",
           "CholeskyOptions", "FalkonOptions")


def _by_precision(dtype, single, double):
    """The fp32 or the fp64 flavour of a tolerance; other dtypes are an error."""
    try:
        return {torch.float32: single, torch.float64: double}[dtype]
    except KeyError:
        raise TypeError(f"Data-type {str(dtype)} invalid") from None


@dataclass
class BaseOptions:
    debug: bool = False                               # carried, unused
    use_cpu: bool = False                             # True is refused: there is no CPU compute path
    max_gpu_mem: float = np.inf                       # cap on the device memory one call may use
    max_cpu_mem: float = np.inf                       # carried (read by the CPU oracle in the tests only)
    compute_arch_speed: bool = False                  # carried, unused
    no_single_kernel: bool = True                     # kernel matrices of fp32 data are evaluated in fp64
    min_cuda_pc_size_32: int = 10000                  # carried, unused (everything runs on the GPU)
    min_cuda_pc_size_64: int = 30000                  # carried, unused
    min_cuda_iter_size_32: int = 10_000 * 10 * 3_000  # carried, unused
    min_cuda_iter_size_64: int = 30_000 * 10 * 3_000  # carried, unused
    never_store_kernel: bool = False                  # True: never store K (overrides the two *_stored_blocks options
                                                      # and the stored K(X, centres) of a fit)
    store_kernel_d_threshold: int = 1200              # beyond this many features a fit keeps K(X, centres) if it fits
    num_fmm_streams: int = 2                          # carried, unused
    memory_slack: float = 0.9                         # fraction of the free device memory a call may plan with
    bf16x3_cross_term: bool = False                   # not in the reference: fp32 products form x.c on the bf16 matrix
                                                      # cores from an exact 3-way bfloat16 split (fp32 accuracy)
    many_rhs_stored_blocks: bool = False              # not in the reference's options: with many right-hand sides
                                                      # (several passes of the product kernels) store blocks of K and
                                                      # contract them with rocBLAS; off: every product is matrix-free
    dmmv_stored_blocks: bool = False                  # not in the reference's options: K^T(K v + w) beyond 64 features
                                                      # evaluates K once, into stored blocks, whatever T (see fmmv.py)


@dataclass
class KeopsOptions:                                   # KeOps is not part of this build; fields carried for compatibility
    keops_acc_dtype: str = "auto"
    keops_sum_scheme: str = "auto"
    keops_active: str = "auto"
    keops_memory_slack: float = 0.7


@dataclass
class ConjugateGradientOptions:
    cg_epsilon_32: float = 1e-7                       # guards the divisions of the CG in fp32
    cg_epsilon_64: float = 1e-15                      # ... in fp64
    cg_tolerance: float = 1e-7                        # stop once every column has |r| below this
    cg_full_gradient_every: int = 10                  # recompute the residual from scratch this often
    cg_differential_convergence: bool = False         # a converged column is frozen while the others go on
    cg_capture_graph: bool = False                    # not in the reference: GPU solves capture each kind of iteration
                                                      # (operator + update) into a HIP graph once and replay it
    cg_pack_once: bool = True                         # not in the reference: a GPU fit packs X and the centres once for
                                                      # the whole solve instead of once per product (same results)

    def cg_epsilon(self, dtype):
        return _by_precision(dtype, self.cg_epsilon_32, self.cg_epsilon_64)


@dataclass
class PreconditionerOptions:
    pc_epsilon_32: float = 1e-5                       # jitter (times M) on the diagonal of K(C,C) in fp32
    pc_epsilon_64: float = 1e-13                      # ... in fp64
    cpu_preconditioner: bool = False                  # carried, unused
    # False: the diagonal blocks of the two Cholesky factorisations go to the library routine (torch.linalg.cholesky)
    # instead of this library's tile kernel (flk_potrf_tile); everything else stays as it is
    pc_tile_factorisation: bool = True

    def pc_epsilon(self, dtype):
        return _by_precision(dtype, self.pc_epsilon_32, self.pc_epsilon_64)


@dataclass
class CholeskyOptions:                                # the reference's out-of-core Cholesky is not part of this build
    chol_force_in_core: bool = False
    chol_force_ooc: bool = False
    chol_par_blk_multiplier: int = 2


@dataclass
class FalkonOptions(BaseOptions, ConjugateGradientOptions, PreconditionerOptions, CholeskyOptions, KeopsOptions):
    """Global options, same fields as falkon/options.py:293-303."""
