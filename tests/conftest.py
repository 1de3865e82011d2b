import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (MI355X); run with -m gpu")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def dev():
    return torch.device("cuda:0")


def rel_err(actual, expected) -> float:
    """Norm-wise relative error per output column, worst column."""
    a = torch.as_tensor(actual).detach().double().cpu()
    e = torch.as_tensor(expected).detach().double().cpu()
    a, e = a.reshape(e.shape[0], -1), e.reshape(e.shape[0], -1)
    num = (a - e).norm(dim=0)
    den = e.norm(dim=0).clamp_min(1e-300)
    return float((num / den).max())


def check_parity(got, ref_same_dtype, ref_f64, tol: float) -> None:
    """Parity of a GPU result with the reference-equivalent CPU path.

    ``ref_same_dtype`` is the CPU oracle run in the data's dtype, ``ref_f64`` the same path run in
    fp64 on the same (exactly widened) inputs, both computed on the CPU.  The GPU result must be within
    ``tol`` of the CPU result in its own dtype.  Where the CPU fp32 path itself is further than tol/2
    from its fp64 twin (ill-conditioned sums: long fp32 accumulations, output columns that nearly
    cancel) two fp32 results cannot be expected to agree to ``tol``; this is a relaxation of the
    literal bar and it is bounded: the GPU result must then be at least as close to the fp64 CPU path
    as the CPU fp32 path is (factor 2 of slack), and never further than ``10 * tol`` from it, however
    far the CPU fp32 path has drifted.
    """
    e_ref = rel_err(ref_same_dtype, ref_f64)
    if e_ref < tol / 2:
        e = rel_err(got, ref_same_dtype)
        assert e < tol, f"GPU vs CPU oracle: {e:.3e} >= {tol:.1e} (CPU fp32 vs fp64: {e_ref:.3e})"
    else:
        e = rel_err(got, ref_f64)
        bound = min(max(tol, 2 * e_ref), 10 * tol)
        assert e < bound, f"GPU vs fp64 oracle: {e:.3e} >= {bound:.1e}; CPU fp32 path vs fp64: {e_ref:.3e}"


def scaled_err(got, ref_f64, scale) -> float:
    """Worst column of ``|got - ref| / |scale|`` (norm-wise), where ``scale`` is the same product formed
    from the absolute values of its terms: the error measured against the size of what was summed rather
    than against a result that may have cancelled.  A backward-stable fp32 summation stays at a small
    multiple of 6e-8 here however strongly a column cancels; an accumulation that loses digits does not."""
    a = torch.as_tensor(got).detach().double().cpu()
    e = torch.as_tensor(ref_f64).detach().double().cpu()
    s = torch.as_tensor(scale).detach().double().cpu()
    a, e, s = a.reshape(e.shape[0], -1), e.reshape(e.shape[0], -1), s.reshape(e.shape[0], -1)
    return float(((a - e).norm(dim=0) / s.norm(dim=0).clamp_min(1e-300)).max())
