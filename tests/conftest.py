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
