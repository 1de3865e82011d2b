"""Seeded synthetic inputs: the reference's test fixtures and the five benchmark configurations.

Test infrastructure only.  Everything is generated on the host with numpy's
``default_rng`` so the same arrays can be rebuilt anywhere from the seed.
"""
import dataclasses
from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch


def gen_random(a: int, b: int, dtype, F: bool = False, seed: int = 0) -> np.ndarray:
    """uniform[0,1) matrix, as falkon/tests/gen_random.py:17-22."""
    out = np.random.default_rng(seed).random(size=(a, b), dtype=dtype)
    return np.asfortranarray(out) if F else out


def reference_test_mats(n: int, m: int, d: int, t: int, dtype, order: str = "C"):
    """A, B, v, w with the seeds the reference's kernel tests use.

    falkon/tests/test_kernels.py:55-71 (seeds 92, 93, 94, 95; drawn in float32,
    then cast) and falkon/tests/conftest.py:78-105 (``fix_mat``: cast + order).
    """
    mats = [gen_random(n, d, "float32", seed=92), gen_random(m, d, "float32", seed=93),
            gen_random(m, t, "float32", seed=94), gen_random(n, t, "float32", seed=95)]
    return tuple(torch.from_numpy(np.asarray(a, dtype=dtype, order=order)) for a in mats)


@dataclass
class Config:
    name: str
    seed: int
    N: int
    d: int
    M: int
    T: int
    dtype: torch.dtype
    op: str            # "fmmv" | "fdmmv"
    has_w: bool


CONFIGS = {
    "C1": Config("C1", 1001, 20_000, 8, 1_000, 1, torch.float64, "fmmv", False),
    "C2": Config("C2", 1002, 1_000_000, 28, 20_000, 1, torch.float32, "fdmmv", True),
    "C3": Config("C3", 1003, 10_000_000, 9, 50_000, 1, torch.float32, "fdmmv", False),
    "C4": Config("C4", 1004, 500_000, 784, 10_000, 10, torch.float32, "fdmmv", True),
}


def make_config(name: str, N: Optional[int] = None, M: Optional[int] = None, dtype: Optional[torch.dtype] = None,
                d: Optional[int] = None, T: Optional[int] = None):
    """Build (X, C, sigma, v, w) for a configuration, optionally at reduced N / M.

    Draw order X, idx, sigma, v, w from ``default_rng(seed)``; ``C = X[idx]`` with
    ``idx = rng.choice(N, M, replace=False)`` as falkon/center_selection.py:227-239.
    A reduced N draws a smaller X from the same generator (not a prefix of the
    full-size X); reduced-size runs are self-consistent, not slices of the full run.
    ``d`` / ``T`` give the configuration's shape another feature count / number of right-hand sides.
    """
    cfg = CONFIGS[name]
    if d is not None or T is not None:
        cfg = dataclasses.replace(cfg, d=cfg.d if d is None else d, T=cfg.T if T is None else T)
    N = cfg.N if N is None else N
    M = cfg.M if M is None else M
    dtype = cfg.dtype if dtype is None else dtype
    rng = np.random.default_rng(cfg.seed)
    np_dt = np.float32 if dtype == torch.float32 else np.float64
    if name in ("C1", "C2"):
        X = rng.standard_normal((N, cfg.d), dtype=np.float32 if name == "C2" else np.float64)
    elif name == "C3":
        X = rng.random((N, cfg.d), dtype=np.float32) * 2.0 - 1.0
    else:  # C4: uniform[0,1) with 80 % of the entries zeroed, stored dense
        X = rng.random((N, cfg.d), dtype=np.float32)
        X *= rng.random((N, cfg.d), dtype=np.float32) < 0.2
    idx = rng.choice(N, size=M, replace=False)
    if name == "C1":
        sigma = torch.tensor([2.0], dtype=torch.float64)
    elif name == "C2":
        sigma = torch.tensor([3.8], dtype=torch.float64)
    elif name == "C3":
        sigma = torch.from_numpy(rng.uniform(0.5, 2.0, cfg.d))
    else:
        sigma = torch.tensor([10.0], dtype=torch.float64)
    v = rng.standard_normal((M, cfg.T))
    w = rng.standard_normal((N, cfg.T)) if cfg.has_w else None
    X = np.ascontiguousarray(X, dtype=np_dt)
    Xt = torch.from_numpy(X)
    Ct = torch.from_numpy(np.ascontiguousarray(X[np.sort(idx)] if False else X[idx]))
    vt = torch.from_numpy(v.astype(np_dt))
    wt = torch.from_numpy(w.astype(np_dt)) if w is not None else None
    return Xt, Ct, sigma, vt, wt
