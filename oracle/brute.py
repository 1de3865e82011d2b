"""Closed-form Gaussian kernel in fp64 difference form (no expanded norm).

Test infrastructure only.  K_ij = exp(-1/2 * sum_k ((x_ik - c_jk) / sigma_k)^2),
the definition the reference documents (falkon/kernels/distance_kernel.py:366-370)
and that its own tests use as the naive oracle (falkon/tests/naive_kernels.py:23-25).
"""
import numpy as np
import torch


def _sigma_vec(sigma, d: int) -> np.ndarray:
    s = np.asarray(sigma.detach().cpu().numpy() if isinstance(sigma, torch.Tensor) else sigma, dtype=np.float64).reshape(-1)
    if s.size == 1:
        s = np.full(d, s[0])
    if s.size != d:
        raise RuntimeError(f"sigma has {s.size} entries, data has {d} columns")
    return s


def gaussian_brute(X, C, sigma) -> np.ndarray:
    """K[n,m] in float64, whatever the input dtype (inputs are widened exactly)."""
    X = np.asarray(X.detach().cpu().numpy() if isinstance(X, torch.Tensor) else X, dtype=np.float64)
    C = np.asarray(C.detach().cpu().numpy() if isinstance(C, torch.Tensor) else C, dtype=np.float64)
    s = _sigma_vec(sigma, X.shape[1])
    Xs, Cs = X / s, C / s
    K = np.empty((X.shape[0], C.shape[0]), dtype=np.float64)
    step = max(1, int(2**24 // max(1, C.shape[0] * X.shape[1])))
    for i in range(0, X.shape[0], step):
        diff = Xs[i:i + step, None, :] - Cs[None, :, :]
        K[i:i + step] = np.exp(-0.5 * np.einsum("nmd,nmd->nm", diff, diff))
    return K


def mmv_brute(X, C, sigma, v) -> np.ndarray:
    v = np.asarray(v.detach().cpu().numpy() if isinstance(v, torch.Tensor) else v, dtype=np.float64)
    return gaussian_brute(X, C, sigma) @ v.reshape(C.shape[0], -1)


def dmmv_brute(X, C, sigma, v, w) -> np.ndarray:
    """K.T @ (K @ v + w); v or w may be None (falkon/kernels/kernel.py:352-356)."""
    K = gaussian_brute(X, C, sigma)
    n, m = K.shape
    u = 0.0
    if v is not None:
        v = np.asarray(v.detach().cpu().numpy() if isinstance(v, torch.Tensor) else v, dtype=np.float64)
        u = K @ v.reshape(m, -1)
    if w is not None:
        w = np.asarray(w.detach().cpu().numpy() if isinstance(w, torch.Tensor) else w, dtype=np.float64)
        u = u + w.reshape(n, -1)
    return K.T @ u
