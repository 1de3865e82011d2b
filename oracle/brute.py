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


def radial_brute(X, C, sigma, kernel_name: str) -> np.ndarray:
    """K[n,m] in float64 from the distances in difference form, for the closed forms the reference documents:
    "gaussian" exp(-D^2/2); "laplacian" exp(-D) (falkon/kernels/distance_kernel.py:449-453); "1.5-matern"
    (1 + sqrt(3) D) exp(-sqrt(3) D) and "2.5-matern" (1 + sqrt(5) D + 5/3 D^2) exp(-sqrt(5) D) (:243-267;
    the naive oracles of the reference's tests, falkon/tests/naive_kernels.py:28-31,48-61)."""
    X = np.asarray(X.detach().cpu().numpy() if isinstance(X, torch.Tensor) else X, dtype=np.float64)
    C = np.asarray(C.detach().cpu().numpy() if isinstance(C, torch.Tensor) else C, dtype=np.float64)
    s = _sigma_vec(sigma, X.shape[1])
    Xs, Cs = X / s, C / s
    D2 = np.empty((X.shape[0], C.shape[0]), dtype=np.float64)
    step = max(1, int(2**24 // max(1, C.shape[0] * X.shape[1])))
    for i in range(0, X.shape[0], step):
        diff = Xs[i:i + step, None, :] - Cs[None, :, :]
        D2[i:i + step] = np.einsum("nmd,nmd->nm", diff, diff)
    D = np.sqrt(D2)
    if kernel_name in ("gaussian", "inf-matern"):
        return np.exp(-0.5 * D2)
    if kernel_name in ("laplacian", "0.5-matern"):
        return np.exp(-D)
    if kernel_name == "1.5-matern":
        return (1 + np.sqrt(3) * D) * np.exp(-np.sqrt(3) * D)
    if kernel_name == "2.5-matern":
        return (1 + np.sqrt(5) * D + 5.0 / 3.0 * D2) * np.exp(-np.sqrt(5) * D)
    raise ValueError(kernel_name)


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
