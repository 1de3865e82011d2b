"""ctypes binding of ``brute.c`` (test infrastructure only)."""
import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force: bool = False) -> str:
    path = os.path.join(_HERE, "libbrute.so")
    if force or not os.path.exists(path):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libbrute.so"])
    return path


def _lib():
    global _LIB
    if _LIB is None:
        _LIB = ctypes.CDLL(build())
        dp, lg = ctypes.POINTER(ctypes.c_double), ctypes.c_long
        _LIB.brute_mmv.argtypes = [dp, lg, dp, lg, lg, dp, lg, dp, lg, dp]
        _LIB.brute_dmmv.argtypes = [dp, lg, dp, lg, lg, dp, lg, dp, dp, lg, dp]
    return _LIB


def _arr(a):
    if a is None:
        return None
    if isinstance(a, torch.Tensor):
        a = a.detach().cpu().numpy()
    return np.ascontiguousarray(a, dtype=np.float64)


def _p(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double)) if a is not None else None


def mmv_brute_c(X, C, sigma, v) -> np.ndarray:
    X, C, s = _arr(X), _arr(C), _arr(sigma).reshape(-1)
    v = _arr(v).reshape(C.shape[0], -1)
    out = np.empty((X.shape[0], v.shape[1]))
    rc = _lib().brute_mmv(_p(X), X.shape[0], _p(C), C.shape[0], X.shape[1], _p(s), s.size, _p(v), v.shape[1], _p(out))
    if rc != 0:
        raise RuntimeError(f"brute_mmv failed with code {rc}")
    return out


def dmmv_brute_c(X, C, sigma, v, w) -> np.ndarray:
    X, C, s = _arr(X), _arr(C), _arr(sigma).reshape(-1)
    v = _arr(v).reshape(C.shape[0], -1) if v is not None else None
    w = _arr(w).reshape(X.shape[0], -1) if w is not None else None
    t = v.shape[1] if v is not None else w.shape[1]
    out = np.empty((C.shape[0], t))
    rc = _lib().brute_dmmv(_p(X), X.shape[0], _p(C), C.shape[0], X.shape[1], _p(s), s.size, _p(v), _p(w), t, _p(out))
    if rc != 0:
        raise RuntimeError(f"brute_dmmv failed with code {rc}")
    return out
