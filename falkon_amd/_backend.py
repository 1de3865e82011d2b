"""Loader and ctypes signatures of ``libfalkon_amd.so``.

Plays the role of falkon/c_ext/_backend.py:79-185 for this build: use the
prebuilt in-tree library if it is there, otherwise build it with ``hipcc``.
There is no pure-Python or CPU substitute: if the library cannot be loaded every
product call raises.
"""
import ctypes
import os
import threading
from ctypes import c_char_p, c_int, c_int64, c_size_t, c_void_p

from . import _build

_lock = threading.Lock()
_lib = None

FLK_F32, FLK_F64, FLK_F32_BF16X3 = 0, 1, 2
FLK_GAUSSIAN, FLK_LAPLACIAN, FLK_MATERN32, FLK_MATERN52, FLK_LAPLACIAN_DU = 0, 1, 2, 3, 4
FLK_EINVAL, FLK_ENOMEM, FLK_EUNSUPPORTED, FLK_EHIP = -1, -2, -3, -4

_MAT = [c_void_p, c_int64, c_int64, c_int64]        # ptr, rows, row_stride, col_stride
_SIGNATURES = {
    "flk_version": (c_int, []),
    "flk_last_error": (c_char_p, []),
    "flk_max_d": (c_int64, [c_int]),
    "flk_max_t": (c_int64, []),
    "flk_kernel_timing_enable": (c_int, [c_int]),
    "flk_kernel_timing_read": (c_int, [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(c_int64)]),
    "flk_gauss_packed_bytes": (c_size_t, [c_int64, c_int64, c_int]),
    "flk_gauss_pack": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64, c_int, c_void_p,
                               c_size_t, c_void_p]),
    "flk_gauss_mmv_packed_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64, c_int]),
    "flk_gauss_mmv_packed": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64,
                                     c_void_p, c_int64, c_int64, c_int64,
                                     c_void_p, c_int64, c_int64,
                                     c_void_p, c_int64, c_int64, c_int,
                                     c_void_p, c_size_t, c_void_p]),
    "flk_gauss_fmmv_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64, c_int]),
    "flk_gauss_fmmv": (c_int, [*_MAT, *_MAT, c_int64, c_void_p, c_int64,
                               c_void_p, c_int64, c_int64, c_int64,
                               c_void_p, c_int64, c_int64, c_int,
                               c_void_p, c_size_t, c_void_p]),
    "flk_gauss_fdmmv_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64, c_int]),
    "flk_gauss_fdmmv": (c_int, [*_MAT, *_MAT, c_int64, c_void_p, c_int64,
                                c_void_p, c_int64, c_int64,
                                c_void_p, c_int64, c_int64, c_int64,
                                c_void_p, c_int64, c_int64, c_int,
                                c_void_p, c_size_t, c_void_p]),
    "flk_gauss_fmm_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int, c_int]),
    "flk_gauss_fmm": (c_int, [*_MAT, *_MAT, c_int64, c_void_p, c_int64,
                              c_void_p, c_int64, c_int64, c_int, c_int,
                              c_void_p, c_size_t, c_void_p]),
}
# (added below the loop that derives the flk_kernel_* signatures: this one has no flk_kernel_* twin)
_NOALLOC = {"flk_gauss_fdmmv_noalloc": (c_int, [*_MAT, *_MAT, c_int64, c_void_p, c_int64,
                                               c_void_p, c_int64, c_int64,
                                               c_void_p, c_int64, c_int64, c_int64,
                                               c_void_p, c_int64, c_int64, c_int, c_void_p])}
# the flk_kernel_* entry points: the flk_gauss_* ones with the kernel function as first argument
for _name in ("pack", "mmv_packed", "fmmv", "fdmmv", "fmm"):
    _res, _args = _SIGNATURES["flk_gauss_" + _name]
    _SIGNATURES["flk_kernel_" + _name] = (_res, [c_int, *_args])
_SIGNATURES.update(_NOALLOC)
_SIGNATURES["flk_cg_state_ints"] = (c_int64, [c_int64])
_SIGNATURES["flk_cg_update"] = (c_int, [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                        c_int64, c_int64, c_void_p, c_void_p, c_int64, ctypes.c_double, ctypes.c_double,
                                        c_int, c_int, c_void_p])
_SIGNATURES["flk_tri_solve_work_elems"] = (c_int64, [c_int64, c_int64, c_int64])
_SIGNATURES["flk_tri_solve"] = (c_int, [c_int, c_int, c_void_p, c_int64, c_int64, c_int, c_void_p, c_void_p, c_int64,
                                        c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_void_p])
_SIGNATURES["flk_potrf_tile_rows"] = (c_int64, [c_int])
_SIGNATURES["flk_potrf_tile"] = (c_int, [c_int, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p])
NOALLOC_SCRATCH_BYTES = 64 << 20


def library_path() -> str:
    return _build.LIB_PATH


def load():
    """Return the loaded library, building it first only if no built library exists."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            path = library_path()
            if not os.path.exists(path):
                _build.build(verbose=False)
            lib = ctypes.CDLL(path)
            for name, (res, args) in _SIGNATURES.items():
                fn = getattr(lib, name)   # AttributeError if the library lacks a declared symbol
                fn.restype, fn.argtypes = res, args
            _lib = lib
    return _lib


def last_error() -> str:
    msg = load().flk_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def raise_for_status(code: int, what: str) -> None:
    """Turn a native status into the exception type the reference raises for that condition."""
    if code == 0:
        return
    msg = f"{what}: {last_error()}"
    if code == FLK_ENOMEM:
        raise MemoryError(msg)
    if code == FLK_EUNSUPPORTED:
        raise NotImplementedError(msg)
    # bad arguments that got past the Python checks and HIP failures surface as RuntimeError,
    # like TORCH_CHECK failures of the reference's native ops (falkon/c_ext/ops/helpers.h:9-10)
    raise RuntimeError(msg)
