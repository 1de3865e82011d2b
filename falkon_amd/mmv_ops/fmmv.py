"""Kernel-vector products of the radial kernels (Gaussian, Laplacian, Matern) on the MI355X: ``fmmv`` and ``fdmmv``.

Drop-in for the two callables the reference's kernels dispatch to
(falkon/mmv_ops/fmmv.py:960-973 ``fmmv`` and :976-1131 ``fdmmv``): same
signatures, same validation, same ``out`` semantics, same exception types.
The work itself is done by ``libfalkon_amd.so`` through its C ABI; the kernel
matrix is never materialised, so the reference's memory-driven blocking over
rows and columns (fmmv.py:60-114,488-544) reduces to "keep the whole problem
resident; split the rows of X1 only if the packed operands do not fit".
There is no CPU computation in this module.
"""
import math
import contextlib
from typing import Dict, Optional, Tuple

import torch

from .. import _backend
from ..options import BaseOptions
from ..utils.helpers import sizeof_dtype
from .utils import check_contiguity, create_output_mat, retry_with_fresh_memory_report, usable_gpu_memory

__all__ = ("fmmv", "fdmmv", "gauss_fmmv_native", "gauss_fdmmv_native", "PackedProducts")

_DTYPE_CODE = {torch.float32: _backend.FLK_F32, torch.float64: _backend.FLK_F64}


def _mat(t: torch.Tensor) -> Tuple[int, int, int, int]:
    """(ptr, rows, row_stride, col_stride) of a 2-D tensor, strides in elements."""
    return t.data_ptr(), t.shape[0], t.stride(0), t.stride(1)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_handle(dev: torch.device) -> int:
    """The HIP stream torch currently works on, as an integer handle."""
    if _raw_stream is not None and dev.index is not None:
        return _raw_stream(dev.index)                      # the same handle without building a Stream object
    return torch.cuda.current_stream(dev).cuda_stream


def _current(dev: torch.device):
    """Context that makes ``dev`` the current GPU; nothing to enter or leave when it already is (a small call's
    host time is a few tens of microseconds, and torch's device guard object costs several of them)."""
    if dev.index is None or torch.cuda.current_device() == dev.index:
        return contextlib.nullcontext()
    return torch.cuda.device(dev)


def _arith_code(dtype: torch.dtype, opt: Optional[BaseOptions]) -> int:
    """The library's dtype code: the data's dtype, or the bf16x3 mode of fp32 when the options ask for it."""
    if dtype == torch.float32 and opt is not None and getattr(opt, "bf16x3_cross_term", False):
        return _backend.FLK_F32_BF16X3
    return _DTYPE_CODE[dtype]


def gauss_fmmv_native(X1, X2, sigma_dev, v, out, kernel_fn: int = _backend.FLK_GAUSSIAN,
                      code: Optional[int] = None) -> None:
    """out[n,t] = K(X1,X2) @ v through ``flk_kernel_fmmv``.  All tensors on one GPU, 2-D, same dtype."""
    lib = _backend.load()
    code = _DTYPE_CODE[X1.dtype] if code is None else code
    n, d = X1.shape
    m, t = v.shape
    ws_bytes = lib.flk_gauss_fmmv_workspace_bytes(n, m, d, t, code)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=X1.device)
    p1, _, r1, c1 = _mat(X1)
    p2, _, r2, c2 = _mat(X2)
    pv, _, rv, cv = _mat(v)
    po, _, ro, co = _mat(out)
    with _current(X1.device):
        rc = lib.flk_kernel_fmmv(kernel_fn, p1, n, r1, c1, p2, m, r2, c2, d, sigma_dev.data_ptr(), sigma_dev.numel(),
                                 pv, rv, cv, t, po, ro, co, code, ws.data_ptr(), ws_bytes, _stream_handle(X1.device))
    _backend.raise_for_status(rc, "flk_kernel_fmmv")


def gauss_fdmmv_native(X1, X2, sigma_dev, v, w, out, kernel_fn: int = _backend.FLK_GAUSSIAN,
                       code: Optional[int] = None) -> None:
    """out[m,t] = K^T (K v + w) through ``flk_kernel_fdmmv``.  ``w`` may be None."""
    lib = _backend.load()
    code = _DTYPE_CODE[X1.dtype] if code is None else code
    n, d = X1.shape
    m, t = v.shape
    ws_bytes = lib.flk_gauss_fdmmv_workspace_bytes(n, m, d, t, code)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=X1.device)
    p1, _, r1, c1 = _mat(X1)
    p2, _, r2, c2 = _mat(X2)
    pv, _, rv, cv = _mat(v)
    pw, rw, cw = (w.data_ptr(), w.stride(0), w.stride(1)) if w is not None else (None, 0, 0)
    po, _, ro, co = _mat(out)
    with _current(X1.device):
        rc = lib.flk_kernel_fdmmv(kernel_fn, p1, n, r1, c1, p2, m, r2, c2, d, sigma_dev.data_ptr(), sigma_dev.numel(),
                                  pv, rv, cv, pw, rw, cw, t, po, ro, co, code, ws.data_ptr(), ws_bytes,
                                  _stream_handle(X1.device))
    _backend.raise_for_status(rc, "flk_kernel_fdmmv")


# ---------------------------------------------------------------------------
# host-side planning
# ---------------------------------------------------------------------------
_KERNEL_FN = {"gaussian": _backend.FLK_GAUSSIAN, "inf-matern": _backend.FLK_GAUSSIAN,
              "laplacian": _backend.FLK_LAPLACIAN, "0.5-matern": _backend.FLK_LAPLACIAN,
              "1.5-matern": _backend.FLK_MATERN32, "2.5-matern": _backend.FLK_MATERN52}


def _kernel_fn(kernel) -> int:
    """The library's code for the kernel object's function (by ``kernel_name``, as the reference names its
    distance kernels, falkon/kernels/distance_kernel.py:382,456,544); other kernels have no MI355X path."""
    code = _KERNEL_FN.get(getattr(kernel, "kernel_name", None))
    if code is None or not hasattr(kernel, "sigma"):
        raise NotImplementedError(
            "falkon_amd covers the Gaussian, Laplacian and Matern kernels; "
            f"kernel '{getattr(kernel, 'name', type(kernel).__name__)}' has no MI355X kernel-vector path")
    return code


def _reject_block_kwargs(kwargs_m1, kwargs_m2):
    if kwargs_m1 or kwargs_m2:
        # the reference forwards these to the kernel's core function, and the Gaussian core takes none
        # (falkon/kernels/diff_kernel.py:90-91, distance_kernel.py:140-142)
        raise TypeError("The Gaussian kernel takes no per-block keyword tensors (kwargs_m1 / kwargs_m2)")


_gpu_seen = False


def _gpu_present() -> bool:
    global _gpu_seen
    if not _gpu_seen:
        _gpu_seen = torch.cuda.is_available()          # asked again on every call only while the answer is no
    return _gpu_seen


def _compute_device(opt: BaseOptions, data_devs) -> torch.device:
    """The GPU to compute on; mirrors the reference's device choice (fmmv.py:906,1038) minus its CPU branch."""
    if opt.use_cpu:
        raise RuntimeError("falkon_amd has no CPU compute path: `use_cpu=True` cannot be honoured "
                           "(the MI355X kernels are the only implementation)")
    if not _gpu_present():
        raise RuntimeError("falkon_amd needs a ROCm GPU (MI355X); torch.cuda.is_available() is False")
    cuda_devs = {d for d in data_devs if d.type == "cuda"}
    if len(cuda_devs) > 1:
        raise RuntimeError("All GPU-resident inputs must be on the same device")
    if cuda_devs:
        return next(iter(cuda_devs))
    return torch.device("cuda", torch.cuda.current_device())


def _rows_that_fit(n: int, bytes_for_rows, usable: float) -> int:
    """Largest row count r <= n with bytes_for_rows(r) <= usable (bytes_for_rows is non-decreasing)."""
    if bytes_for_rows(n) <= usable:
        return n
    lo, hi = 0, n
    while hi - lo > 1:
        mid = (lo + hi) // 2
        if bytes_for_rows(mid) <= usable:
            lo = mid
        else:
            hi = mid
    if lo < 1:
        raise MemoryError("Available memory %.2fMB is not enough." % (usable / 2**20))
    return lo


# ---------------------------------------------------------------------------
# host-resident rows: upload overlapped with compute
# ---------------------------------------------------------------------------
_STREAM_MIN_BYTES = 32 << 20      # smaller host operands are uploaded in one piece
_STREAM_PIECES = 4                # pieces a host operand that fits is cut into


class _HostRowStream:
    """Row chunks of host tensors on their way to the GPU, two chunks in flight.

    The reference's CPU-data / GPU-compute mode copies a row block, computes on it, copies the next
    (falkon/mmv_ops/fmmv.py:730-767).  Here the copies run on a stream of their own (default priority):
    while the kernels of chunk k run, chunk k+1 crosses PCIe and the host stages chunk k+2 into pinned
    memory (pageable sources only; pinned sources are copied from where they are).  Each slot's device
    buffer is reused only after the kernels that read it have finished (event recorded by the consumer),
    each pinned buffer only after its upload has finished.
    """

    def __init__(self, tensors, n_rows: int, dev: torch.device, chunk_rows: int):
        self.tensors, self.n_rows, self.dev, self.chunk = list(tensors), n_rows, dev, chunk_rows
        self.copy_stream = torch.cuda.Stream(dev)
        on_host = [t is not None and t.device.type == "cpu" for t in self.tensors]
        self.dev_bufs = [[self._like(t, dev, False) if h else None for t, h in zip(self.tensors, on_host)]
                         for _ in range(2)]
        self.pin_bufs = [[self._like(t, None, True) if h and not t.is_pinned() else None
                          for t, h in zip(self.tensors, on_host)] for _ in range(2)]
        self.uploaded = [None, None]
        self.consumed = [None, None]

    def _like(self, t: torch.Tensor, dev, pinned: bool) -> torch.Tensor:
        """A chunk-sized buffer in the memory order of ``t`` (rows of an F-ordered matrix stay F-ordered)."""
        shape = (self.chunk, t.shape[1])
        f_order = t.shape[1] > 1 and t.stride(0) == 1
        strides = (1, self.chunk) if f_order else (t.shape[1], 1)
        if pinned:
            return torch.empty_strided(shape, strides, dtype=t.dtype, pin_memory=True)
        return torch.empty_strided(shape, strides, dtype=t.dtype, device=dev)

    def _issue(self, k: int):
        slot, i = k & 1, k * self.chunk
        li = min(self.chunk, self.n_rows - i)
        if self.uploaded[slot] is not None:
            self.uploaded[slot].synchronize()                 # the pinned buffer of this slot is free again
        chunk = []
        with torch.cuda.stream(self.copy_stream):
            if self.consumed[slot] is not None:
                self.copy_stream.wait_event(self.consumed[slot])   # the device buffer of this slot is free again
            for t, dbuf, pbuf in zip(self.tensors, self.dev_bufs[slot], self.pin_bufs[slot]):
                if t is None or dbuf is None:                 # absent, or already on the GPU: just the rows
                    chunk.append(None if t is None else t[i:i + li])
                    continue
                src = t[i:i + li]
                if pbuf is not None:
                    pbuf[:li].copy_(src)
                    src = pbuf[:li]
                dbuf[:li].copy_(src, non_blocking=True)
                chunk.append(dbuf[:li])
            done = torch.cuda.Event()
            done.record(self.copy_stream)
        self.uploaded[slot] = done
        return i, li, chunk, done

    def __iter__(self):
        """Yields (first row, rows, [device views]); the consumer enqueues its kernels on the current stream
        before asking for the next chunk, whose staging and upload then overlap those kernels."""
        n_chunks = (self.n_rows + self.chunk - 1) // self.chunk
        compute = torch.cuda.current_stream(self.dev)
        ahead = self._issue(0) if n_chunks else None
        for k in range(n_chunks):
            i, li, chunk, done = ahead
            compute.wait_event(done)
            yield i, li, chunk
            used = torch.cuda.Event()
            used.record(compute)
            self.consumed[k & 1] = used
            ahead = self._issue(k + 1) if k + 1 < n_chunks else None


def _streamed_chunk_rows(n: int, row_bytes: int, rows_that_fit: int) -> int:
    """Rows per chunk for a host operand of n rows: what fits, and no more than a quarter of the operand
    (so that upload and compute overlap) once the operand is big enough for that to matter."""
    if n * row_bytes < _STREAM_MIN_BYTES:
        return rows_that_fit
    piece = -(-n // _STREAM_PIECES)
    piece = -(-piece // 1024) * 1024
    return max(1, min(rows_that_fit, piece))


def _on(t: Optional[torch.Tensor], dev: torch.device) -> Optional[torch.Tensor]:
    if t is None or t.device == dev:
        return t
    return t.to(dev, non_blocking=True)


def _check_dtype(dtype):
    if dtype not in _DTYPE_CODE:
        raise TypeError(f"Dtype {dtype} not valid")


class _KernelMmvFn(torch.autograd.Function):
    """``K(X1, X2) @ v`` with its backward pass (the reference's KernelMmvFnFull, falkon/mmv_ops/fmmv.py:771-957).
    The forward is the plain product; the backward is closed form on the same kernels (``fmmv_grad``)."""

    @staticmethod
    def forward(ctx, kernel, opt, out, X1, X2, v, *kernel_params):
        kernel_fn = _kernel_fn(kernel)
        res = _fmmv_run(X1, X2, v, kernel, kernel_fn, out, opt, cached_sigma=False)
        if out is not None:
            ctx.mark_dirty(out)
        ctx.save_for_backward(X1, X2, v, *kernel_params)
        ctx.kernel_fn, ctx.opt = kernel_fn, opt
        return res

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_out):
        from .fmmv_grad import fmmv_backward
        X1, X2, v, sigma = ctx.saved_tensors
        grads = fmmv_backward(ctx.kernel_fn, X1, X2, v, sigma, grad_out, ctx.needs_input_grad[3:7], ctx.opt)
        like = (X1, X2, v, sigma)
        grads = [None if g is None else g.reshape(t.shape).to(device=t.device, dtype=t.dtype)
                 for g, t in zip(grads, like)]
        return (None, None, None, *grads)


# ---------------------------------------------------------------------------
# many right-hand sides: kernel blocks stored once, contracted by library GEMMs
# ---------------------------------------------------------------------------
# The product kernels never store K and pay for it by evaluating K once per pass of 16 to 64 right-hand sides.  That
# is the default for any number of right-hand sides.  ``FalkonOptions(many_rhs_stored_blocks=True)`` opts into the
# other trade where it is the faster one: a stored kernel value costs 4 (8) bytes written and a read per product, so
# beyond a break-even the drivers then do what the reference does on every call
# (falkon/mmv_ops/fmmv.py:358-396,740-762): evaluate a block of rows of K with the kernel-matrix kernel and contract it
# with rocBLAS (``K_b @ v``, ``K_b.T @ u``), block by block, K blocks as large as the memory budget allows, and K
# evaluated once for both products of ``fdmmv``.  ``FalkonOptions.never_store_kernel`` overrides the option.
# Break-even in passes of the product kernels, measured on one MI355X (N = 2.5e5 .. 1e6, M = 1e4 .. 2e4):
#   d = 784: T = 17 (2 passes) fp32 mmv 61.9 -> 32.6 ms, dmmv 122 -> 35 ms; T = 256: 986 -> 49 ms; fp64 2097 -> 114 ms;
#   d = 100: T = 17 fp32 mmv 40.9 -> 29.1, dmmv 81 -> 36; T = 256: 741 -> 94;
#   d = 28 fp32: T = 65 (3 passes) mmv 53.5 against 58.6 stored, T = 128 (4 passes) 86.9 -> 61.9, dmmv 172 -> 99;
#   d = 9 fp32: T = 128 mmv 58.6 against 56.5, dmmv 116 -> 95; T = 65 dmmv 67 against 95 stored;
#   d = 28 fp64: T = 64 (4 passes) mmv 72 against 75 stored, T = 128 143 -> 75, dmmv 286 -> 135.
_EXPLICIT_BLOCK_BYTES = 8 * 2**30          # size of a stored block of K, memory permitting


def _explicit_blocks_pay(d: int, t: int, dtype: torch.dtype, opt: BaseOptions, two_products: bool = False) -> bool:
    """Whether the caller opted into stored blocks of K (``many_rhs_stored_blocks``) and t right-hand sides are
    enough for them to be the faster route.  The product kernels serve up to 64 columns with one evaluation of K
    (for fp64 up to 32 features the break-even is placed from the 64-column kernel's times: d = 28, T = 128:
    137 ms matrix-free against 134 stored for dmmv, 68 against 74 for mmv); ``two_products`` (``dmmv``) evaluates K twice on the matrix-free route and once on this
    one.  Break-even measured at N = 5e5, M = 2e4 (d = 784: N = 2.5e5, M = 1e4) for d = 9, 28, 64, 100, 784 and
    T = 17 ... 256; e.g. fp32 d = 28: mmv T = 64 17.8 ms matrix-free against 23.0 stored, T = 96 28.8 / 27.1;
    dmmv T = 64 34.8 / 33.1, T = 128 69.5 / 49.3; fp64 d = 100: dmmv T = 64 131.8 / 151.5, T = 96 229.5 / 151.7."""
    if getattr(opt, "never_store_kernel", False) or not getattr(opt, "many_rhs_stored_blocks", False):
        return False
    if dtype == torch.float64:
        least = (128, 128) if d <= 32 else (96, 64) if d <= 64 else (64, 64) if d <= 256 else (64, 16)
    else:
        least = (96, 64) if d <= 32 else (64, 32) if d <= 64 else (32, 16)
    return t > least[1 if two_products else 0]


def _block_leading_dim(M: int, sz: int) -> int:
    """Leading dimension of a stored block: rows start on multiples of 128 bytes, so that the kernel-matrix kernel's
    128-byte store segments never straddle two lines."""
    per_line = 128 // sz
    return -(-M // per_line) * per_line


def _explicit_block_rows(N: int, M: int, D: int, T: int, sz: int, dev, opt: BaseOptions, upload_bytes: int) -> int:
    """Rows of K per stored block (0: not even a sliver fits next to the operands; the caller keeps to the
    product kernels).  Per row: the block itself, its products with v, and the packed copy of the row."""
    usable = usable_gpu_memory(dev, opt.max_gpu_mem, opt.memory_slack) - upload_bytes - 2 * M * (D + T) * sz
    per_row = (_block_leading_dim(M, sz) + 2 * T + 3 * D) * sz
    rows = int(min(_EXPLICIT_BLOCK_BYTES, usable / 2) // per_row)
    return min(N, rows) if rows >= 32 else 0


def _fmmv_explicit(X1, X2, v, out, sigma_dev, kernel_fn: int, dev, opt: BaseOptions) -> bool:
    """``out = K(X1, X2) @ v`` through stored blocks of K; False if the memory budget does not allow it."""
    from .fmm import gauss_fmm_native
    (N, D), (M, T), sz = X1.shape, v.shape, sizeof_dtype(X1.dtype)
    upload = sum(t.numel() * sz for t in (X1, X2, v) if t.device != dev) + (0 if out.device == dev else N * T * sz)
    rows = _explicit_block_rows(N, M, D, T, sz, dev, opt, upload)
    if rows == 0:
        return False
    X1d, X2d, vd = _on(X1, dev), _on(X2, dev), _on(v, dev)
    outd = out if out.device == dev else torch.empty((N, T), dtype=out.dtype, device=dev)
    block = torch.empty((rows, _block_leading_dim(M, sz)), dtype=X1.dtype, device=dev)[:, :M]
    for i in range(0, N, rows):
        li = min(rows, N - i)
        gauss_fmm_native(X1d[i:i + li], X2d, sigma_dev, block[:li], False, kernel_fn, _arith_code(X1.dtype, opt))
        outd[i:i + li].copy_(block[:li] @ vd)
    if outd is not out:
        out.copy_(outd)
    return True


def _fdmmv_explicit(X1, X2, v, w, out, sigma_dev, kernel_fn: int, dev, opt: BaseOptions) -> bool:
    """``out = K^T (K v + w)`` through stored blocks of K; False if the memory budget does not allow it."""
    from .fmm import gauss_fmm_native
    (N, D), (M, T), sz = X1.shape, v.shape, sizeof_dtype(X1.dtype)
    upload = (sum(t.numel() * sz for t in (X1, X2, v, w) if t is not None and t.device != dev)
              + (0 if out.device == dev else M * T * sz))
    rows = _explicit_block_rows(N, M, D, T, sz, dev, opt, upload)
    if rows == 0:
        return False
    X1d, X2d, vd = _on(X1, dev), _on(X2, dev), _on(v, dev)
    wd = _on(w, dev) if w is not None else None
    outd = out if out.device == dev else torch.empty((M, T), dtype=out.dtype, device=dev)
    outd.zero_()
    block = torch.empty((rows, _block_leading_dim(M, sz)), dtype=X1.dtype, device=dev)[:, :M]
    for i in range(0, N, rows):
        li = min(rows, N - i)
        gauss_fmm_native(X1d[i:i + li], X2d, sigma_dev, block[:li], False, kernel_fn, _arith_code(X1.dtype, opt))
        u = block[:li] @ vd
        if wd is not None:
            u += wd[i:i + li]
        outd.addmm_(block[:li].T, u)
    if outd is not out:
        out.copy_(outd)
    return True


class PackedProducts:
    """``K(X1, X2)`` with both matrices packed once, for callers that multiply by the same kernel matrix many times
    (a conjugate-gradient solve: falkon/optim/conjgrad.py:262-285 calls ``dmmv`` on the same X and centres in every
    iteration).  The one-shot products pack their operands on every call (for a million rows of 28 features 64 us,
    5 % of a product with a thousand centres); here ``flk_kernel_pack`` runs once and every product is
    ``flk_kernel_mmv_packed`` on the packed copies, which gives bit for bit what ``fmmv`` / ``fdmmv`` give.

    ``create`` returns None where this does not apply (operands not both on one GPU, a gradient required, the bf16x3
    mode, or packed copies and workspace that do not fit the memory budget next to the data): the caller then keeps
    to ``kernel.mmv`` / ``kernel.dmmv``."""

    def __init__(self, X1, X2, kernel_fn, code, sigma_dev, p1, p2):
        self.n, self.d = X1.shape
        self.m = X2.shape[0]
        self.dtype, self.device = X1.dtype, X1.device
        self.kernel_fn, self.code, self.sigma_dev = kernel_fn, code, sigma_dev
        self.p1, self.p2 = p1, p2
        self._ws = None

    @classmethod
    def create(cls, X1: torch.Tensor, X2: torch.Tensor, kernel, opt: Optional[BaseOptions] = None,
               columns: int = 1) -> Optional["PackedProducts"]:
        opt = opt if opt is not None else BaseOptions()
        if not (X1.is_cuda and X2.is_cuda and X1.device == X2.device and X1.dim() == 2 and X2.dim() == 2):
            return None
        if X1.dtype not in _DTYPE_CODE or X1.dtype != X2.dtype or X1.shape[1] != X2.shape[1] or opt.use_cpu:
            return None
        if X1.requires_grad or X2.requires_grad or any(p.requires_grad for p in kernel.diff_params.values()):
            return None
        code = _arith_code(X1.dtype, opt)
        if code != _DTYPE_CODE[X1.dtype] or X1.shape[0] == 0 or X2.shape[0] == 0:
            return None
        try:
            kernel_fn = _kernel_fn(kernel)
            check_contiguity((X1, "X1"), (X2, "X2"))
        except (NotImplementedError, ValueError):
            return None
        lib = _backend.load()
        (n, d), m = X1.shape, X2.shape[0]
        if d > lib.flk_max_d(code):
            return None
        b1, b2 = lib.flk_gauss_packed_bytes(n, d, code), lib.flk_gauss_packed_bytes(m, d, code)
        ws = max(lib.flk_gauss_mmv_packed_workspace_bytes(m, n, d, columns, code),
                 lib.flk_gauss_mmv_packed_workspace_bytes(n, m, d, columns, code))
        sz = sizeof_dtype(X1.dtype)
        need = b1 + b2 + ws + (n + m) * columns * sz
        if need > usable_gpu_memory(X1.device, opt.max_gpu_mem, opt.memory_slack, enough=need):
            return None
        with torch.inference_mode():
            sigma_dev = kernel._sigma_on(X1.device, X1.dtype, cached=False)
            packed = []
            with _current(X1.device):
                stream = _stream_handle(X1.device)
                for A, nbytes in ((X1, b1), (X2, b2)):
                    buf = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=X1.device)
                    rc = lib.flk_kernel_pack(kernel_fn, A.data_ptr(), A.shape[0], d, A.stride(0), A.stride(1),
                                             sigma_dev.data_ptr(), sigma_dev.numel(), code, buf.data_ptr(), nbytes, stream)
                    _backend.raise_for_status(rc, "flk_kernel_pack")
                    packed.append(buf)
            made = cls(X1, X2, kernel_fn, code, sigma_dev, packed[0], packed[1])
            made._ws = torch.empty(max(ws, 1), dtype=torch.uint8, device=X1.device)     # (no allocation under a graph capture)
        return made

    def _product(self, pa, na, pb, nb, vec, addend, out):
        lib = _backend.load()
        t = vec.shape[1]
        ws_bytes = lib.flk_gauss_mmv_packed_workspace_bytes(na, nb, self.d, t, self.code)
        if self._ws is None or self._ws.numel() < ws_bytes:
            self._ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=self.device)
        add = (addend.data_ptr(), addend.stride(0), addend.stride(1)) if addend is not None else (None, 0, 0)
        with _current(self.device):
            rc = lib.flk_kernel_mmv_packed(self.kernel_fn, pa.data_ptr(), na, pb.data_ptr(), nb, self.d, vec.data_ptr(),
                                           vec.stride(0), vec.stride(1), t, *add, out.data_ptr(), out.stride(0),
                                           out.stride(1), self.code, self._ws.data_ptr(), ws_bytes,
                                           _stream_handle(self.device))
        _backend.raise_for_status(rc, "flk_kernel_mmv_packed")
        return out

    def _check(self, name, t, rows):
        if t.dim() != 2 or t.shape[0] != rows or t.dtype != self.dtype or t.device != self.device:
            raise ValueError(f"{name} must be a {rows}-row matrix of {self.dtype} on {self.device}")
        check_contiguity((t, name))

    def mmv(self, v: torch.Tensor, w: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``K(X1, X2) @ v (+ w)``, N x T."""
        self._check("v", v, self.m)
        if w is not None:
            self._check("w", w, self.n)
        out = torch.empty((self.n, v.shape[1]), dtype=self.dtype, device=self.device) if out is None else out
        return self._product(self.p2, self.m, self.p1, self.n, v, w, out)

    def mmv_t(self, u: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``K(X1, X2)^T @ u``, M x T."""
        self._check("u", u, self.n)
        out = torch.empty((self.m, u.shape[1]), dtype=self.dtype, device=self.device) if out is None else out
        return self._product(self.p1, self.n, self.p2, self.m, u, None, out)

    def dmmv(self, v: torch.Tensor, w: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``K^T (K v + w)``, M x T."""
        return self.mmv_t(self.mmv(v, w), out)


def fmmv(X1: torch.Tensor, X2: torch.Tensor, v: torch.Tensor, kernel, out: Optional[torch.Tensor] = None,
         opt: Optional[BaseOptions] = None, kwargs_m1: Optional[Dict[str, torch.Tensor]] = None,
         kwargs_m2: Optional[Dict[str, torch.Tensor]] = None) -> torch.Tensor:
    """``out = K(X1, X2) @ v`` (N x T), same contract as falkon/mmv_ops/fmmv.py:960-973 / :887-932; differentiable
    with respect to X1, X2, v and the kernel's lengthscale when any of them requires a gradient."""
    opt = opt if opt is not None else BaseOptions()
    kernel_fn = _kernel_fn(kernel)
    _reject_block_kwargs(kwargs_m1, kwargs_m2)
    check_contiguity((X1, "X1"), (X2, "X2"), (v, "v"), (out, "out"))
    kernel_params = list(kernel.diff_params.values())
    if any(t.requires_grad for t in [X1, X2, v] + kernel_params):
        return _KernelMmvFn.apply(kernel, opt, out, X1, X2, v, *kernel_params)
    return retry_with_fresh_memory_report(lambda: _fmmv_run(X1, X2, v, kernel, kernel_fn, out, opt, cached_sigma=True))


def _fmmv_run(X1, X2, v, kernel, kernel_fn: int, out, opt: BaseOptions, cached_sigma: bool) -> torch.Tensor:
    _check_dtype(X1.dtype)
    data_devs = (X1.device, X2.device, v.device)
    dev = _compute_device(opt, data_devs)
    N, D = X1.shape
    M, T = v.shape
    out = create_output_mat(out, data_devs, shape=(N, T), dtype=v.dtype, other_mat=X1)
    lib = _backend.load()
    code, sz = _arith_code(X1.dtype, opt), sizeof_dtype(X1.dtype)
    x1_in, out_in = X1.device == dev, out.device == dev

    with torch.inference_mode():
        sigma_dev = kernel._sigma_on(dev, X1.dtype, cached=cached_sigma)
        if N > 0 and M > 0 and _explicit_blocks_pay(D, T, X1.dtype, opt):
            if _fmmv_explicit(X1, X2, v, out, sigma_dev, kernel_fn, dev, opt):
                return out
        fixed = (0 if X2.device == dev else M * D * sz) + (0 if v.device == dev else M * T * sz)

        def need(rows: int) -> float:
            stage = 0 if x1_in else 2 * rows * D * sz                                    # two chunks in flight
            result = 0 if out_in else (rows if x1_in else N) * T * sz                    # see below
            return lib.flk_gauss_fmmv_workspace_bytes(rows, M, D, T, code) + stage + result + fixed

        usable = usable_gpu_memory(dev, opt.max_gpu_mem, opt.memory_slack, enough=need(N))
        blk = _rows_that_fit(N, need, usable) if N > 0 else 0
        X2d, vd = _on(X2, dev), _on(v, dev)
        if x1_in:
            for i in range(0, N, max(blk, 1)):
                li = min(blk, N - i)
                outd = out[i:i + li] if out_in else torch.empty((li, T), dtype=out.dtype, device=dev)
                gauss_fmmv_native(X1[i:i + li], X2d, sigma_dev, vd, outd, kernel_fn, code)
                if not out_in:
                    out[i:i + li].copy_(outd)
        elif N > 0:
            # host rows stream through; their results wait on the device and leave in one copy at the end
            # (a copy per chunk would stall the host, and with it the staging of the next chunk)
            chunk = _streamed_chunk_rows(N, D * sz, blk)
            full = out if out_in else torch.empty((N, T), dtype=out.dtype, device=dev)
            for i, li, (X1d,) in _HostRowStream([X1], N, dev, chunk):
                gauss_fmmv_native(X1d, X2d, sigma_dev, vd, full[i:i + li], kernel_fn, code)
            if not out_in:
                out.copy_(full)
    return out


def fdmmv(X1: torch.Tensor, X2: torch.Tensor, v: torch.Tensor, w: Optional[torch.Tensor], kernel,
          out: Optional[torch.Tensor] = None, differentiable: bool = False, opt: Optional[BaseOptions] = None,
          kwargs_m1: Optional[Dict[str, torch.Tensor]] = None,
          kwargs_m2: Optional[Dict[str, torch.Tensor]] = None) -> torch.Tensor:
    """``out = K(X1, X2).T @ (K(X1, X2) @ v + w)`` (M x T), same contract as falkon/mmv_ops/fmmv.py:976-1131.

    ``v`` is required (the reference reads ``v.shape`` unconditionally, fmmv.py:1035-1041); ``w`` may be None.
    """
    return retry_with_fresh_memory_report(
        lambda: _fdmmv_run(X1, X2, v, w, kernel, out, differentiable, opt, kwargs_m1, kwargs_m2))


def _fdmmv_run(X1, X2, v, w, kernel, out, differentiable, opt, kwargs_m1, kwargs_m2) -> torch.Tensor:
    opt = opt if opt is not None else BaseOptions()
    if differentiable:
        raise NotImplementedError(
            "Manual D-MMV is not implemented for differentiable inputs. Try using the KeOps version instead.")
    kernel_fn = _kernel_fn(kernel)
    _reject_block_kwargs(kwargs_m1, kwargs_m2)
    check_contiguity((X1, "X1"), (X2, "X2"), (v, "v"), (out, "out"))
    if v is None:
        raise ValueError("fdmmv needs `v`; to compute K.T @ w alone call mmv(X2, X1, w)")
    _check_dtype(X1.dtype)
    data_devs = [X1.device, X2.device, v.device] + ([w.device] if w is not None else [])
    dev = _compute_device(opt, data_devs)
    N, D = X1.shape[-2:]
    M, T = v.shape[-2:]
    lib = _backend.load()
    code, sz = _arith_code(X1.dtype, opt), sizeof_dtype(X1.dtype)

    with torch.inference_mode():
        out = create_output_mat(out, data_devs, shape=(M, T), dtype=v.dtype, other_mat=X1)
        x1_in, out_in = X1.device == dev, out.device == dev
        w_in = w is None or w.device == dev
        sigma_dev = kernel._sigma_on(dev, X1.dtype)
        # (opt-in beyond 64 features whatever T: a stored block costs about one pass of the product kernel there,
        # and K^T(K v + w) then needs K once instead of twice; C4: 122 -> 69 ms.  Off by default: the path is
        # specified as one that never materialises K.)
        stored = _explicit_blocks_pay(D, T, X1.dtype, opt, two_products=True) or (
            getattr(opt, "dmmv_stored_blocks", False) and D > 64 and not getattr(opt, "never_store_kernel", False))
        if N > 0 and M > 0 and stored:
            if _fdmmv_explicit(X1, X2, v, w, out, sigma_dev, kernel_fn, dev, opt):
                return out
        fixed = ((0 if X2.device == dev else M * D * sz) + (0 if v.device == dev else M * T * sz)
                 + (0 if out_in else M * T * sz))

        def need(rows: int) -> float:
            stage = 2 * ((0 if x1_in else rows * D * sz) + (0 if w_in else rows * T * sz))    # two chunks in flight
            extra = M * T * sz if rows < N else 0          # per-block result that is added into out
            return lib.flk_gauss_fdmmv_workspace_bytes(rows, M, D, T, code) + stage + fixed + extra

        usable = usable_gpu_memory(dev, opt.max_gpu_mem, opt.memory_slack, enough=need(N))
        blk = _rows_that_fit(N, need, usable) if N > 0 else 0
        X2d, vd = _on(X2, dev), _on(v, dev)
        outd = out if out_in else torch.empty((M, T), dtype=out.dtype, device=dev)
        if x1_in and w_in:
            chunks = ((i, min(blk, N - i), (X1[i:i + blk], None if w is None else w[i:i + blk]))
                      for i in range(0, N, max(blk, 1)))
        elif N > 0:
            chunk = _streamed_chunk_rows(N, (0 if x1_in else D * sz) + (0 if w_in else T * sz), blk)
            chunks = iter(_HostRowStream([X1, w], N, dev, chunk))
        else:
            chunks = iter(())
        tmp = None
        first = True
        for _, _, (X1d, wd) in chunks:
            if first:
                gauss_fdmmv_native(X1d, X2d, sigma_dev, vd, wd, outd, kernel_fn, code)
            else:
                tmp = torch.empty((M, T), dtype=out.dtype, device=dev) if tmp is None else tmp
                gauss_fdmmv_native(X1d, X2d, sigma_dev, vd, wd, tmp, kernel_fn, code)
                outd.add_(tmp)
            first = False
        if first:                                           # no rows at all: K^T (K v + w) is an empty sum
            outd.zero_()
        if not out_in:
            out.copy_(outd)
    return out
