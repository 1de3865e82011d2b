"""Falkon's two-Cholesky Nystroem preconditioner on torch-ROCm linear algebra.

Same algebra as falkon/preconditioner/flk_preconditioner.py:94-300: with K_MM the kernel matrix of
the centres, ``T = chol(K_MM + eps*M*I)`` (upper, K = T^T T) and ``A = chol(T T^T / M + lambda*I)``
(upper); the preconditioner is ``B = 1/sqrt(n) T^-1 A^-1``.  The reference runs this on its own
out-of-core Cholesky/LAUUM; here everything is stock torch-ROCm linear algebra on the GPU, arranged so that
the work lands in routines that run near their roofline (``_cholesky_lower_``, ``_gram_of_lower_factor``).

The four triangular solves of every CG iteration (falkon/optim/conjgrad.py:262-285) have one to a few
right-hand sides, where a library ``trsm`` runs far below the memory roofline (M = 50 000: about 100 ms
per solve against 2 ms for a matrix-vector product over the same factor).  ``_BlockedTriangular`` does
the solve by blocks instead: the diagonal blocks are inverted once when the factor is built, and a
solve is then a chain of small matrix products with those inverses and matrix-vector products over
the row panels of the factor, each element of which is read once.  For a device-resident factor and up to
four right-hand sides those products are the library's own kernels (``flk_tri_solve``, csrc/trsv.hip: two
launches per diagonal block, the triangle streamed once at 5 TB/s, fixed summation order); host tensors and
wider right-hand sides take the same chain in torch ops.
"""
from typing import Optional

import torch

from .options import FalkonOptions

__all__ = ("FalkonPreconditioner", "LogisticPreconditioner")

TRSV_BLOCK = 2048        # rows per diagonal block of the blocked triangular solves
TRSV_MIN_SIZE = 4096     # smaller factors on the host go to torch.linalg.solve_triangular directly
# Device-resident factors take the blocked route from this size on: the library's triangular solve with one right-hand
# side costs 0.18 ms at M = 1 000 and 1.0 ms at M = 4 000 on the GPU, the product with the inverted block 11 to 30 us.
TRSV_MIN_SIZE_DEVICE = 64


GRAM_TERMS = 2048        # products summed at once in T T^T


def _gram_of_lower_factor(L: torch.Tensor, block: Optional[int] = None, terms: Optional[int] = None) -> torch.Tensor:
    """``L^T L`` for a lower-triangular ``L``, valid in the lower triangle (and the diagonal blocks); the
    blocks above the diagonal are left zero.  Enough for a Cholesky factorisation, which reads one triangle.

    Row block i of the product only involves rows i0.. of L (the rows above are zero in those columns) and
    only its columns up to the diagonal block are needed: M^3/3 flop instead of the 2 M^3 of a full product,
    the saving the reference gets from its LAUUM kernel (falkon/preconditioner/flk_preconditioner.py:133-138).
    The sum over the rows of L is taken ``terms`` rows at a time and added up block by block: one product over all
    M rows rounds a sum of tens of thousands of products in single precision at once (M = 40 000: entries of
    size 900 came out 6.8e-3 from the double-precision product, which is 1.7e-7 after the division by M, next to
    a penalty of 1e-6), in pieces of 2048 it is 1.9e-4, for 6 % more time.
    """
    M = L.shape[0]
    block = TRSV_BLOCK if block is None else block
    terms = GRAM_TERMS if terms is None else terms
    G = torch.zeros_like(L)
    for i0 in range(0, M, block):
        i1 = min(i0 + block, M)
        for k0 in range(i0, M, terms):
            k1 = min(k0 + terms, M)
            G[i0:i1, :i1].addmm_(L[k0:k1, i0:i1].T, L[k0:k1, :i1])
    return G


CHOL_BLOCK = 4096          # columns per panel of the blocked Cholesky factorisation
CHOL_MIN_SIZE = 16384      # smaller matrices go to torch.linalg.cholesky directly (host matrices; device: see below)
# Device-resident row-major matrices from this size on factorise their diagonal blocks by tiles (``flk_potrf_tile``): the
# library routine takes 3 us per column whatever the size (0.63 ms at 256 rows, 12.8 ms at 4096).
CHOL_TILE_MIN_SIZE = 256
# Block columns of the right-looking device factorisation: every update is then a product of 2048 terms (M = 40 000:
# 228 ms and L L^T 3.9e-6 from the matrix, against 234 ms and 6.1e-6 with 4096, 236 ms and 2.9e-6 with 1024).
CHOL_BLOCK_DEVICE = 2048


def _not_positive_definite(order: int):
    return torch.linalg.LinAlgError(
        "linalg.cholesky: The factorization could not be completed because the input is not positive-definite "
        f"(the leading minor of order {order} is not positive-definite).")


def _tiles_apply(A: torch.Tensor) -> bool:
    return (A.is_cuda and A.dim() == 2 and A.shape[0] >= CHOL_TILE_MIN_SIZE and A.stride(1) == 1
            and A.dtype in (torch.float32, torch.float64))


def _cholesky_by_tiles_(B: torch.Tensor, info: torch.Tensor, first_row: int) -> None:
    """Lower Cholesky factor of the symmetric positive definite device matrix ``B`` (row-major view; its lower triangle
    is read, all of it may be overwritten) in place, right-looking over tiles of ``flk_potrf_tile_rows`` columns: the
    library's tile kernel (csrc/potrf.hip) factorises the diagonal tile in one workgroup and returns the inverse of its
    factor, the product with that inverse solves for the rows below, and one rank-128 product updates the rest of the
    matrix.  (Left-looking, with one long product per block column, the factor came out three to seven times further
    from the double-precision one than the library's on the preconditioner's kernel matrices: a sum of thousands of
    products rounded in single precision before it meets the entry it updates.)  Nothing here waits for the GPU: a
    pivot that is not positive leaves its row number (plus ``first_row``) in ``info``, which the caller reads once."""
    from . import _backend
    from .mmv_ops.fmmv import _DTYPE_CODE, _current, _stream_handle
    lib = _backend.load()
    code = _DTYPE_CODE[B.dtype]
    n, ld, t = B.shape[0], B.stride(0), int(lib.flk_potrf_tile_rows(code))
    inv = torch.empty((t, t), dtype=B.dtype, device=B.device)
    # A product with the inverse of a tile's factor is off by the rounding error times that factor's condition number.
    # Single precision always comes with a jitter of 1e-5 M on the diagonal (condition of a factor: a few hundred) and
    # measures as close as the library; double precision comes with 1e-13 M, and on kernel matrices of one- to
    # three-dimensional data L L^T was 1e-12 from the matrix against the library's 1e-14: there the panel takes one
    # step of refinement (two more small products per tile).
    refine = B.dtype == torch.float64
    with _current(B.device):
        stream = _stream_handle(B.device)
        for j0 in range(0, n, t):
            j1 = min(j0 + t, n)
            rc = lib.flk_potrf_tile(code, B[j0:j1, j0:j1].data_ptr(), j1 - j0, ld, inv.data_ptr(), t, info.data_ptr(),
                                    first_row + j0, stream)
            _backend.raise_for_status(rc, "flk_potrf_tile")
            if j1 < n:
                inv_t = inv[:j1 - j0, :j1 - j0].T
                panel = B[j1:, j0:j1] @ inv_t
                if refine:                          # one step of refinement against the factor itself
                    residual = torch.addmm(B[j1:, j0:j1], panel, B[j0:j1, j0:j1].tril().T, alpha=-1.0)
                    panel.addmm_(residual, inv_t)
                B[j1:, j0:j1] = panel
                B[j1:, j1:].addmm_(panel, panel.T, alpha=-1.0)


def _cholesky_lower_(A: torch.Tensor, block: Optional[int] = None, min_size: Optional[int] = None,
                     use_tiles: bool = True) -> torch.Tensor:
    """Lower Cholesky factor of the symmetric positive definite ``A`` (only its lower triangle is read; ``A`` may be
    overwritten).  Raises ``torch.linalg.LinAlgError`` like the library routine if the matrix is not positive definite.

    Device matrices (row-major, from 256 rows on) are factorised in place, right-looking by block columns: the
    diagonal block by tiles (``_cholesky_by_tiles_``), the rows below it through the library's triangular solve, then
    one product per block column of the rest of the lower block triangle, so that nearly all of the M^3/3 flop run in
    large matrix products and no entry meets a sum of more than 2048 products at once (up to 4096 rows: one block,
    rank-128 updates only).  Large host matrices take the same steps with the library's factorisation of the diagonal
    blocks; small host matrices and column-major device matrices go to the library routine whole.
    """
    M = A.shape[0]
    tiles = use_tiles and _tiles_apply(A) and min_size is None
    if block is None:
        block = CHOL_BLOCK_DEVICE if tiles and M > CHOL_BLOCK else CHOL_BLOCK     # up to 4096 rows: rank-128 updates only
    min_size = CHOL_MIN_SIZE if min_size is None else min_size
    info = torch.zeros(1, dtype=torch.int32, device=A.device) if tiles else None
    if tiles and M <= block:
        _cholesky_by_tiles_(A, info, 0)
    elif M < min_size and not tiles or M <= block:
        return torch.linalg.cholesky(A)
    else:
        # right-looking by block columns: the diagonal block (by tiles on the device, by the library on the host), the
        # rows below it through the library's triangular solve, then one product per block column of the rest (its
        # lower block triangle only)
        for k0 in range(0, M, block):
            k1 = min(k0 + block, M)
            if tiles:
                _cholesky_by_tiles_(A[k0:k1, k0:k1], info, k0)
                Lkk = A[k0:k1, k0:k1].tril()
            else:
                Lkk = torch.linalg.cholesky(A[k0:k1, k0:k1])
                A[k0:k1, k0:k1] = Lkk
            if k1 < M:
                below = torch.linalg.solve_triangular(Lkk.T, A[k1:, k0:k1], upper=True, left=False)
                if tiles and A.dtype == torch.float64:
                    # the device library's solve works through inverted diagonal blocks, as the tiles do: the same
                    # step of refinement (see _cholesky_by_tiles_)
                    residual = torch.addmm(A[k1:, k0:k1], below, Lkk.T, alpha=-1.0)
                    below += torch.linalg.solve_triangular(Lkk.T, residual, upper=True, left=False)
                A[k1:, k0:k1] = below
                for c0 in range(k1, M, block):
                    c1 = min(c0 + block, M)
                    A[c0:, c0:c1].addmm_(A[c0:, k0:k1], A[c0:c1, k0:k1].T, alpha=-1.0)
    if tiles:
        failed = int(info.item())
        if failed:
            raise _not_positive_definite(failed)
    return A.tril_()


class _BlockedTriangular:
    """Solves with a lower-triangular factor L (M x M) and with its transpose.

    Both solves apply exactly transposed operators (the same inverted diagonal blocks, the same panels),
    which is what the preconditioned CG needs from ``invT`` / ``invTt`` and ``invA`` / ``invAt``.

    Every off-diagonal product runs over a panel of 2048 long, contiguous rows: of L itself when L is stored
    row-major (the part of a block row left of its diagonal block), of ``L^T`` when L is stored column-major, as
    ``torch.linalg.cholesky`` returns it (the part of a block row of the upper factor right of its diagonal
    block).  The other choice, a panel of 2048-element row fragments, runs several times slower.
    """

    def __init__(self, L: torch.Tensor, block: Optional[int] = None, min_size: Optional[int] = None):
        self.L = L
        M = L.shape[0]
        block = TRSV_BLOCK if block is None else block
        self._block, self._min_size = block, min_size
        self._set_bounds()
        self._build()

    def _set_bounds(self):
        M = self.L.shape[0]
        min_size = self._min_size
        if min_size is None:
            min_size = TRSV_MIN_SIZE_DEVICE if self.L.is_cuda else TRSV_MIN_SIZE
        self.bounds = [(k, min(k + self._block, M)) for k in range(0, M, self._block)] if M >= min_size else []

    def _build(self):
        L = self.L
        M = L.shape[0]
        self.row_major = M < 2 or L.stride(1) == 1
        self.dinv, self.panels = [], []
        self._stack = self._stack_t = None
        if not self.bounds:
            return
        block = self.bounds[0][1] - self.bounds[0][0]
        if len(self.bounds) == 1:
            block = (block + 3) // 4 * 4             # a single block: any leading dimension serves; flk_tri_solve wants a multiple of 4
        # the inverted diagonal blocks, block k at [k] with leading dimension `block` (zero beyond a smaller last
        # block), and their transposes: the layout flk_tri_solve reads; the torch path uses views of the same memory
        self._stack = torch.zeros(len(self.bounds), block, block, dtype=L.dtype, device=L.device)
        for k, (k0, k1) in enumerate(self.bounds):
            eye = torch.eye(k1 - k0, dtype=L.dtype, device=L.device)
            self._stack[k, :k1 - k0, :k1 - k0] = torch.linalg.solve_triangular(L[k0:k1, k0:k1], eye, upper=False).tril_()
            self.dinv.append(self._stack[k, :k1 - k0, :k1 - k0])
            # views with unit column stride: L[k, :k] (row-major L) or (L^T)[k, k+1:] (column-major L)
            self.panels.append(L[k0:k1, :k0] if self.row_major else L[k1:, k0:k1].T)
        if L.is_cuda:
            self._stack_t = self._stack.transpose(1, 2).contiguous()

    def to(self, device):
        self.L = self.L.to(device)
        self._set_bounds()
        self._build()
        return self

    NATIVE_MAX_RHS = 4

    def _native_applies(self, b: torch.Tensor) -> bool:
        """The library's solve (``flk_tri_solve``: two launches per diagonal block, every element of the factor read
        once at streaming rate) serves device-resident fp32 / fp64 factors with up to four right-hand sides; the
        torch-op path below serves host tensors and wider right-hand sides."""
        L = self.L
        return (self._stack_t is not None and self._stack.shape[1] % 4 == 0 and b.is_cuda and b.device == L.device
                and b.dtype == L.dtype
                and L.dtype in (torch.float32, torch.float64) and b.dim() == 2 and 1 <= b.shape[1] <= self.NATIVE_MAX_RHS
                and (L.stride(1) == 1 or L.stride(0) == 1))

    def _solve_native(self, b: torch.Tensor, transposed: bool) -> torch.Tensor:
        from . import _backend
        from .mmv_ops.fmmv import _current, _stream_handle
        lib = _backend.load()
        L = self.L
        m, t = b.shape
        cols = b.T.contiguous()                     # [t][m]: one contiguous column per right-hand side
        ld = L.stride(0) if self.row_major else L.stride(1)
        block = self._stack.shape[1]
        x = torch.empty_like(cols)
        work = torch.empty(int(lib.flk_tri_solve_work_elems(m, t, block)), dtype=L.dtype, device=L.device)
        code = _backend.FLK_F32 if L.dtype == torch.float32 else _backend.FLK_F64
        with _current(L.device):
            rc = lib.flk_tri_solve(code, int(transposed), L.data_ptr(), m, ld, int(self.row_major), self._stack.data_ptr(),
                                   self._stack_t.data_ptr(), block, cols.data_ptr(), m, x.data_ptr(), m, t, work.data_ptr(),
                                   _stream_handle(L.device))
        _backend.raise_for_status(rc, "flk_tri_solve")
        return x.view(m, 1) if t == 1 else x.T

    @staticmethod
    def _as_columns(b: torch.Tensor):
        """One right-hand side goes through the matrix-vector routines (a one-column matrix product runs at a
        fifth of their rate): returns the working view and the matching product functions."""
        if b.shape[1] == 1:
            return b[:, 0], torch.mv, torch.addmv
        return b, torch.mm, torch.addmm

    def _substitute(self, b: torch.Tensor, transposed: bool) -> torch.Tensor:
        rhs, mul, addmul = self._as_columns(b)
        # row-major L: L x = b looks left (panel_k x[:k0]) and L^T x = b pushes right-to-left (panel_k^T x_k);
        # column-major L: the roles swap, with panels of L^T
        ascending = not transposed
        looks_back = self.row_major != transposed        # each block subtracts panel_k times the solved part
        order = range(len(self.bounds)) if ascending else range(len(self.bounds) - 1, -1, -1)
        x = torch.empty_like(rhs, memory_format=torch.contiguous_format)
        r = rhs if looks_back else rhs.clone(memory_format=torch.contiguous_format)
        for k in order:
            k0, k1 = self.bounds[k]
            dinv = self.dinv[k].T if transposed else self.dinv[k]
            panel = self.panels[k]
            solved = slice(0, k0) if self.row_major else slice(k1, None)   # the rows the panel's columns index
            if looks_back:
                rk = addmul(r[k0:k1], panel, x[solved], alpha=-1.0) if panel.shape[1] > 0 else r[k0:k1]
                mul(dinv, rk, out=x[k0:k1])
            else:
                xk = x[k0:k1]
                mul(dinv, r[k0:k1], out=xk)
                if panel.shape[1] > 0:
                    addmul(r[solved], panel.T, xk, alpha=-1.0, out=r[solved])
        return x.unsqueeze(1) if b.shape[1] == 1 else x

    def solve(self, b: torch.Tensor) -> torch.Tensor:
        """x with L x = b."""
        if not self.bounds:
            return torch.linalg.solve_triangular(self.L, b, upper=False)
        if self._native_applies(b):
            return self._solve_native(b, transposed=False)
        return self._substitute(b, transposed=False)

    def solve_t(self, b: torch.Tensor) -> torch.Tensor:
        """x with L^T x = b."""
        if not self.bounds:
            return torch.linalg.solve_triangular(self.L.T, b, upper=True)
        if self._native_applies(b):
            return self._solve_native(b, transposed=True)
        return self._substitute(b, transposed=True)


class FalkonPreconditioner:
    def __init__(self, penalty: float, kernel, opt: Optional[FalkonOptions] = None):
        self.params = opt if opt is not None else FalkonOptions()
        self._lambda = penalty
        self.kernel = kernel
        self.LT: Optional[torch.Tensor] = None   # lower factor of K_MM + eps*M*I  (T = LT^T)
        self.LA: Optional[torch.Tensor] = None   # lower factor of T T^T / M + lambda*I  (A = LA^T)
        self._T: Optional[_BlockedTriangular] = None
        self._A: Optional[_BlockedTriangular] = None

    def init(self, X: torch.Tensor, weight_vec: Optional[torch.Tensor] = None) -> None:
        """Factorise for the centres X.  ``weight_vec`` (M x 1, the weights of the centres) is for weighted least
        squares: ``A = chol(T W T^T / M + lambda I)``, the reference's CPU algebra (flk_preconditioner.py:122-127,
        which weighs the columns of T by sqrt(w) before the triangular product)."""
        M = X.shape[0]
        if weight_vec is not None and weight_vec.numel() != M:
            raise ValueError(f"weight_vec must have one entry per centre ({M}), found {weight_vec.numel()}")
        with torch.inference_mode():
            C = self.kernel(X, X, opt=self.params)                     # fp64-computed when no_single_kernel
            eps = self.params.pc_epsilon(C.dtype)
            C.diagonal().add_(eps * M)
            LT = _cholesky_lower_(C, use_tiles=self.params.pc_tile_factorisation)
            del C
            if weight_vec is None:
                G = _gram_of_lower_factor(LT)                           # T T^T, lower triangle only
            else:                                                       # T W T^T = (sqrt(W) LT)^T (sqrt(W) LT)
                root = weight_vec.reshape(-1, 1).to(device=LT.device, dtype=LT.dtype).sqrt()
                G = _gram_of_lower_factor(LT * root)
            G.mul_(1.0 / M)
            G.diagonal().add_(self._lambda)
            self.LA = _cholesky_lower_(G, use_tiles=self.params.pc_tile_factorisation)
            self.LT = LT
            self._T, self._A = _BlockedTriangular(self.LT), _BlockedTriangular(self.LA)

    def _check(self):
        if self.LT is None or self.LA is None:
            raise RuntimeError("FALKON preconditioner is not initialized. Please run `init` before any other "
                               "method on the preconditioner.")

    def to(self, device):
        if self.LT is not None:
            self._T, self._A = self._T.to(device), self._A.to(device)
            self.LT, self.LA = self._T.L, self._A.L
        return self

    def invA(self, v):
        self._check()
        return self._A.solve_t(v)            # A = LA^T

    def invAt(self, v):
        self._check()
        return self._A.solve(v)

    def invT(self, v):
        self._check()
        return self._T.solve_t(v)            # T = LT^T

    def invTt(self, v):
        self._check()
        return self._T.solve(v)

    def apply(self, v):
        """T^-1 A^-1 v: preconditioned solution -> kernel coefficients."""
        return self.invT(self.invA(v))

    def apply_t(self, v):
        """A^-T T^-T v."""
        return self.invAt(self.invTt(v))


class LogisticPreconditioner(FalkonPreconditioner):
    """The preconditioner of one Newton step of Logistic Falkon (falkon/preconditioner/logistic_preconditioner.py:17-350):
    ``T = chol(K_MM + eps*M*I)`` once, then for every step ``A = chol(T W T^T / N + penalty*I)`` with
    ``W = diag(l''(Y_M, T^T beta))``, the loss' curvature at the centres for the current iterate (``T^T beta`` are
    the function values at the centres, since the coefficients are ``T^-1 beta``)."""

    def __init__(self, kernel, loss, opt: Optional[FalkonOptions] = None):
        super().__init__(0.0, kernel, opt)
        self.loss = loss

    def init(self, X: torch.Tensor, Y: torch.Tensor, alpha: torch.Tensor, penalty: float, N: int) -> None:
        if Y.shape[1] != 1:
            raise ValueError("Logistic preconditioner can only deal with 1D outputs.")
        M = X.shape[0]
        with torch.inference_mode():
            if self.LT is None:                                         # first step only
                C = self.kernel(X, X, opt=self.params)
                C.diagonal().add_(self.params.pc_epsilon(C.dtype) * M)
                self.LT = _cholesky_lower_(C, use_tiles=self.params.pc_tile_factorisation)
                self._T = _BlockedTriangular(self.LT)
            at_centres = self.LT @ alpha.to(self.LT.dtype)              # T^T beta
            root = self.loss.ddf(Y.to(self.LT.dtype), at_centres).reshape(-1, 1).sqrt()
            G = _gram_of_lower_factor(self.LT * root)                   # T W T^T, lower triangle
            G.mul_(1.0 / N)                                             # 1/N here, not 1/M (logistic_preconditioner.py:146)
            G.diagonal().add_(penalty)
            self.LA = _cholesky_lower_(G, use_tiles=self.params.pc_tile_factorisation)
            self._A = _BlockedTriangular(self.LA)
            self._lambda = penalty
