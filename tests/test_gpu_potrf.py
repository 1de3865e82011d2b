"""The tile kernel of the preconditioner's Cholesky factorisations (flk_potrf_tile, through the C ABI) and the blocked
factorisation built on it (falkon_amd.preconditioner._cholesky_lower_ on device matrices), against LAPACK in fp64.

Reference behaviour: falkon/preconditioner/flk_preconditioner.py:115,152 (potrf_wrapper: lower factor, LinAlgError-like
failure on a matrix that is not positive definite); falkon/tests/test_chol_prec.py:17-67 pins the factors through
their products, as the reconstruction checks below do.
"""

import pytest
import torch

from falkon_amd import _backend

pytestmark = pytest.mark.gpu

_CODE = {torch.float32: _backend.FLK_F32, torch.float64: _backend.FLK_F64}
_TOL = {torch.float32: 2e-5, torch.float64: 1e-12}


def _spd(n, dtype, seed, dev):
    g = torch.Generator().manual_seed(seed)
    B = torch.randn(n, n + 3, generator=g, dtype=torch.float64)
    A = B @ B.T / (n + 3) + torch.eye(n, dtype=torch.float64)
    return A.to(dtype).to(dev)


def _tile(lib, A, n, inv, info, base=0):
    rc = lib.flk_potrf_tile(_CODE[A.dtype], A.data_ptr(), n, A.stride(0), inv.data_ptr(), inv.stride(0), info.data_ptr(),
                            base, torch.cuda.current_stream().cuda_stream)
    _backend.raise_for_status(rc, "flk_potrf_tile")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("n", [1, 2, 5, 16, 63, 64, 100, 127, 128])
def test_tile_factor_and_inverse(n, dtype):
    dev = torch.device("cuda:0")
    lib = _backend.load()
    assert lib.flk_potrf_tile_rows(_CODE[dtype]) >= 128
    big = torch.full((n + 7, n + 9), 7.0, dtype=dtype, device=dev)          # the tile sits inside a larger matrix
    A = _spd(n, dtype, 100 + n, dev)
    big[3:3 + n, 4:4 + n] = A
    view = big[3:3 + n, 4:4 + n]
    inv = torch.full((n, n + 2), -3.0, dtype=dtype, device=dev)
    info = torch.zeros(1, dtype=torch.int32, device=dev)
    _tile(lib, view, n, inv, info)
    torch.cuda.synchronize()
    assert int(info.item()) == 0
    ref = torch.linalg.cholesky(A.double().cpu())
    got = view.tril().double().cpu()
    assert (got - ref).abs().max().item() <= _TOL[dtype] * ref.abs().max().item()
    # above the diagonal the tile is untouched, and so is everything around it
    assert torch.equal(view.triu(1), A.triu(1))
    outside = big.clone()
    outside[3:3 + n, 4:4 + n] = 7.0
    assert bool((outside == 7.0).all())
    # inv: the inverse of the factor, zeros above the diagonal, nothing written past its n columns
    X = inv[:, :n].double().cpu()
    assert torch.equal(X.triu(1), torch.zeros_like(X))
    assert bool((inv[:, n:] == -3.0).all())
    assert (X @ ref - torch.eye(n, dtype=torch.float64)).abs().max().item() <= 20 * _TOL[dtype]


def test_tile_reports_the_first_bad_pivot_and_keeps_an_earlier_failure():
    dev = torch.device("cuda:0")
    lib = _backend.load()
    n = 40
    A = _spd(n, torch.float64, 7, dev)
    A[25, 25] = -1.0                                   # the leading minor of order 26 is not positive definite
    inv = torch.empty(n, n, dtype=torch.float64, device=dev)
    info = torch.zeros(1, dtype=torch.int32, device=dev)
    _tile(lib, A.clone(), n, inv, info, base=1000)
    assert int(info.item()) == 1000 + 26
    with pytest.raises(torch.linalg.LinAlgError, match="order 26"):
        torch.linalg.cholesky(A.cpu())                 # the library reports the same order
    _tile(lib, A.clone(), n, inv, info, base=0)        # a recorded failure is not overwritten
    assert int(info.item()) == 1000 + 26
    nan = _spd(8, torch.float32, 8, dev)
    nan[2, 1] = float("nan")
    info.zero_()
    _tile(lib, nan, 8, torch.empty(8, 8, device=dev), info)
    assert int(info.item()) == 3                       # the NaN reaches the pivot of row 2


def test_tile_rejects_bad_arguments():
    dev = torch.device("cuda:0")
    lib = _backend.load()
    A = torch.eye(200, device=dev)
    inv = torch.empty(200, 200, device=dev)
    info = torch.zeros(1, dtype=torch.int32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    too_big = lib.flk_potrf_tile_rows(_backend.FLK_F32) + 1
    assert lib.flk_potrf_tile(_backend.FLK_F32, A.data_ptr(), too_big, 200, inv.data_ptr(), 200, info.data_ptr(), 0, st) != 0
    assert lib.flk_potrf_tile(_backend.FLK_F32, A.data_ptr(), 16, 8, inv.data_ptr(), 200, info.data_ptr(), 0, st) != 0
    assert lib.flk_potrf_tile(_backend.FLK_F32, A.data_ptr(), 16, 200, A.data_ptr(), 200, info.data_ptr(), 0, st) != 0
    assert lib.flk_potrf_tile(_backend.FLK_F32, None, 16, 200, inv.data_ptr(), 200, info.data_ptr(), 0, st) != 0
    assert lib.flk_potrf_tile(7, A.data_ptr(), 16, 200, inv.data_ptr(), 200, info.data_ptr(), 0, st) != 0
    assert lib.flk_potrf_tile(_backend.FLK_F32, A.data_ptr(), 0, 200, inv.data_ptr(), 200, info.data_ptr(), 0, st) == 0
    assert lib.flk_potrf_tile_rows(7) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("m,block", [(256, None), (300, None), (1000, None), (1337, 512), (2048, 512), (4100, None), (4500, 1024)])
def test_blocked_factorisation_on_the_device(m, block, dtype):
    """_cholesky_lower_ on a device matrix: tiles inside the diagonal blocks, matrix products around them."""
    from falkon_amd.preconditioner import _cholesky_lower_, _tiles_apply
    dev = torch.device("cuda:0")
    A = _spd(m, dtype, m, dev)
    assert _tiles_apply(A)
    ref = torch.linalg.cholesky(A.double().cpu())
    L = _cholesky_lower_(A.clone(), block=block)
    assert torch.equal(L.triu(1), torch.zeros_like(L))
    assert (L.double().cpu() - ref).abs().max().item() <= 4 * _TOL[dtype] * ref.abs().max().item()
    Ad = A.double().cpu()
    rec = L.double().cpu() @ L.double().cpu().T
    assert (rec - Ad).abs().max().item() <= 4 * _TOL[dtype] * Ad.abs().max().item()


def test_blocked_factorisation_of_a_kernel_matrix_and_failure():
    """The preconditioner's own case (a Gaussian kernel matrix plus eps * M on the diagonal, fp32) against the library
    routine on the same matrix, and the error a matrix that is not positive definite raises."""
    from falkon_amd import GaussianKernel
    from falkon_amd.preconditioner import _cholesky_lower_
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(5)
    C = torch.randn(3000, 10, generator=g).to(dev)
    K = GaussianKernel(3.0)(C, C)
    K.diagonal().add_(1e-5 * 3000)
    lib_factor = torch.linalg.cholesky(K)
    L = _cholesky_lower_(K.clone())
    Kd = K.double()
    err = ((L.double() @ L.double().T) - Kd).abs().max().item()
    err_lib = ((lib_factor.double() @ lib_factor.double().T) - Kd).abs().max().item()
    assert err <= max(2 * err_lib, 1e-6), (err, err_lib)
    bad = K.clone()
    bad[1500, 1500] = -1.0
    with pytest.raises(torch.linalg.LinAlgError, match="order 1501"):
        _cholesky_lower_(bad)
    # a column-major matrix keeps the library routine (the tile kernel reads rows)
    from falkon_amd.preconditioner import _tiles_apply
    assert not _tiles_apply(K.T.contiguous().T)
    torch.testing.assert_close(_cholesky_lower_(K.T.contiguous().T.clone()), lib_factor, rtol=1e-4, atol=1e-5)


def test_factorisation_at_config5_size_reconstructs_the_kernel_matrix():
    """M = 50 000 centres in 28 dimensions (config 5's preconditioner): the factor of K + eps * M * I reproduces sampled
    rows of the matrix, in double precision, to a few hundred units in the last place of its entries (the sums
    behind an entry are taken 2048 products at a time), and T T^T formed from it agrees with the double-precision
    product of the same factor on sampled rows."""
    from falkon_amd import GaussianKernel
    from falkon_amd.preconditioner import _cholesky_lower_, _gram_of_lower_factor
    dev = torch.device("cuda:0")
    M = 50_000
    g = torch.Generator().manual_seed(1005)
    C = torch.randn(M, 28, generator=g).to(dev)
    K = GaussianKernel(3.8)(C, C)
    K.diagonal().add_(1e-5 * M)
    rows = torch.tensor([0, 1, 127, 128, 2047, 2048, 4095, 4096, 25_000, 49_871, M - 1], device=dev)
    want = K[rows].double()
    L = _cholesky_lower_(K)                                    # in place: K's storage now holds the factor
    assert bool((L.diagonal() > 0).all())
    got = torch.zeros_like(want)
    for k0 in range(0, M, 5000):                               # (L L^T)[rows] in double precision, 5000 columns of L at a time
        got += L[rows, k0:k0 + 5000].double() @ L[:, k0:k0 + 5000].double().T
    assert (got - want).abs().max().item() <= 2e-5 * want.abs().max().item()
    G = _gram_of_lower_factor(L)
    cols = slice(0, 2048)
    want_g = L[:, rows].double().T @ L[:, cols].double()       # (L^T L)[rows, :2048]; valid where column <= row
    mask = torch.arange(2048, device=dev)[None, :] <= rows[:, None]
    diff = ((G[rows, cols].double() - want_g) * mask).abs().max().item()
    assert diff <= 2e-6 * want_g.abs().max().item(), (diff, want_g.abs().max().item())


@pytest.mark.parametrize("m,d,sigma", [(383, 1, 4.52), (1000, 1, 1.89), (4097, 3, 2.36), (6145, 1, 2.29)])
def test_double_precision_on_nearly_singular_kernel_matrices(m, d, sigma):
    """Kernel matrices of low-dimensional data with the double-precision jitter of 1e-13 M (condition number beyond
    1e14): the products with inverted tiles take a step of refinement there, and L L^T stays as close to the
    matrix as the library's factor leaves it (without the step: 1e-12 against 1e-14)."""
    from falkon_amd import GaussianKernel
    from falkon_amd.preconditioner import _cholesky_lower_
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(m)
    C = torch.randn(m, d, generator=g, dtype=torch.float64).to(dev)
    K = GaussianKernel(sigma)(C, C)
    K.diagonal().add_(1e-13 * m)
    lib_factor = torch.linalg.cholesky(K)
    L = _cholesky_lower_(K.clone())
    err = ((L @ L.T) - K).abs().max().item()
    err_lib = ((lib_factor @ lib_factor.T) - K).abs().max().item()
    assert err <= max(8 * err_lib, 1e-13), (err, err_lib)


def test_option_keeps_the_library_factorisation():
    """FalkonOptions(pc_tile_factorisation=False): the preconditioner's factors come from the library routine and agree
    with the default's to single-precision rounding on a well-conditioned problem."""
    from falkon_amd import FalkonOptions, GaussianKernel
    from falkon_amd.preconditioner import FalkonPreconditioner
    import falkon_amd.preconditioner as pcm
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(11)
    C = torch.randn(1500, 10, generator=g).to(dev)
    factors = {}
    for tiles in (True, False):
        opt = FalkonOptions(pc_tile_factorisation=tiles)
        calls = []
        real = pcm._cholesky_by_tiles_
        pcm._cholesky_by_tiles_ = lambda *a, **k: (calls.append(1), real(*a, **k))[1]
        try:
            pc = FalkonPreconditioner(1e-3, GaussianKernel(3.0, opt=opt), opt)
            pc.init(C)
        finally:
            pcm._cholesky_by_tiles_ = real
        assert bool(calls) == tiles
        factors[tiles] = (pc.LT.clone(), pc.LA.clone())
    for a, b in zip(factors[True], factors[False]):
        assert (a - b).abs().max().item() <= 2e-4 * b.abs().max().item()
