"""The library's blocked triangular solves (flk_tri_solve, through the C ABI) against LAPACK-style solves in fp64.

They replace the triangular solves of every CG iteration (falkon/preconditioner/flk_preconditioner.py:166-256, the
library's trsm in the reference).  Checked: both directions, both storage orders of the factor, one to four
right-hand sides, sizes that are no multiple of the block or of the vector width, agreement with the torch-op path
of the same class, and bit-identical repeats (no atomics, fixed summation order)."""
import ctypes

import numpy as np
import pytest
import torch

from falkon_amd import _backend
from falkon_amd.preconditioner import _BlockedTriangular

pytestmark = pytest.mark.gpu


def _factor(m, dtype, seed, order):
    g = torch.Generator().manual_seed(seed)
    A = torch.randn(m, m + 8, dtype=torch.float64, generator=g)
    S = A @ A.T / m + 0.5 * torch.eye(m, dtype=torch.float64)
    L = torch.linalg.cholesky(S).to(dtype)
    return L.contiguous() if order == "C" else L.T.contiguous().T


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("order", ["C", "F"])
@pytest.mark.parametrize("m,block,t", [(4096, 2048, 1), (6000, 2048, 1), (5003, 1024, 2), (4500, 512, 3), (4099, 1024, 4),
                                       (700, 256, 1)])
def test_blocked_solves_match_lapack(dev, dtype, order, m, block, t):
    L = _factor(m, dtype, seed=m + t, order=order).to(dev)
    if order == "F":
        L = L.T.contiguous().T
    assert (L.stride(1) == 1) == (order == "C")
    tri = _BlockedTriangular(L, block=block, min_size=256)
    b = torch.randn(m, t, dtype=dtype, generator=torch.Generator().manual_seed(3)).to(dev)
    assert tri._native_applies(b)
    L64, b64 = L.double(), b.double()
    tol = 2e-5 if dtype == torch.float32 else 1e-12
    for transposed, solve in ((False, tri.solve), (True, tri.solve_t)):
        want = torch.linalg.solve_triangular(L64.T if transposed else L64, b64, upper=transposed)
        got = solve(b)
        assert got.shape == (m, t)
        err = float((got.double() - want).norm() / want.norm())
        assert err < tol, (transposed, err)
        # residual of the system itself, which does not depend on the conditioning of the test matrix
        op = L64.T if transposed else L64
        res = float((op @ got.double() - b64).norm() / b64.norm())
        assert res < (5e-6 if dtype == torch.float32 else 1e-13), (transposed, res)
        assert torch.equal(got, solve(b))                       # reproducible
        # the torch-op path of the same class applies the same blocks and panels
        other = tri._substitute(b, transposed)
        assert float((got.double() - other.double()).norm() / want.norm()) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("m,t", [(64, 1), (130, 2), (1001, 1), (2000, 4), (2047, 3), (3000, 1)])
def test_small_device_factors_take_the_blocked_route(dev, dtype, m, t):
    """Factors below 4096 rows on the GPU (small models: the library's single-right-hand-side triangular solve costs 0.2 to
    1 ms there) run the same blocked solve with the default sizes: one inverted block up to 2048 rows, whatever m is
    modulo 4; on the host such factors keep the library routine."""
    L = _factor(m, dtype, seed=m + t, order="C")
    assert not _BlockedTriangular(L).bounds                         # host: library solve
    tri = _BlockedTriangular(L.to(dev))
    b = torch.randn(m, t, dtype=dtype, generator=torch.Generator().manual_seed(4)).to(dev)
    assert tri.bounds and tri._native_applies(b)
    moved = _BlockedTriangular(L).to(dev)                           # built on the host, then moved
    assert moved.bounds and moved._native_applies(b)
    L64, b64 = L.double().to(dev), b.double()
    for transposed, solve, solve_moved in ((False, tri.solve, moved.solve), (True, tri.solve_t, moved.solve_t)):
        got = solve(b)
        op = L64.T if transposed else L64
        res = float((op @ got.double() - b64).norm() / b64.norm())
        assert res < (5e-6 if dtype == torch.float32 else 1e-13), (transposed, res)
        assert torch.equal(got, solve_moved(b)) and torch.equal(got, solve(b))


def test_raw_c_abi_call_and_argument_checks(dev):
    lib = _backend.load()
    m, block = 2048 + 512, 1024
    L = _factor(m, torch.float32, seed=5, order="C").to(dev)
    tri = _BlockedTriangular(L, block=block, min_size=256)
    b = torch.randn(1, m, device=dev)
    x = torch.empty_like(b)
    work = torch.empty(int(lib.flk_tri_solve_work_elems(m, 1, block)), device=dev)
    assert work.numel() == 2 * m
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    rc = lib.flk_tri_solve(_backend.FLK_F32, 0, L.data_ptr(), m, L.stride(0), 1, tri._stack.data_ptr(), tri._stack_t.data_ptr(),
                           block, b.data_ptr(), m, x.data_ptr(), m, 1, work.data_ptr(), stream)
    assert rc == 0
    want = torch.linalg.solve_triangular(L.double(), b.double().T, upper=False)
    assert float((x.double().T - want).norm() / want.norm()) < 2e-5
    # rejected: more than four right-hand sides, aliased buffers, a block size that is no multiple of 4
    assert lib.flk_tri_solve(_backend.FLK_F32, 0, L.data_ptr(), m, L.stride(0), 1, tri._stack.data_ptr(), tri._stack_t.data_ptr(),
                             block, b.data_ptr(), m, x.data_ptr(), m, 5, work.data_ptr(), stream) != 0
    assert lib.flk_tri_solve(_backend.FLK_F32, 0, L.data_ptr(), m, L.stride(0), 1, tri._stack.data_ptr(), tri._stack_t.data_ptr(),
                             block, b.data_ptr(), m, b.data_ptr(), m, 1, work.data_ptr(), stream) != 0
    assert lib.flk_tri_solve(_backend.FLK_F32, 0, L.data_ptr(), m, L.stride(0), 1, tri._stack.data_ptr(), tri._stack_t.data_ptr(),
                             1022, b.data_ptr(), m, x.data_ptr(), m, 1, work.data_ptr(), stream) != 0


def test_wide_right_hand_sides_take_the_torch_path(dev):
    L = _factor(4200, torch.float32, seed=9, order="C").to(dev)
    tri = _BlockedTriangular(L, block=1024, min_size=256)
    b = torch.randn(4200, 7, device=dev)
    assert not tri._native_applies(b)
    want = torch.linalg.solve_triangular(L.double(), b.double(), upper=False)
    assert float((tri.solve(b).double() - want).norm() / want.norm()) < 2e-5
