"""Configurations 2, 3 and 4 at their full sizes on the GPU.

The CPU oracle cannot run these sizes in test time, so parity is checked where the structure of the
problem makes a piece of it cheap (rows of ``K v`` are independent; a few columns of ``K`` give a few
rows of ``K^T u``) and through properties that hold at any size: the adjoint identity that ties the two
orientations of the product kernel together, ``dmmv`` = composition of two ``mmv``, linearity in ``v``,
invariance under a permutation of the rows of X, the closed form for sigma -> infinity, run-to-run
determinism.  Tolerances: 1e-5 (fp32) and 1e-11 (fp64), relative, norm-wise per output column.
"""
import numpy as np
import pytest
import torch

from falkon_amd import FalkonOptions, GaussianKernel
from oracle import gaussian_ref, inputs, mmv_ref
from conftest import check_parity, rel_err

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.float64: 1e-11}


def _columns_of_kt_u(X, C_sub, sigma, u, block=500_000):
    """(K(X, C_sub))^T u in fp64 on the CPU, row block by row block (rbf_core restated, fp64)."""
    acc = torch.zeros(C_sub.shape[0], u.shape[1], dtype=torch.float64)
    Cd = C_sub.double()
    for i in range(0, X.shape[0], block):
        Kb = gaussian_ref.rbf_core_ref(X[i:i + block].double(), Cd, None, sigma)
        acc += Kb.T @ u[i:i + block].double()
    return acc


def _full_size_checks(dev, name, dtype, n_rows=3000, n_centres=48, bf16x3=False, d=None, T=None):
    X, C, sigma, v, w = inputs.make_config(name, dtype=dtype, d=d, T=T)
    opt = FalkonOptions(bf16x3_cross_term=bf16x3)
    N, M, T = X.shape[0], C.shape[0], v.shape[1]
    tol = TOL[dtype]
    g = np.random.default_rng(7)
    k = GaussianKernel(sigma, opt=opt)
    Xg, Cg, vg = X.to(dev), C.to(dev), v.to(dev)
    wg = w.to(dev) if w is not None else None

    u = k.mmv(Xg, Cg, vg)                       # N x T
    out = k.dmmv(Xg, Cg, vg, wg)                # M x T
    assert u.shape == (N, T) and out.shape == (M, T) and bool(torch.isfinite(out).all())

    # (1) rows of K v are independent of each other: a random subset against the CPU oracle
    rows = torch.from_numpy(np.sort(g.choice(N, n_rows, replace=False)))
    Xs = X[rows].contiguous()
    check_parity(u[rows.to(dev)], mmv_ref.fmmv_ref(Xs, C, v, sigma),
                 mmv_ref.fmmv_ref(Xs.double(), C.double(), v.double(), sigma), tol)

    # (2) a few rows of K^T (K v + w): needs only those columns of K, all N rows, fp64 on the CPU
    J = torch.from_numpy(np.sort(g.choice(M, n_centres, replace=False)))
    uw = (u if wg is None else u + wg).cpu()
    exp_J = _columns_of_kt_u(X, C[J], sigma, uw)
    assert rel_err(out[J.to(dev)], exp_J) < tol

    # (3) adjoint identity <z, K v> = <K^T z, v> (K^T z is the other orientation of the product kernel)
    z = torch.from_numpy(g.standard_normal((N, T))).to(dtype).to(dev)
    ktz = k.mmv(Cg, Xg, z)
    lhs = (z.double() * u.double()).sum(0)
    rhs = (ktz.double() * vg.double()).sum(0)
    scale = z.double().norm(dim=0) * u.double().norm(dim=0)
    assert float(((lhs - rhs).abs() / scale).max()) < tol

    # (4) dmmv is the composition of the two products
    comp = k.mmv(Cg, Xg, u if wg is None else u + wg)
    assert rel_err(out, comp) < tol / 10

    # (5) linearity in v
    v2 = torch.from_numpy(g.standard_normal((M, T))).to(dtype).to(dev)
    lin = k.mmv(Xg, Cg, 2.0 * vg - 3.0 * v2)
    assert rel_err(lin, 2.0 * u - 3.0 * k.mmv(Xg, Cg, v2)) < tol

    # (6) a permutation of the rows of X (and w) leaves K^T (K v + w) unchanged
    perm = torch.from_numpy(g.permutation(N)).to(dev)
    out_p = k.dmmv(Xg[perm], Cg, vg, wg[perm] if wg is not None else None)
    assert rel_err(out_p, out) < tol
    del perm, out_p

    # (7) sigma -> infinity: K -> 1, K v -> column sums of v
    flat = GaussianKernel(1e7, opt=opt).mmv(Xg, Cg, vg)
    sums = vg.double().sum(0, keepdim=True)
    assert float(((flat.double() - sums).abs().max(0).values / vg.double().abs().sum(0)).max()) < tol

    # (8) run-to-run determinism (fixed-order reduction, no atomics)
    assert torch.equal(out, k.dmmv(Xg, Cg, vg, wg))


@pytest.mark.parametrize("bf16x3", [False, True], ids=["fp32-mfma", "bf16x3"])
def test_config2_full_size(dev, bf16x3):
    """N=1e6, d=28, M=20000, T=1, sigma=3.8, fp32 (plain, and with the cross term on the bf16 matrix cores)."""
    _full_size_checks(dev, "C2", torch.float32, bf16x3=bf16x3)


def test_config2_full_size_against_the_cpu_path(dev):
    """The headline configuration, every row, against the reference-equivalent CPU path run on the CPU in fp32
    (max_cpu_mem = 16 GiB) and in fp64.  Three distances, every anchor CPU-computed:
    GPU fp32 to CPU fp64, CPU fp32 to CPU fp64, GPU fp32 to CPU fp32; and GPU fp64 to CPU fp64 at 1e-11.
    The fp32 CPU path accumulates ``out.addmm_(K.T, u)`` over a million positive terms in fp32
    (falkon/mmv_ops/fmmv.py:740-762) and ends up about 1.5e-5 from its fp64 twin, so the literal
    'GPU fp32 within 1e-5 of CPU fp32' can only hold if the GPU result shared that drift.  What is asserted instead
    where it does not hold: the GPU fp32 result is within 1e-5 of the fp64 CPU result (measured: 3e-7), closer to it
    than the fp32 CPU path is, and the gap between the two fp32 results is the CPU path's own error (triangle
    inequality, to 10 %)."""
    X, C, sigma, v, w = inputs.make_config("C2", dtype=torch.float32)
    k = GaussianKernel(sigma)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    gpu32 = k.dmmv(Xg, Cg, vg, wg).cpu()
    gpu64 = k.dmmv(Xg.double(), Cg.double(), vg.double(), wg.double()).cpu()
    del Xg, wg
    cpu32 = mmv_ref.fdmmv_ref(X, C, v, w, sigma, max_cpu_mem=16 * 2**30)
    cpu64 = mmv_ref.fdmmv_ref(X.double(), C.double(), v.double(), w.double(), sigma, max_cpu_mem=16 * 2**30)
    e_gpu32, e_cpu32, e_pair = rel_err(gpu32, cpu64), rel_err(cpu32, cpu64), rel_err(gpu32, cpu32)
    e_gpu64 = rel_err(gpu64, cpu64)
    print(f"C2 full size: gpu32-cpu64 {e_gpu32:.3e}  cpu32-cpu64 {e_cpu32:.3e}  gpu32-cpu32 {e_pair:.3e}  "
          f"gpu64-cpu64 {e_gpu64:.3e}")
    assert e_gpu64 < TOL[torch.float64]
    assert e_gpu32 < 1e-6                                  # far inside the fp32 bar against the fp64 CPU result
    if e_pair >= TOL[torch.float32]:
        assert e_gpu32 < e_cpu32 / 10                      # the GPU is the more accurate of the two fp32 results
        assert abs(e_pair - e_cpu32) < 0.1 * e_cpu32       # and their distance is the CPU path's own error
        assert e_pair < 10 * TOL[torch.float32]


@pytest.mark.parametrize("d,t", [(40, 1), (64, 1), (96, 1), (128, 1), (100, 3)])
def test_config2_shape_at_33_to_128_features(dev, d, t):
    """Configuration 2's sizes with 40 to 128 features: the register-resident fp32 kernels with four, three (one column)
    or two (three columns) resident blocks per wave, from 65 features on on operands packed for the LDS-tiled kernel."""
    _full_size_checks(dev, "C2", torch.float32, n_rows=1500, n_centres=24, d=d, T=t)


@pytest.mark.parametrize("bf16x3", [False, True], ids=["fp32-mfma", "bf16x3"])
def test_config3_full_size(dev, bf16x3):
    """N=1e7, d=9, M=50000, T=1, per-dimension sigma, w=None, fp32."""
    _full_size_checks(dev, "C3", torch.float32, n_rows=2000, n_centres=24, bf16x3=bf16x3)


@pytest.mark.parametrize("dtype,bf16x3", [(torch.float32, False), (torch.float32, True), (torch.float64, False)],
                         ids=["fp32-mfma", "bf16x3", "fp64"])
def test_config4_full_size(dev, dtype, bf16x3):
    """N=5e5, d=784 (80 % zeros), M=10000, T=10, sigma=10, fp32 (both modes) and fp64."""
    _full_size_checks(dev, "C4", dtype, n_rows=2000, n_centres=32, bf16x3=bf16x3)


@pytest.mark.parametrize("name,dtype,t", [("C2", torch.float32, 64), ("C2", torch.float32, 40), ("C2", torch.float64, 64),
                                          ("C4", torch.float32, 64), ("C4", torch.float64, 64), ("C4", torch.float32, 24)],
                         ids=["C2-fp32-64", "C2-fp32-40", "C2-fp64-64", "C4-fp32-64", "C4-fp64-64", "C4-fp32-24"])
def test_many_columns_full_size(dev, name, dtype, t):
    """The matrices of configurations 2 and 4 with 24 to 64 right-hand sides (one evaluation of K serves them all): rows of
    K v against the CPU oracle, the adjoint identity in every column, and sampled columns of K^T (K v + w) against the
    single-column kernels, which the tests above check at this size."""
    X, C, sigma, _, _ = inputs.make_config(name, dtype=dtype)
    N, M = X.shape[0], C.shape[0]
    tol = TOL[dtype]
    g = np.random.default_rng(11)
    v = torch.from_numpy(g.standard_normal((M, t))).to(dtype)
    w = torch.from_numpy(g.standard_normal((N, t))).to(dtype)
    k = GaussianKernel(sigma)
    Xg, Cg, vg, wg = X.to(dev), C.to(dev), v.to(dev), w.to(dev)
    u = k.mmv(Xg, Cg, vg)
    out = k.dmmv(Xg, Cg, vg, wg)
    assert u.shape == (N, t) and out.shape == (M, t) and bool(torch.isfinite(out).all())
    rows = torch.from_numpy(np.sort(g.choice(N, 1000, replace=False)))
    Xs = X[rows].contiguous()
    check_parity(u[rows.to(dev)], mmv_ref.fmmv_ref(Xs, C, v, sigma),
                 mmv_ref.fmmv_ref(Xs.double(), C.double(), v.double(), sigma), tol)
    z = torch.from_numpy(g.standard_normal((N, t))).to(dtype).to(dev)
    ktz = k.mmv(Cg, Xg, z)
    lhs, rhs = (z.double() * u.double()).sum(0), (ktz.double() * vg.double()).sum(0)
    scale = z.double().norm(dim=0) * u.double().norm(dim=0)
    assert float(((lhs - rhs).abs() / scale).max()) < tol
    cols = sorted(c for c in {0, 15, 16, 31, 32, t - 1} if c < t)
    for c in cols:
        one = k.dmmv(Xg, Cg, vg[:, c:c + 1].contiguous(), wg[:, c:c + 1].contiguous())
        assert rel_err(out[:, c:c + 1], one) < tol, c
    assert torch.equal(out, k.dmmv(Xg, Cg, vg, wg))


@pytest.mark.parametrize("bf16x3", [False, True], ids=["fp32-mfma", "bf16x3"])
def test_kernel_matrix_large_square(dev, bf16x3):
    """K(A, A) for 30 000 rows of 256 features, evaluated in fp32 (3.6 GB): properties no sample can miss — a unit
    diagonal and symmetry (each to rounding of the expanded norm), the F-ordered result equal to the transpose —
    and 40 rows against the fp64 closed form."""
    from oracle import brute
    n, d, sigma = 30_000, 256, 16.0
    g = torch.Generator().manual_seed(77)
    A = torch.randn(n, d, generator=g, dtype=torch.float32)
    Ag = A.to(dev)
    k = GaussianKernel(sigma, opt=FalkonOptions(no_single_kernel=False, bf16x3_cross_term=bf16x3))
    K = k(Ag, Ag)
    assert float((K.diagonal() - 1).abs().max()) < 2e-5
    assert float((K - K.T).abs().max()) < 2e-6
    Kf = k(Ag, Ag, out=torch.empty(n, n, dtype=torch.float32, device=dev).T)
    assert float((Kf - K).abs().max()) < 2e-6
    rows = torch.randint(0, n, (40,), generator=g)
    exact = torch.from_numpy(brute.gaussian_brute(A[rows], A, torch.tensor([sigma], dtype=torch.float64)))
    assert float((K[rows.to(dev)].cpu().double() - exact).abs().max()) < 2e-6
    assert torch.isfinite(K).all()
