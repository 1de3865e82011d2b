"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs.

Tolerances are the ones the task states: relative error (norm-wise per output column)
1e-5 in fp32 and 1e-11 in fp64 against the reference-equivalent CPU path (``oracle.mmv_ref``).
"""
import numpy as np
import pytest
import torch

from falkon_amd import FalkonOptions, GaussianKernel
from oracle import brute, inputs, mmv_ref
from conftest import check_parity, rel_err, scaled_err

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.float64: 1e-11}


def _rand(n, d, m, t, dtype, seed, scale=1.0):
    g = np.random.default_rng(seed)
    np_dt = np.float32 if dtype == torch.float32 else np.float64
    X = torch.from_numpy((g.standard_normal((n, d)) * scale).astype(np_dt))
    C = torch.from_numpy((g.standard_normal((m, d)) * scale).astype(np_dt))
    v = torch.from_numpy(g.standard_normal((m, t)).astype(np_dt))
    w = torch.from_numpy(g.standard_normal((n, t)).astype(np_dt))
    return X, C, v, w


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("n,m,d,t", [
    (20, 5, 3, 2),          # the reference's basic test shape (tests/test_kernels.py:32-35)
    (1500, 250, 3, 2),      # its multi-block shape (:529-535)
    (100, 250, 28, 1),
    (1000, 333, 9, 1),
    (777, 129, 1, 3),
    (515, 1031, 17, 4),
    (300, 200, 33, 5),
    (257, 100, 64, 1),
    (64, 64, 2, 7),
    (2000, 900, 10, 10),    # the reference's mmv benchmark columns (benchmarks/timing_benchmarks/mmv_timings.py:48-127)
    (400, 3000, 9, 16),
    (600, 500, 28, 6),
    (500, 400, 31, 21),     # more columns than one pass holds
    (300, 300, 40, 9),      # d > 32: column chunks of four
    (700, 1300, 40, 1),     # 33 .. 64 features, one column: four resident blocks per wave (fp32), two waves per SIMD
    (333, 1111, 47, 1),     # ... an odd feature count, and 48 padded features: from there on one wave per SIMD
    (450, 2049, 63, 1),
    (450, 700, 50, 2),      # two columns keep two resident blocks
])
def test_mmv_dmmv_vs_oracle(dev, dtype, n, m, d, t):
    X, C, v, w = _rand(n, d, m, t, dtype, seed=n * 7 + m)
    sigma = 1.0 + 0.5 * np.sqrt(d)
    k = GaussianKernel(sigma)
    exp_mmv = mmv_ref.fmmv_ref(X, C, v, sigma)
    exp_dmmv = mmv_ref.fdmmv_ref(X, C, v, w, sigma)
    exp_dmmv_now = mmv_ref.fdmmv_ref(X, C, v, None, sigma)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    got_mmv = k.mmv(Xg, Cg, vg)
    got_dmmv = k.dmmv(Xg, Cg, vg, wg)
    got_dmmv_now = k.dmmv(Xg, Cg, vg, None)
    assert got_mmv.shape == (n, t) and got_dmmv.shape == (m, t)
    assert rel_err(got_mmv, exp_mmv) < TOL[dtype]
    assert rel_err(got_dmmv, exp_dmmv) < TOL[dtype]
    assert rel_err(got_dmmv_now, exp_dmmv_now) < TOL[dtype]
    # and against the closed form, which does not share the expanded-norm route
    assert rel_err(got_mmv, brute.mmv_brute(X, C, sigma, v)) < 5 * TOL[dtype]
    assert rel_err(got_dmmv, brute.dmmv_brute(X, C, sigma, v, w)) < 5 * TOL[dtype]


@pytest.mark.parametrize("order", ["C", "F"])
@pytest.mark.parametrize("sig", ["single", "vec"])
def test_reference_fixture_fp64(dev, order, sig):
    """Reference TestGaussianKernel.test_dense_kernel: seeds 92..95, n=20 m=5 d=3 t=2, fp64,
    sigma 3.0 and [3,3,3], C and F order, rtol=atol=1e-8 (tests/test_kernels.py:299-319)."""
    A, B, v, w = inputs.reference_test_mats(20, 5, 3, 2, np.float64, order)
    sigma = torch.tensor([3.0]) if sig == "single" else torch.tensor([3.0] * 3)
    k = GaussianKernel(sigma)
    K = torch.from_numpy(brute.gaussian_brute(A, B, sigma))
    Ag, Bg, vg, wg = (a.to(dev) for a in (A, B, v, w))
    if order == "F":
        Ag, Bg, vg, wg = (torch.empty_strided(a.shape, (1, a.shape[0]), dtype=a.dtype, device=dev).copy_(a) for a in (Ag, Bg, vg, wg))
    out = torch.empty(20, 2, dtype=torch.float64, device=dev)
    got = k.mmv(Ag, Bg, vg, out=out)
    assert got.data_ptr() == out.data_ptr(), "MMV output tensor was not used"
    torch.testing.assert_close(got.cpu(), K @ v, rtol=1e-8, atol=1e-8)
    torch.testing.assert_close(k.mmv(Ag, Bg, vg).cpu(), K @ v, rtol=1e-8, atol=1e-8)
    dout = torch.empty(5, 2, dtype=torch.float64, device=dev)
    dgot = k.dmmv(Ag, Bg, vg, wg, out=dout)
    assert dgot.data_ptr() == dout.data_ptr(), "D-MMV output tensor was not used"
    torch.testing.assert_close(dgot.cpu(), K.T @ (K @ v + w), rtol=1e-8, atol=1e-8)
    torch.testing.assert_close(k.dmmv(Ag, Bg, vg, wg).cpu(), K.T @ (K @ v + w), rtol=1e-8, atol=1e-8)
    # output follows X1's memory order (mmv_ops/utils.py:124-155)
    assert (k.mmv(Ag, Bg, vg).stride(0) == 1) == (order == "F")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("n,m,d,t", [
    (100, 250, 110, 2),     # the reference's large-d shape (tests/test_kernels.py:594-601)
    (300, 257, 65, 1),      # 65 .. 128 features, one column: the register-resident fp32 kernel on operands packed for the
    (1500, 1030, 72, 1),    # LDS-tiled one (fp64 and more columns: the LDS-tiled kernel); an odd number of reduction blocks
    (260, 3000, 81, 1),
    (900, 520, 96, 1),
    (900, 520, 97, 1),      # 97 .. 128 features: three resident blocks per wave
    (1100, 2100, 112, 1),
    (700, 1033, 113, 1),
    (520, 900, 128, 1),
    (520, 900, 129, 1),     # first d beyond the register-resident kernels
    (640, 333, 90, 2),      # ... two to four columns up to 128 features: two resident blocks per wave
    (300, 1400, 70, 4),
    (500, 300, 127, 3),
    (500, 300, 128, 5),     # five columns beyond 64 features: the LDS-tiled kernel
    (1000, 700, 200, 3),
    (513, 300, 784, 10),    # configuration 4's d and T
    (40, 1100, 131, 17),    # more columns than one pass holds, odd d
    (700, 20, 1000, 5),
    (600, 400, 96, 16),     # a full 16-column pass (the MFMA contraction of kernel values against v)
    (333, 520, 300, 7),
    (257, 129, 70, 8),      # eight columns (per-lane FMAs in fp64), a last feature chunk that is mostly padding
    (130, 300, 97, 9),      # one real feature in the last chunk
    (400, 300, 784, 32),    # 17 .. 32 columns in one pass: the full width of the fp32 step, two groups of 16 in fp64
    (260, 300, 97, 24),     # ... partly filled, with whole feature chunks of padding behind the data (fp64: chunks of 16)
    (150, 520, 131, 48),    # 33 .. 64 columns in one pass: column groups on one evaluation of K, the last one half full
    (300, 200, 70, 64),
    (280, 150, 200, 70),    # a 64-column pass and a narrow one
])
def test_large_d_vs_oracle(dev, dtype, n, m, d, t):
    """d > 64 runs the LDS-tiled kernel (up to 64 right-hand sides per pass); same tolerances against the blocked CPU
    oracle."""
    X, C, v, w = _rand(n, d, m, t, dtype, seed=n + d, scale=0.5)
    sigma = 0.6 * np.sqrt(d)
    k = GaussianKernel(sigma)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    got_mmv = k.mmv(Xg, Cg, vg)
    got_dmmv = k.dmmv(Xg, Cg, vg, wg)
    assert rel_err(got_mmv, mmv_ref.fmmv_ref(X, C, v, sigma)) < TOL[dtype]
    assert rel_err(got_dmmv, mmv_ref.fdmmv_ref(X, C, v, w, sigma)) < TOL[dtype]
    assert rel_err(got_mmv, brute.mmv_brute(X, C, sigma, v)) < 5 * TOL[dtype]
    if t > 16:      # several passes of the product kernels above; the opt-in stored-block route as well
        kf = GaussianKernel(sigma, opt=FalkonOptions(many_rhs_stored_blocks=True))
        assert rel_err(kf.mmv(Xg, Cg, vg), mmv_ref.fmmv_ref(X, C, v, sigma)) < TOL[dtype]
        assert rel_err(kf.dmmv(Xg, Cg, vg, wg), mmv_ref.fdmmv_ref(X, C, v, w, sigma)) < TOL[dtype]


def test_config4_shape_reduced(dev):
    """Config 4 (d=784, T=10, sigma=10, 80 % zeros) at N=20000, M=2000, fp32 and fp64, fmmv and dfmmv.

    All kernel values lie in [0.53, 1] here, so a column of K v is close to mean(K) * sum(v[:, t]) and
    columns whose sum(v) is small are ill-conditioned: the CPU fp32 path is itself 5e-6..5e-5 away from
    its fp64 twin.  check_parity handles that case.
    """
    for dtype in (torch.float32, torch.float64):
        X, C, sigma, v, w = inputs.make_config("C4", N=20_000, M=2_000, dtype=dtype)
        k = GaussianKernel(sigma)
        Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
        Xd, Cd, vd, wd = (a.double() for a in (X, C, v, w))
        budget = 2 * 2**30
        check_parity(k.mmv(Xg, Cg, vg), mmv_ref.fmmv_ref(X, C, v, sigma, max_cpu_mem=budget),
                     mmv_ref.fmmv_ref(Xd, Cd, vd, sigma, max_cpu_mem=budget), TOL[dtype])
        check_parity(k.dmmv(Xg, Cg, vg, wg), mmv_ref.fdmmv_ref(X, C, v, w, sigma, max_cpu_mem=budget),
                     mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma, max_cpu_mem=budget), TOL[dtype])


def test_per_dimension_sigma_fp32(dev):
    g = np.random.default_rng(5)
    X = torch.from_numpy(g.uniform(-1, 1, (4000, 9)).astype(np.float32))
    C = X[g.choice(4000, 500, replace=False)].clone()
    sigma = torch.from_numpy(g.uniform(0.5, 2.0, 9))
    v = torch.from_numpy(g.standard_normal((500, 1)).astype(np.float32))
    k = GaussianKernel(sigma)
    got = k.dmmv(X.to(dev), C.to(dev), v.to(dev), None)
    assert rel_err(got, mmv_ref.fdmmv_ref(X, C, v, None, sigma)) < 1e-5
    # per-dimension sigma == isotropic sigma=1 on pre-divided data (distance_kernel.py:151-152)
    k1 = GaussianKernel(1.0)
    s32 = sigma.float()
    got1 = k1.dmmv((X / s32).to(dev), (C / s32).to(dev), v.to(dev), None)
    assert rel_err(got, got1) < 1e-5


def test_sigma_changed_through_data_is_seen(dev):
    """mmv, dmmv and the kernel matrix after ``sigma.data.fill_``: the results of a kernel built with the new value."""
    X, C, v, w = (a.to(dev) for a in _rand(500, 7, 120, 2, torch.float32, seed=5))
    k = GaussianKernel(2.0)
    before = k.dmmv(X, C, v, w)
    k.sigma.data.fill_(3.5)
    fresh = GaussianKernel(3.5)
    assert torch.equal(k.dmmv(X, C, v, w), fresh.dmmv(X, C, v, w)) and not torch.equal(before, fresh.dmmv(X, C, v, w))
    assert torch.equal(k.mmv(X, C, v), fresh.mmv(X, C, v))
    assert torch.equal(k(X, C), fresh(X, C))


def test_wrong_sigma_length_raises(dev):
    X, C, v, w = _rand(20, 3, 5, 2, torch.float64, 1)
    k = GaussianKernel(torch.tensor([2.0, 2.0], dtype=torch.float64))
    with pytest.raises(RuntimeError):
        k.mmv(X.to(dev), C.to(dev), v.to(dev))


def test_host_data_round_trip(dev):
    """CPU-resident inputs are computed on the GPU and returned on the host, as the reference's
    CPU-data / GPU-compute mode does (fmmv.py:797-839)."""
    X, C, v, w = _rand(3000, 10, 400, 2, torch.float32, 3)
    k = GaussianKernel(2.5)
    got = k.mmv(X, C, v)
    assert got.device.type == "cpu"
    assert rel_err(got, mmv_ref.fmmv_ref(X, C, v, 2.5)) < 1e-5
    got = k.dmmv(X, C, v, w)
    assert got.device.type == "cpu"
    assert rel_err(got, mmv_ref.fdmmv_ref(X, C, v, w, 2.5)) < 1e-5


def test_row_blocking_under_memory_budget(dev):
    """A small max_gpu_mem forces several row blocks; results equal the unblocked ones
    (the reference's TestLargeComputations idea, tests/test_kernels.py:529-573)."""
    X, C, v, w = _rand(20000, 8, 300, 2, torch.float32, 4)
    k = GaussianKernel(2.0)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    full_m, full_d = k.mmv(Xg, Cg, vg), k.dmmv(Xg, Cg, vg, wg)
    opt = FalkonOptions(max_gpu_mem=400 * 2**10)
    blk_m, blk_d = k.mmv(Xg, Cg, vg, opt=opt), k.dmmv(Xg, Cg, vg, wg, opt=opt)
    assert rel_err(blk_m, full_m) < 1e-6
    assert rel_err(blk_d, full_d) < 1e-5
    with pytest.raises(MemoryError):
        k.mmv(Xg, Cg, vg, opt=FalkonOptions(max_gpu_mem=1024))


def test_determinism(dev):
    X, C, v, w = _rand(50000, 28, 2000, 1, torch.float32, 6)
    k = GaussianKernel(3.8)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    a = k.dmmv(Xg, Cg, vg, wg).clone()
    b = k.dmmv(Xg, Cg, vg, wg)
    assert torch.equal(a, b)


def test_config2_shape_reduced(dev):
    """Config 2 (d=28, sigma=3.8, fp32 dfmmv) at N=100k, M=5k against the blocked CPU oracle."""
    X, C, sigma, v, w = inputs.make_config("C2", N=100_000, M=5_000)
    k = GaussianKernel(sigma)
    got = k.dmmv(X.to(dev), C.to(dev), v.to(dev), w.to(dev))
    exp = mmv_ref.fdmmv_ref(X, C, v, w, sigma, max_cpu_mem=2 * 2**30)
    assert rel_err(got, exp) < 1e-5


def test_config1_full(dev):
    """Config 1 at full size: fp64 fmmv, N=20000 d=8 M=1000, sigma=2, tolerance 1e-11."""
    X, C, sigma, v, _ = inputs.make_config("C1")
    k = GaussianKernel(sigma)
    got = k.mmv(X.to(dev), C.to(dev), v.to(dev))
    exp = mmv_ref.fmmv_ref(X, C, v, sigma, max_cpu_mem=2 * 2**30)
    assert rel_err(got, exp) < 1e-11


# --------------------------------------------------------------------------------------------------
# explicit kernel matrix (the preconditioner's K(C, C)) through flk_gauss_fmm
# --------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("n,m,d", [(1, 1, 1), (33, 70, 3), (200, 131, 28), (129, 257, 9), (64, 300, 110), (50, 45, 784),
                                   (600, 700, 130), (257, 513, 65), (1, 300, 100), (300, 1, 97)])
def test_kernel_matrix_vs_oracle(dev, dtype, n, m, d):
    """kernel(X1, X2) against rbf_core (falkon/kernels/distance_kernel.py:140-159) restated on the CPU and
    against the fp64 difference form; per-dimension sigma; fp32 in both evaluation modes of
    falkon/mmv_ops/fmm.py:619-622."""
    from oracle import gaussian_ref
    X, C, _, _ = _rand(n, d, m, 1, dtype, seed=7 * n + d, scale=0.7)
    sigma = torch.from_numpy(np.random.default_rng(d).uniform(0.8, 1.6, d) * np.sqrt(d))
    k = GaussianKernel(sigma)
    exact = torch.from_numpy(brute.gaussian_brute(X, C, sigma))
    ref = gaussian_ref.rbf_core_ref(X, C, None, sigma)
    Xg, Cg = X.to(dev), C.to(dev)
    if dtype == torch.float64:
        got = k(Xg, Cg).cpu()
        assert got.dtype == dtype and got.shape == (n, m)
        assert float((got - ref).abs().max()) < 1e-12 and float((got - exact).abs().max()) < 1e-12
        return
    got64 = k(Xg, Cg, opt=FalkonOptions(no_single_kernel=True)).cpu()          # fp64 arithmetic, one rounding
    assert got64.dtype == torch.float32
    assert float((got64.double() - exact).abs().max()) <= 6.0e-8
    got32 = k(Xg, Cg, opt=FalkonOptions(no_single_kernel=False)).cpu()         # fp32 arithmetic
    err_ref = float((ref.double() - exact).abs().max())                       # what the CPU fp32 path itself loses
    assert float((got32.double() - exact).abs().max()) <= max(2e-6, 2 * err_ref)
    assert float((got32 - ref).norm() / ref.norm()) < 1e-5


def test_kernel_matrix_layouts_and_out(dev):
    """F-ordered inputs give an F-ordered result (falkon/mmv_ops/utils.py:124-155); ``out=`` is written in
    place in either order; host inputs come back on the host; a unit diagonal for X1 == X2."""
    from oracle import gaussian_ref
    X, C, _, _ = _rand(150, 12, 90, 1, torch.float64, seed=5)
    k = GaussianKernel(2.5)
    ref = gaussian_ref.rbf_core_ref(X, C, None, k.sigma)
    Xf = torch.empty_strided(X.shape, (1, X.shape[0]), dtype=X.dtype).copy_(X).to(dev)
    got_f = k(Xf, C.to(dev))
    assert got_f.stride(0) == 1 and float((got_f.cpu() - ref).abs().max()) < 1e-12
    for strides in ((90, 1), (1, 150)):
        out = torch.empty_strided((150, 90), strides, dtype=X.dtype, device=dev)
        res = k(X.to(dev), C.to(dev), out=out)
        assert res.data_ptr() == out.data_ptr() and float((out.cpu() - ref).abs().max()) < 1e-12
    host = k(X, C)
    assert host.device.type == "cpu" and float((host - ref).abs().max()) < 1e-12
    # forced row blocking of X1
    small = k(X.to(dev), C.to(dev), opt=FalkonOptions(max_gpu_mem=20_000))
    assert float((small.cpu() - ref).abs().max()) < 1e-12
    Kcc = k(C.to(dev), C.to(dev)).cpu()
    assert float((Kcc.diagonal() - 1).abs().max()) < 1e-12 and float((Kcc - Kcc.T).abs().max()) < 1e-13
    d = k(X.to(dev), X.to(dev), diag=True)
    assert d.shape == (150,) and float((d.cpu() - 1).abs().max()) < 1e-12


def test_kernel_matrix_layouts_large_d(dev):
    """The same for d > 64, where the kernel matrix comes from the LDS-tiled kernel: F-ordered result (operand roles
    swapped), ``out=`` in either order, row blocking, unit diagonal, other kernel functions, non-finite rows."""
    from oracle import gaussian_ref
    from falkon_amd import LaplacianKernel
    X, C, _, _ = _rand(700, 150, 390, 1, torch.float64, seed=5, scale=0.5)
    k = GaussianKernel(9.0)
    ref = gaussian_ref.rbf_core_ref(X, C, None, k.sigma)
    Xf = torch.empty_strided(X.shape, (1, X.shape[0]), dtype=X.dtype).copy_(X).to(dev)
    got_f = k(Xf, C.to(dev))
    assert got_f.stride(0) == 1 and float((got_f.cpu() - ref).abs().max()) < 1e-12
    for strides in ((390, 1), (1, 700)):
        out = torch.empty_strided((700, 390), strides, dtype=X.dtype, device=dev)
        res = k(X.to(dev), C.to(dev), out=out)
        assert res.data_ptr() == out.data_ptr() and float((out.cpu() - ref).abs().max()) < 1e-12
    small = k(X.to(dev), C.to(dev), opt=FalkonOptions(max_gpu_mem=3_000_000))
    assert float((small.cpu() - ref).abs().max()) < 1e-12
    Kcc = k(C.to(dev), C.to(dev)).cpu()
    assert float((Kcc.diagonal() - 1).abs().max()) < 1e-12 and float((Kcc - Kcc.T).abs().max()) < 1e-13
    lap = LaplacianKernel(9.0)(X.to(dev), C.to(dev)).cpu()
    assert float((lap - torch.from_numpy(brute.radial_brute(X, C, torch.tensor([9.0]), "laplacian"))).abs().max()) < 1e-9
    Xb = X.clone()
    Xb[5, 100] = float("nan")
    bad, clean = k(Xb.to(dev), C.to(dev)).cpu(), k(X.to(dev), C.to(dev)).cpu()
    assert torch.isnan(bad[5]).all() and torch.equal(bad[6:], clean[6:]) and torch.equal(bad[:5], clean[:5])


# --------------------------------------------------------------------------------------------------
# edge cases of the shapes and layouts
# --------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_degenerate_shapes(dev, dtype):
    """No centres (K v is an empty sum: zeros, K^T(.) has no rows), no data rows (K^T(K v + w) is an empty sum),
    a single row on either side, a 1-D v (reshaped to one column, falkon/kernels/kernel.py:92-95)."""
    k = GaussianKernel(1.5)
    X, C, v, w = _rand(70, 5, 9, 2, dtype, seed=3)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    none_c, none_v = Cg[:0], vg[:0]
    r = k.mmv(Xg, none_c, none_v)
    assert r.shape == (70, 2) and float(r.abs().max()) == 0.0
    r = k.dmmv(Xg, none_c, none_v, wg)
    assert r.shape == (0, 2)
    r = k.dmmv(Xg[:0], Cg, vg, wg[:0])
    assert r.shape == (9, 2) and float(r.abs().max()) == 0.0
    r = k.mmv(Xg[:0], Cg, vg)
    assert r.shape == (0, 2)
    for n, m in ((1, 9), (70, 1), (1, 1)):
        got = k.dmmv(Xg[:n], Cg[:m], vg[:m], wg[:n])
        assert rel_err(got, mmv_ref.fdmmv_ref(X[:n], C[:m], v[:m], w[:n], k.sigma)) < TOL[dtype]
    one_d = k.mmv(Xg, Cg, vg[:, 0].contiguous())
    assert one_d.shape == (70, 1)
    assert rel_err(one_d, mmv_ref.fmmv_ref(X, C, v[:, :1].contiguous(), k.sigma)) < TOL[dtype]


def test_strided_views_and_column_order(dev):
    """Row-sliced views (row stride larger than the row length) and F-ordered v / w / out are taken as they
    are (falkon/mmv_ops/utils.py:36-39 only asks for one unit stride); a view with no unit stride is refused."""
    X, C, v, w = _rand(300, 12, 80, 3, torch.float64, seed=8)
    k = GaussianKernel(2.0)
    big = torch.zeros(300, 20, dtype=torch.float64, device=dev)
    big[:, :12] = X.to(dev)
    Xv = big[:, :12]                                   # strides (20, 1)
    vf = torch.empty_strided((80, 3), (1, 80), dtype=torch.float64, device=dev).copy_(v)
    wf = torch.empty_strided((300, 3), (1, 300), dtype=torch.float64, device=dev).copy_(w)
    out = torch.empty_strided((80, 3), (1, 80), dtype=torch.float64, device=dev)
    got = k.dmmv(Xv, C.to(dev), vf, wf, out=out)
    assert got.data_ptr() == out.data_ptr()
    assert rel_err(got, mmv_ref.fdmmv_ref(X, C, v, w, k.sigma)) < 1e-11
    with pytest.raises(ValueError):
        k.mmv(big[::2, ::2][:, :6], C.to(dev)[:, :6].contiguous(), v.to(dev))


@pytest.mark.parametrize("t", [2, 20, 70])
def test_dmmv_replays_from_a_hip_graph(dev, t):
    """The library allocates nothing, clears memory with kernels and never synchronises, so a dmmv call can be
    captured into a HIP graph (e.g. a whole CG iteration).  Every replay, with the program's own eager work and
    synchronisations in between, must reproduce the eager result bit for bit.  Two right-hand sides run on the
    FMA kernel, 20 on the many-column kernel, 70 in two column chunks."""
    X, C, v, w = _rand(30_000, 28, 1_500, t, torch.float32, seed=21)
    k = GaussianKernel(3.8)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    out = torch.empty(1_500, t, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        k.dmmv(Xg, Cg, vg, wg, out=out)               # warm-up outside the capture (sigma upload, allocator)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        k.dmmv(Xg, Cg, vg, wg, out=out)
    g = np.random.default_rng(5)
    for _ in range(4):
        vg.copy_(torch.from_numpy(g.standard_normal((1_500, t)).astype(np.float32)))
        wg.copy_(torch.from_numpy(g.standard_normal((30_000, t)).astype(np.float32)))
        graph.replay()
        torch.cuda.synchronize()
        replayed = out.clone()
        eager = k.dmmv(Xg, Cg, vg, wg)
        torch.cuda.synchronize()
        assert torch.equal(replayed, eager)
    assert rel_err(eager, mmv_ref.fdmmv_ref(X, C, vg.cpu(), wg.cpu(), k.sigma)) < 1e-5


@pytest.mark.parametrize("order", ["C", "F"])
@pytest.mark.parametrize("pinned", [False, True])
def test_host_rows_streamed_in_chunks(dev, monkeypatch, order, pinned):
    """Host-resident X (and w) cut into chunks whose upload overlaps the kernels of the previous chunk: same
    results as with resident data, for pageable and pinned sources, either memory order, a ragged last chunk,
    w on either side, host and device outputs."""
    import sys
    drv = sys.modules["falkon_amd.mmv_ops.fmmv"]          # the package attribute of that name is the function
    monkeypatch.setattr(drv, "_STREAM_MIN_BYTES", 0)
    monkeypatch.setattr(drv, "_STREAM_PIECES", 5)
    X, C, v, w = _rand(10_007, 12, 300, 3, torch.float64, seed=44)
    if order == "F":
        X = torch.empty_strided(X.shape, (1, X.shape[0]), dtype=X.dtype).copy_(X)
        w = torch.empty_strided(w.shape, (1, w.shape[0]), dtype=w.dtype).copy_(w)
    if pinned:
        X, w = X.pin_memory(), w.pin_memory()
    k = GaussianKernel(2.5)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    exp_m, exp_d = k.mmv(Xg, Cg, vg), k.dmmv(Xg, Cg, vg, wg)
    got = k.mmv(X, Cg, vg)                                  # host rows, device everything else: result on the GPU
    assert got.device.type == "cuda" and rel_err(got, exp_m) < 1e-13
    got = k.mmv(X, C, v)                                    # everything on the host: result on the host
    assert got.device.type == "cpu" and rel_err(got, exp_m) < 1e-13
    out_dev = torch.empty(10_007, 3, dtype=torch.float64, device=dev)
    assert rel_err(k.mmv(X, Cg, vg, out=out_dev), exp_m) < 1e-13
    assert rel_err(k.dmmv(X, C, v, w), exp_d) < 1e-12       # X and w streamed together
    assert rel_err(k.dmmv(X, Cg, vg, wg), exp_d) < 1e-12    # only X streamed
    assert rel_err(k.dmmv(Xg, Cg, vg, w), exp_d) < 1e-12    # only w streamed
    assert rel_err(k.dmmv(X, Cg, vg, None), k.dmmv(Xg, Cg, vg, None)) < 1e-12


@pytest.mark.parametrize("d,t", [(3, 17), (3, 40), (9, 32), (15, 13), (16, 33), (17, 9), (28, 10), (28, 32), (31, 9),
                                 (33, 5), (40, 12), (63, 7), (64, 33), (9, 50), (28, 47), (40, 37), (64, 100), (31, 64),
                                 (3, 9), (9, 16), (64, 16), (9, 44), (28, 20), (64, 24), (16, 39), (40, 48), (57, 41)])
def test_many_right_hand_sides_small_d(dev, d, t):
    """More right-hand sides than the per-lane FMA kernels take in one pass: the register-resident kernel whose
    contraction runs on the matrix cores, in every form (8 to 64 columns per pass: groups of 32 columns on the
    32x32x2 step, a group of 16 on the four-block 16x16x1 step, a group of 8 on two 16-block 4x4x1 steps, and their
    combinations), folded and plain operands, four and two resident blocks per wave, a second pass beyond 64 columns; its 64-column form (two groups of 32 on one evaluation of K) with a second group
    that is partly filled, two and one resident blocks per wave, and a remainder pass after a full one."""
    n, m = 900 + d, 260 + t
    X, C, v, w = _rand(n, d, m, t, torch.float32, seed=d * 100 + t)
    k = GaussianKernel(0.9 * np.sqrt(d))
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    Xd, Cd, vd, wd = (a.double() for a in (X, C, v, w))
    check_parity(k.mmv(Xg, Cg, vg), mmv_ref.fmmv_ref(X, C, v, k.sigma), mmv_ref.fmmv_ref(Xd, Cd, vd, k.sigma), 1e-5)
    got = k.dmmv(Xg, Cg, vg, wg)
    check_parity(got, mmv_ref.fdmmv_ref(X, C, v, w, k.sigma), mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, k.sigma), 1e-5)
    assert torch.equal(got, k.dmmv(Xg, Cg, vg, wg))
    # column by column through the single-column kernels: the same numbers up to rounding
    cols = torch.cat([k.dmmv(Xg, Cg, vg[:, i:i + 1].contiguous(), wg[:, i:i + 1].contiguous()) for i in (0, t - 1)], 1)
    assert rel_err(got[:, [0, t - 1]], cols) < 5e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("t", [33, 64, 65, 128])
@pytest.mark.parametrize("d", [9, 28, 40, 100])
def test_many_right_hand_sides_stay_matrix_free(dev, dtype, d, t, monkeypatch):
    """33 to 128 right-hand sides on the default route: several passes of the product kernels, no stored block of K
    (the kernel-matrix entry point is never reached), parity with the CPU path, bit-identical repeats, and the same
    numbers as the single-column kernels on the first and last column.  The shapes of the reference's own timing of
    this case: falkon/benchmarks/timing_benchmarks/mmv_timings.py:48-127 (T = 10 .. 100)."""
    import importlib
    fmm_mod = importlib.import_module("falkon_amd.mmv_ops.fmm")

    def refuse(*a, **k):
        raise AssertionError("a kernel matrix was stored on the default route")
    monkeypatch.setattr(fmm_mod, "gauss_fmm_native", refuse)
    n, m = 700 + d, 257
    X, C, v, w = _rand(n, d, m, t, dtype, seed=d * 1000 + t, scale=0.7)
    sigma = 0.9 * np.sqrt(d)
    k = GaussianKernel(sigma)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    Xd, Cd, vd, wd = (a.double() for a in (X, C, v, w))
    tol = TOL[dtype]
    got_m, got_d = k.mmv(Xg, Cg, vg), k.dmmv(Xg, Cg, vg, wg)
    check_parity(got_m, mmv_ref.fmmv_ref(X, C, v, sigma), mmv_ref.fmmv_ref(Xd, Cd, vd, sigma), tol)
    check_parity(got_d, mmv_ref.fdmmv_ref(X, C, v, w, sigma), mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma), tol)
    assert torch.equal(got_d, k.dmmv(Xg, Cg, vg, wg))
    cols = torch.cat([k.dmmv(Xg, Cg, vg[:, i:i + 1].contiguous(), wg[:, i:i + 1].contiguous()) for i in (0, t - 1)], 1)
    assert rel_err(got_d[:, [0, t - 1]], cols) < (5e-6 if dtype == torch.float32 else 1e-12)


@pytest.mark.parametrize("d,t", [(28, 1), (28, 2), (12, 1), (40, 1), (64, 2)])
def test_output_norms_on_both_sides_of_the_factoring_guard(dev, d, t):
    """The fp32 Gaussian kernel for even d and one or two columns takes the output rows' half norms out of the
    exponent when they are small (at most 64 bits) and keeps them inside otherwise, wave by wave.  Rows drift away
    from the origin here so that one launch holds waves on either side of the guard, rows far beyond it (whose
    factored partial sums would overflow), and blocks that mix both: parity with the CPU path for both orientations."""
    n, m = 6000, 900
    g = np.random.default_rng(d + t)
    drift = np.linspace(0.0, 4.0, n)[:, None] * np.sign(g.standard_normal((1, d)))
    X = torch.from_numpy((g.standard_normal((n, d)) + drift).astype(np.float32))
    C = X[torch.from_numpy(np.sort(g.choice(n, m, replace=False)))].clone()
    v = torch.from_numpy(g.standard_normal((m, t)).astype(np.float32))
    w = torch.from_numpy(g.standard_normal((n, t)).astype(np.float32))
    sigma = 1.0
    half_bits = 0.5 * np.log2(np.e) * (X.double() ** 2).sum(1) / sigma ** 2
    assert float(half_bits.min()) < 40 and float(half_bits.max()) > 200          # both sides, and far beyond
    k = GaussianKernel(sigma)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    Xd, Cd, vd, wd = (a.double() for a in (X, C, v, w))
    check_parity(k.mmv(Xg, Cg, vg), mmv_ref.fmmv_ref(X, C, v, sigma), mmv_ref.fmmv_ref(Xd, Cd, vd, sigma), 1e-5)
    check_parity(k.dmmv(Xg, Cg, vg, wg), mmv_ref.fdmmv_ref(X, C, v, w, sigma), mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma), 1e-5)
    got = k.mmv(Cg, Xg, wg)
    assert bool(torch.isfinite(got).all())
    check_parity(got, mmv_ref.fmmv_ref(C, X, w, sigma), mmv_ref.fmmv_ref(Cd, Xd, wd, sigma), 1e-5)


@pytest.mark.parametrize("mode", ["f32", "f64", "bf16x3"])
@pytest.mark.parametrize("d,t", [(8, 1), (28, 2), (28, 20), (40, 6), (100, 1), (100, 10)])
def test_non_finite_rows_give_nan(dev, mode, d, t):
    """A NaN or an infinity in a data row must surface as NaN where the reference's result is NaN
    (falkon/kernels/distance_kernel.py:88-101,140-159 propagate it through the squared distance), although the
    kernels clamp the kernel value: rows of K(X1, X2) v whose X1 row is bad, everything when an X2 row is bad (every
    output sums over it), every entry of K^T(K v + w) either way; all other rows are what they are without the bad
    rows.  Every kernel family is visited (d, T: register-resident, 32-column, LDS-tiled, their bf16x3 twins)."""
    from falkon_amd import LaplacianKernel
    dtype = torch.float64 if mode == "f64" else torch.float32
    opt = FalkonOptions(bf16x3_cross_term=mode == "bf16x3")
    X, C, v, w = _rand(300, d, 170, t, dtype, seed=21)
    Xb = X.clone()
    Xb[3, d // 2] = float("nan")
    Xb[150, 0] = float("inf")
    Xb[299, d - 1] = float("-inf")
    bad = torch.zeros(300, dtype=torch.bool)
    bad[[3, 150, 299]] = True
    Cb = C.clone()
    Cb[7, 0] = float("nan")
    for K in (GaussianKernel, LaplacianKernel):
        k = K(float(d) ** 0.5, opt=opt)
        clean = k.mmv(X.to(dev), C.to(dev), v.to(dev)).cpu()
        got = k.mmv(Xb.to(dev), C.to(dev), v.to(dev)).cpu()
        assert torch.isnan(got[bad]).all()
        # (to rounding, not bit for bit: a wave of the fp32 Gaussian kernel that holds a bad output row keeps the
        # rows' half norms inside the exponent instead of factoring them out of the sums; measured against the size of
        # the summed terms, because at d = 100 with sigma = 10 the kernel matrix is nearly constant and the sums cancel)
        summed = k.mmv(X.to(dev), C.to(dev), v.abs().to(dev)).cpu()
        assert scaled_err(got[~bad], clean[~bad], summed[~bad]) < (5e-7 if dtype == torch.float32 else 1e-14)
        assert rel_err(got[~bad], clean[~bad]) < 5e-6
        assert torch.isnan(k.mmv(X.to(dev), Cb.to(dev), v.to(dev))).all()
        assert torch.isnan(k.dmmv(Xb.to(dev), C.to(dev), v.to(dev), w.to(dev))).all()
        assert torch.isnan(k.dmmv(X.to(dev), Cb.to(dev), v.to(dev), None)).all()
        assert not torch.isnan(k.dmmv(X.to(dev), C.to(dev), v.to(dev), w.to(dev))).any()
        if t == 1:
            full_clean = k(X.to(dev), C.to(dev)).cpu()
            full = k(Xb.to(dev), Cb.to(dev)).cpu()
            assert torch.isnan(full[bad]).all() and torch.isnan(full[:, 7]).all()
            keep = ~bad
            cols = torch.arange(170) != 7
            assert torch.equal(full[keep][:, cols], full_clean[keep][:, cols])
    # the CPU path says NaN in the same places for a NaN entry (an infinity gives it NaN or 0, depending on signs)
    if mode != "bf16x3" and t == 1:
        ref = mmv_ref.fmmv_ref(Xb, C, v, float(d) ** 0.5)
        assert torch.isnan(ref[3]).all() and not torch.isnan(ref[~bad]).any()


@pytest.mark.parametrize("d,t", [(1, 5), (3, 16), (9, 7), (12, 40), (28, 29), (32, 9), (33, 17), (50, 6), (64, 16), (61, 4),
                                 (64, 20), (12, 70), (28, 50), (40, 64), (64, 37), (28, 48), (9, 33)])
def test_many_right_hand_sides_small_d_fp64(dev, d, t):
    """More than four right-hand sides at d <= 64 in fp64: the 16-column kernel whose contraction runs on the matrix
    cores (one evaluation of K for 16 columns) and its 32- and 64-column forms (two / four groups of 16, the last one partly
    filled; half the resident blocks per wave with four groups),
    including more columns than one pass holds and a last pass that is narrow enough for the FMA kernel; 1e-11 against the CPU path, and the same numbers as column-by-column calls."""
    n, m = 900, 333
    X, C, v, w = _rand(n, d, m, t, torch.float64, seed=100 * d + t, scale=0.8)
    k = GaussianKernel(0.9 * np.sqrt(d) + 0.5)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    got_mmv = k.mmv(Xg, Cg, vg)
    got = k.dmmv(Xg, Cg, vg, wg)
    assert rel_err(got_mmv, mmv_ref.fmmv_ref(X, C, v, k.sigma)) < 1e-11
    assert rel_err(got, mmv_ref.fdmmv_ref(X, C, v, w, k.sigma)) < 1e-11
    assert rel_err(got_mmv, brute.mmv_brute(X, C, k.sigma, v)) < 5e-11
    assert torch.equal(got, k.dmmv(Xg, Cg, vg, wg))
    cols = torch.cat([k.dmmv(Xg, Cg, vg[:, i:i + 1].contiguous(), wg[:, i:i + 1].contiguous()) for i in (0, t - 1)], 1)
    assert rel_err(got[:, [0, t - 1]], cols) < 1e-12
    # F-ordered right-hand sides and output
    vf, of = vg.T.contiguous().T, torch.empty(t, n, dtype=torch.float64, device=dev).T
    assert k.mmv(Xg, Cg, vf, out=of).data_ptr() == of.data_ptr()
    assert torch.equal(of, got_mmv)


def test_torch_ops_entry_points(dev):
    """``torch.ops.falkon.kernel_fmmv / kernel_fdmmv`` give what the kernel objects give, bit for bit, in every
    arithmetic mode, and write ``out`` in place."""
    import falkon_amd.torch_ops  # noqa: F401
    from falkon_amd import LaplacianKernel
    for dtype, bf16x3 in ((torch.float32, False), (torch.float32, True), (torch.float64, False)):
        X, C, v, w = (a.to(dev) for a in _rand(500, 12, 130, 3, dtype, seed=5))
        sigma = torch.tensor([1.7], dtype=dtype, device=dev)
        opt = FalkonOptions(bf16x3_cross_term=bf16x3)
        out = torch.empty(500, 3, dtype=dtype, device=dev)
        assert torch.ops.falkon.kernel_fmmv(X, C, sigma, v, out, 0, bf16x3) is None
        assert torch.equal(out, GaussianKernel(1.7, opt=opt).mmv(X, C, v))
        out2 = torch.empty(130, 3, dtype=dtype, device=dev)
        torch.ops.falkon.kernel_fdmmv(X, C, sigma, v, w, out2, 1, bf16x3)
        assert torch.equal(out2, LaplacianKernel(1.7, opt=opt).dmmv(X, C, v, w))
        torch.ops.falkon.kernel_fdmmv(X, C, sigma, v, None, out2, 0, bf16x3)
        assert torch.equal(out2, GaussianKernel(1.7, opt=opt).dmmv(X, C, v, None))
    with pytest.raises(TypeError):
        torch.ops.falkon.kernel_fmmv(X, C.float(), sigma, v, out)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("n,m,d,t", [(1000, 300, 9, 1), (700, 130, 28, 3), (260, 200, 100, 2)])
def test_packed_entry_points(dev, dtype, n, m, d, t):
    """``flk_kernel_pack`` + ``flk_kernel_mmv_packed`` (pack X and C once, then K v + w and K^T u as two products on the
    packed operands) give what ``dmmv`` gives, and the packed operand itself is the scaled data, block by block, with
    the half squared norms behind it (the reference's ``square_norm``, falkon/c_ext/ops/cpu/cpu_square_norm.cpp:14-60,
    pinned there against ``torch.norm``: falkon/tests/test_matrix_ops.py:72-108)."""
    from falkon_amd import _backend
    lib = _backend.load()
    code = _backend.FLK_F32 if dtype == torch.float32 else _backend.FLK_F64
    blk = 32 if dtype == torch.float32 else 16
    X, C, v, w = (a.to(dev) for a in _rand(n, d, m, t, dtype, seed=n + d))
    sigma = torch.linspace(1.5, 3.0, d, dtype=dtype, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    packed = {}
    for name, A in (("X", X), ("C", C)):
        nbytes = lib.flk_gauss_packed_bytes(A.shape[0], d, code)
        buf = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        rc = lib.flk_gauss_pack(A.data_ptr(), A.shape[0], d, A.stride(0), A.stride(1), sigma.data_ptr(), d, code,
                                buf.data_ptr(), nbytes, stream)
        _backend.raise_for_status(rc, "flk_gauss_pack")
        packed[name] = buf
    # layout: [block][feature][row] (fp64 rows permuted inside a block), then -1/2 |x~|^2, x~ = sqrt(log2 e) x / sigma
    # (fp64: x~ = sqrt(2048 log2 e) x / sigma: the Gaussian's exponent is carried times 2048 in double precision)
    if d <= 64:
        dpad = (d + 1) // 2 * 2 if dtype == torch.float32 else (d + 3) // 4 * 4
    else:
        dpad = (d + 15) // 16 * 16 if dtype == torch.float32 else (d + 31) // 32 * 32
    nblk = (n + blk - 1) // blk
    flat = packed["X"].view(dtype)
    data = flat[:nblk * dpad * blk].view(nblk, dpad, blk)
    scaled = (X.double() * np.sqrt(np.log2(np.e) * (1.0 if dtype == torch.float32 else 2048.0)) / sigma.double())
    pos = torch.arange(blk) if dtype == torch.float32 else torch.tensor([4 * (r % 4) + r // 4 for r in range(blk)])
    rows = torch.arange(n)
    got_rows = data[rows // blk, :d, pos[rows % blk]]
    assert rel_err(got_rows, scaled.cpu()) < (1e-6 if dtype == torch.float32 else 1e-15)
    off = (nblk * dpad * blk * flat.element_size() + 255) // 256 * 256 // flat.element_size()
    half_norms = flat[off:off + n]
    want = -0.5 * (scaled * scaled).sum(1)
    assert rel_err(half_norms.reshape(-1, 1), want.reshape(-1, 1).cpu()) < (1e-6 if dtype == torch.float32 else 1e-15)
    # two products on the packed operands
    u = torch.empty(n, t, dtype=dtype, device=dev)
    out = torch.empty(m, t, dtype=dtype, device=dev)
    for (pa, na, pb, nb, vec, add, res) in ((packed["C"], m, packed["X"], n, v, w, u), (packed["X"], n, packed["C"], m, u, None, out)):
        ws_bytes = lib.flk_gauss_mmv_packed_workspace_bytes(na, nb, d, t, code)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
        rc = lib.flk_gauss_mmv_packed(pa.data_ptr(), na, pb.data_ptr(), nb, d, vec.data_ptr(), vec.stride(0), vec.stride(1), t,
                                      add.data_ptr() if add is not None else None,
                                      add.stride(0) if add is not None else 0, add.stride(1) if add is not None else 0,
                                      res.data_ptr(), res.stride(0), res.stride(1), code, ws.data_ptr(), ws_bytes, stream)
        _backend.raise_for_status(rc, "flk_gauss_mmv_packed")
    k = GaussianKernel(sigma)
    assert torch.equal(u, k.mmv(X, C, v) + w) or rel_err(u, k.mmv(X, C, v) + w) < (1e-6 if dtype == torch.float32 else 1e-14)
    assert torch.equal(out, k.dmmv(X, C, v, w))
    assert rel_err(out, mmv_ref.fdmmv_ref(X.cpu(), C.cpu(), v.cpu(), w.cpu(), sigma.cpu())) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("n,m,d,t", [(700, 300, 100, 70), (300, 520, 784, 40), (2000, 333, 28, 130), (900, 257, 40, 100),
                                     (500, 129, 9, 200)])
def test_many_right_hand_sides_through_stored_blocks(dev, dtype, n, m, d, t, monkeypatch):
    """Opt-in ``many_rhs_stored_blocks``: with enough right-hand sides the drivers store blocks of K and contract them
    with library GEMMs (the reference's own scheme, falkon/mmv_ops/fmmv.py:358-396,740-762): same tolerances against
    the CPU path, agreement with the matrix-free default, several blocks (block size forced down), strided
    operands, ``out=``, host data, ``w = None``."""
    import importlib
    drv = importlib.import_module("falkon_amd.mmv_ops.fmmv")
    stored = FalkonOptions(many_rhs_stored_blocks=True)
    assert drv._explicit_blocks_pay(d, t, dtype, stored, two_products=True)
    assert drv._explicit_blocks_pay(d, t, dtype, stored) or (dtype == torch.float64 and d == 784)
    X, C, v, w = _rand(n, d, m, t, dtype, seed=n + t, scale=0.6)
    sigma = 0.8 * np.sqrt(d)
    k, k_free = GaussianKernel(sigma, opt=stored), GaussianKernel(sigma)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    Xd, Cd, vd, wd = (a.double() for a in (X, C, v, w))
    tol = TOL[dtype]
    got_mmv, got_dmmv = k.mmv(Xg, Cg, vg), k.dmmv(Xg, Cg, vg, wg)
    check_parity(got_mmv, mmv_ref.fmmv_ref(X, C, v, sigma), mmv_ref.fmmv_ref(Xd, Cd, vd, sigma), tol)
    check_parity(got_dmmv, mmv_ref.fdmmv_ref(X, C, v, w, sigma), mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma), tol)
    assert rel_err(got_mmv, k_free.mmv(Xg, Cg, vg)) < tol and rel_err(got_dmmv, k_free.dmmv(Xg, Cg, vg, wg)) < tol
    check_parity(k.dmmv(Xg, Cg, vg, None), mmv_ref.fdmmv_ref(X, C, v, None, sigma),
                 mmv_ref.fdmmv_ref(Xd, Cd, vd, None, sigma), tol)
    # several stored blocks, F-ordered operands, out=, host data
    monkeypatch.setattr(drv, "_EXPLICIT_BLOCK_BYTES", 64 * m * X.element_size())
    f = lambda a: a.T.contiguous().T                                                      # noqa: E731
    out = torch.empty(t, n, dtype=dtype, device=dev).T
    assert k.mmv(f(Xg), f(Cg), f(vg), out=out).data_ptr() == out.data_ptr()
    # (other layouts make the library GEMMs sum in another order: compare with the CPU path again, not bit for bit)
    ref_mmv = (mmv_ref.fmmv_ref(X, C, v, sigma), mmv_ref.fmmv_ref(Xd, Cd, vd, sigma))
    ref_dmmv = (mmv_ref.fdmmv_ref(X, C, v, w, sigma), mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma))
    check_parity(out, *ref_mmv, tol)
    check_parity(k.dmmv(f(Xg), Cg, vg, f(wg)), *ref_dmmv, tol)
    host = k.dmmv(X, C, v, w)
    assert host.device.type == "cpu"
    check_parity(host, *ref_dmmv, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_dmmv_stored_blocks_option(dev, dtype):
    """``FalkonOptions(dmmv_stored_blocks=True)``: K^T(K v + w) beyond 64 features through stored blocks of K for any
    number of right-hand sides; same tolerances; at 64 features or fewer the option changes nothing."""
    opt = FalkonOptions(dmmv_stored_blocks=True)
    for (n, m, d, t) in ((600, 257, 100, 1), (513, 300, 784, 10)):
        X, C, v, w = _rand(n, d, m, t, dtype, seed=n + d, scale=0.5)
        sigma = 0.6 * np.sqrt(d)
        Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
        got = GaussianKernel(sigma, opt=opt).dmmv(Xg, Cg, vg, wg)
        Xd, Cd, vd, wd = (a.double() for a in (X, C, v, w))
        check_parity(got, mmv_ref.fdmmv_ref(X, C, v, w, sigma), mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma), TOL[dtype])
        assert rel_err(got, GaussianKernel(sigma).dmmv(Xg, Cg, vg, wg)) < TOL[dtype]
    X, C, v, w = (a.to(dev) for a in _rand(500, 28, 200, 2, dtype, seed=1))
    assert torch.equal(GaussianKernel(3.0, opt=opt).dmmv(X, C, v, w), GaussianKernel(3.0).dmmv(X, C, v, w))


@pytest.mark.parametrize("d", [9, 28])
@pytest.mark.parametrize("blocks", [1, 5, 37])
def test_odd_reduction_blocks_single_column_and_coincident_points(dev, d, blocks):
    """One right-hand side in fp32 with an odd number of 32-row blocks on the reduction side (the single-column loop
    walks two blocks per trip and handles the last block of an odd chunk a second time against zeros), the centres
    being rows of X, so that kernel values of exactly 1 occur (the reference clamps the squared distance at 1e-20,
    falkon/kernels/distance_kernel.py:100, i.e. K <= 1): parity with the CPU path, K <= 1 to rounding, and an
    infinite entry of v in the repeated block gives infinities, not NaN."""
    m = 32 * blocks
    X, _, v, w = _rand(1500, d, m, 1, torch.float32, seed=40 + blocks)
    C = X[:m].clone()
    sigma = float(d) ** 0.5
    k = GaussianKernel(sigma)
    Xg, Cg, vg, wg = X.to(dev), C.to(dev), v.to(dev), w.to(dev)
    Xd, Cd, vd, wd = X.double(), C.double(), v.double(), w.double()
    check_parity(k.mmv(Xg, Cg, vg), mmv_ref.fmmv_ref(X, C, v, sigma), mmv_ref.fmmv_ref(Xd, Cd, vd, sigma), 1e-5)
    check_parity(k.dmmv(Xg, Cg, vg, wg), mmv_ref.fdmmv_ref(X, C, v, w, sigma), mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma), 1e-5)
    # a column of K through a unit vector: the entry of the coincident pair is 1 (to rounding on the factored path)
    for j in (0, m - 1):
        unit = torch.zeros(m, 1)
        unit[j] = 1.0
        col = k.mmv(Xg, Cg, unit.to(dev)).cpu()
        assert abs(float(col[j]) - 1.0) <= 2e-6 and float(col.max()) <= 1.0 + 2e-6
        want = torch.from_numpy(brute.gaussian_brute(X, C[j:j + 1], sigma))
        assert float((col.double() - want).abs().max()) < 2e-6
    # an infinite right-hand side entry in the last block
    vi = v.clone()
    vi[m - 1] = float("inf")
    got = k.mmv(Xg, Cg, vi.to(dev)).cpu()
    ref = mmv_ref.fmmv_ref(X, C, vi, sigma)
    assert torch.isinf(ref).all() and torch.equal(torch.isinf(got), torch.isinf(ref)) and not torch.isnan(got).any()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("name,n,m,d,t", [("gaussian", 3000, 700, 28, 1), ("gaussian", 1500, 333, 9, 3), ("laplacian", 900, 257, 40, 2),
                                           ("2.5-matern", 700, 300, 100, 5), ("gaussian", 640, 129, 300, 1), ("1.5-matern", 33, 1, 3, 70)])
def test_products_on_operands_packed_once(dev, dtype, name, n, m, d, t):
    """``PackedProducts`` (X and the centres packed once, what a GPU fit's solver uses for its products) gives bit for
    bit what ``mmv`` / ``dmmv`` give, for strided operands and per-dimension lengthscales too, and does not apply where
    the one-shot calls have work it does not do (host operands, gradients, the bf16x3 mode, a tiny memory budget)."""
    from falkon_amd import FalkonOptions, LaplacianKernel, MaternKernel
    from falkon_amd.mmv_ops.fmmv import PackedProducts
    X, C, v, w = (a.to(dev) for a in _rand(n, d, m, t, dtype, seed=n + d + t))
    sigma = torch.linspace(1.5, 3.0, d, dtype=torch.float64) * (d ** 0.5) / 3
    k = {"gaussian": lambda: GaussianKernel(sigma), "laplacian": lambda: LaplacianKernel(sigma),
         "1.5-matern": lambda: MaternKernel(sigma, 1.5), "2.5-matern": lambda: MaternKernel(sigma, 2.5)}[name]()
    Xf = X.T.contiguous().T                                      # an F-ordered X, a v with a row stride
    vs = torch.zeros(m, t + 2, dtype=dtype, device=dev)[:, 1:1 + t]
    vs.copy_(v)
    pp = PackedProducts.create(Xf, C, k, columns=t)
    assert pp is not None
    assert torch.equal(pp.mmv(vs), k.mmv(X, C, v))
    assert torch.equal(pp.mmv(v, w), k.mmv(X, C, v) + w) or rel_err(pp.mmv(v, w), k.mmv(X, C, v) + w) < TOL[dtype]
    u = torch.randn(n, t, dtype=dtype, device=dev)
    assert torch.equal(pp.mmv_t(u), k.mmv(C, X, u))
    assert torch.equal(pp.dmmv(v, w), k.dmmv(X, C, v, w))
    assert torch.equal(pp.dmmv(v), k.dmmv(X, C, v, None))
    out = torch.empty(m, t, dtype=dtype, device=dev)
    assert pp.dmmv(v, w, out=out) is out and torch.equal(out, k.dmmv(X, C, v, w))
    with pytest.raises(ValueError):
        pp.mmv(v[:-1] if m > 1 else v.to(torch.float64 if dtype == torch.float32 else torch.float32))
    assert PackedProducts.create(X.cpu(), C, k) is None
    assert PackedProducts.create(X.clone().requires_grad_(True), C, k) is None
    assert PackedProducts.create(X, C, k, FalkonOptions(bf16x3_cross_term=True)) is None or dtype == torch.float64
    assert PackedProducts.create(X, C, k, FalkonOptions(max_gpu_mem=1000.0)) is None
