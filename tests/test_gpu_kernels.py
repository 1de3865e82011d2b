"""GPU parity of the Laplacian and Matern kernels (through the C ABI) with the CPU oracle's restatement of the
reference cores (falkon/kernels/distance_kernel.py:182-269) and with the closed forms in fp64 difference form.

Tolerances as for the Gaussian: 1e-5 (fp32) / 1e-11 (fp64), relative, norm-wise per output column.  These
kernels take the square root of a squared distance that both the reference and this build form through the
expanded norm: where two points coincide, that square root turns rounding noise of size eps |x|^2 into an error
of size sqrt(eps) |x|, in the reference's CPU path as much as here, and two such results cannot be expected to
agree with each other; there the GPU result is required to be as close to the closed form as the CPU path is.
"""
import numpy as np
import pytest
import torch

from falkon_amd import FalkonOptions, GaussianKernel, LaplacianKernel, MaternKernel
from oracle import brute, gaussian_ref, mmv_ref
from conftest import check_parity, rel_err

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.float64: 1e-11}
KERNELS = {
    "laplacian": lambda s: LaplacianKernel(s),
    "0.5-matern": lambda s: MaternKernel(s, 0.5),
    "1.5-matern": lambda s: MaternKernel(s, 1.5),
    "2.5-matern": lambda s: MaternKernel(s, 2.5),
    "inf-matern": lambda s: MaternKernel(s, float("inf")),
}


def _data(n, m, d, t, dtype, seed):
    g = np.random.default_rng(seed)
    np_dt = np.float32 if dtype == torch.float32 else np.float64
    mk = lambda *shape: torch.from_numpy(g.standard_normal(shape).astype(np_dt))     # noqa: E731
    return mk(n, d) * 0.7, mk(m, d) * 0.7, mk(m, t), mk(n, t)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("name", sorted(KERNELS))
@pytest.mark.parametrize("n,m,d,t", [
    (200, 131, 28, 1), (513, 300, 9, 3), (257, 100, 64, 1),      # register-resident kernels, folded (d = 9) and plain
    (150, 260, 16, 4), (140, 200, 52, 4),      # column counts where the fp64 kernels differ by kernel function
    (300, 257, 65, 2), (129, 64, 200, 10), (64, 300, 784, 5),    # LDS-tiled kernel, both epilogues
    (600, 1090, 44, 1), (500, 777, 89, 1), (400, 650, 121, 1), (350, 420, 77, 3),   # beyond 32 features (fp32): one column on four resident blocks up to 96 features, three up to 128; few columns on two
])
def test_products_vs_oracle(dev, dtype, name, n, m, d, t):
    X, C, v, w = _data(n, m, d, t, dtype, seed=n + 3 * d)
    sigma = torch.tensor([0.8 * np.sqrt(d)], dtype=torch.float64)
    k = KERNELS[name](sigma)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    Xd, Cd, vd, wd = (a.double() for a in (X, C, v, w))
    check_parity(k.mmv(Xg, Cg, vg), mmv_ref.fmmv_ref(X, C, v, sigma, kernel_name=name),
                 mmv_ref.fmmv_ref(Xd, Cd, vd, sigma, kernel_name=name), TOL[dtype])
    check_parity(k.dmmv(Xg, Cg, vg, wg), mmv_ref.fdmmv_ref(X, C, v, w, sigma, kernel_name=name),
                 mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma, kernel_name=name), TOL[dtype])
    K = brute.radial_brute(X, C, sigma, name)
    assert rel_err(k.mmv(Xg, Cg, vg), K @ vd.numpy()) < 5 * TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("name", ["laplacian", "1.5-matern", "2.5-matern"])
def test_kernel_matrix_and_coincident_points(dev, dtype, name):
    """kernel(X1, X2) in every arithmetic mode, per-dimension lengthscales; then centres that are data points
    (zero distances), where the error against the closed form is bounded by the CPU path's own."""
    X, C, v, _ = _data(220, 90, 12, 2, dtype, seed=31)
    sigma = torch.from_numpy(np.random.default_rng(1).uniform(2.0, 4.0, 12))
    k = KERNELS[name](sigma)
    exact = torch.from_numpy(brute.radial_brute(X, C, sigma, name))
    ref = gaussian_ref.core_ref_for(name)(X, C, None, sigma)
    err_ref = float((ref.double() - exact).abs().max())
    Xg, Cg = X.to(dev), C.to(dev)
    if dtype == torch.float64:
        assert float((k(Xg, Cg).cpu() - exact).abs().max()) < 1e-11
    else:
        once_rounded = k(Xg, Cg, opt=FalkonOptions(no_single_kernel=True)).cpu()       # fp64 arithmetic
        assert once_rounded.dtype == torch.float32 and float((once_rounded.double() - exact).abs().max()) <= 6.0e-8
        single = k(Xg, Cg, opt=FalkonOptions(no_single_kernel=False)).cpu()
        assert float((single.double() - exact).abs().max()) <= max(2e-6, 2 * err_ref)
    # coincident points
    Cx = X[:90].contiguous()
    exact = torch.from_numpy(brute.radial_brute(X, Cx, sigma, name))
    ref = gaussian_ref.core_ref_for(name)(X, Cx, None, sigma)
    err_ref = float((ref.double() - exact).abs().max())
    got = k(Xg, Cx.to(dev), opt=FalkonOptions(no_single_kernel=False)).cpu()
    floor = 1e-6 if dtype == torch.float32 else 1e-12
    assert float((got.double() - exact).abs().max()) <= 4 * err_ref + floor
    u_exact = exact.numpy() @ v.double().numpy()
    e_gpu = rel_err(k.mmv(Xg, Cx.to(dev), v.to(dev)), u_exact)
    e_cpu = rel_err(mmv_ref.fmmv_ref(X, Cx, v, sigma, kernel_name=name), u_exact)
    assert e_gpu <= 4 * e_cpu + TOL[dtype]


def test_limits_and_equivalences(dev):
    """Matern 1/2 is the Laplacian and Matern inf the Gaussian, bit for bit; a huge lengthscale gives K = 1."""
    X, C, v, w = _data(400, 150, 10, 2, torch.float32, seed=2)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    assert torch.equal(MaternKernel(2.0, 0.5).dmmv(Xg, Cg, vg, wg), LaplacianKernel(2.0).dmmv(Xg, Cg, vg, wg))
    assert torch.equal(MaternKernel(2.0, float("inf")).dmmv(Xg, Cg, vg, wg), GaussianKernel(2.0).dmmv(Xg, Cg, vg, wg))
    for k in (LaplacianKernel(1e9), MaternKernel(1e9, 1.5), MaternKernel(1e9, 2.5)):
        flat = k.mmv(Xg, Cg, vg)
        sums = vg.double().sum(0, keepdim=True)
        assert float(((flat.double() - sums).abs().max(0).values / vg.double().abs().sum(0)).max()) < 1e-5


def test_config2_shape_reduced_other_kernels(dev):
    """Config 2's shape (d = 28, sigma = 3.8, fp32 dfmmv) at N = 100k, M = 5k, centres drawn from the data."""
    from oracle import inputs
    X, C, sigma, v, w = inputs.make_config("C2", N=100_000, M=5_000)
    Xd, Cd, vd, wd = (a.double() for a in (X, C, v, w))
    for name in ("laplacian", "2.5-matern"):
        k = KERNELS[name](sigma)
        got = k.dmmv(X.to(dev), C.to(dev), v.to(dev), w.to(dev))
        check_parity(got, mmv_ref.fdmmv_ref(X, C, v, w, sigma, kernel_name=name, max_cpu_mem=2 * 2**30),
                     mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma, kernel_name=name, max_cpu_mem=4 * 2**30), 1e-5)


@pytest.mark.parametrize("d", [1, 80])
def test_fp64_exponential_accuracy(dev, d):
    """The fp64 kernels evaluate 2^e with a routine of their own (the hardware has none): check it against numpy's exp
    on a grid where the argument is exact (x = k/64 in the first feature, centre 0, sigma 1: K = exp(-k^2/8192)), from
    K = 1 through the subnormal range down to 0, in the kernel matrix and in both product kernels (d = 1 and 80)."""
    k = np.arange(0, 64 * 40, dtype=np.float64)         # x up to 40: argument down to -800; exp is 0 below -745.2
    arg = -(k * k) / 8192
    want = np.exp(arg)
    X = torch.zeros(k.size, d, dtype=torch.float64)
    X[:, 0] = torch.from_numpy(k / 64)
    C = torch.zeros(1, d, dtype=torch.float64)
    kern = GaussianKernel(1.0)
    # the argument reaches the exponential with a relative rounding error of a few eps: allow eps * |argument| on top
    tol = 1e-15 * (1 + np.abs(arg)) * want + 1e-323
    for got in (kern(X.to(dev), C.to(dev))[:, 0], kern.mmv(X.to(dev), C.to(dev), torch.ones(1, 1, dtype=torch.float64, device=dev))[:, 0]):
        got = got.cpu().numpy()
        worst = np.max((np.abs(got - want) - tol) / np.maximum(want, 1e-300))
        assert np.all(np.abs(got - want) <= tol), f"worst excess {worst:.3e}"
        assert got[0] == 1.0 and np.all(got[arg < -760] == 0) and np.all(got[arg > -700] > 0)
    # the other kernel functions share the routine: Laplacian exp(-x); at x = 0 the reference's clamp of the squared
    # distance at 1e-20 makes it exp(-1e-10) (falkon/kernels/distance_kernel.py:100)
    lap = LaplacianKernel(1.0)(X.to(dev), C.to(dev))[:, 0].cpu().numpy()
    want_l = np.exp(-np.maximum(k / 64, 1e-10))
    assert np.all(np.abs(lap - want_l) <= 1e-15 * (1 + k / 64) * want_l)
