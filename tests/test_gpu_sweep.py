"""Many right-hand sides beyond 64 features, and a fixed-seed sweep over shapes, kernels, layouts and dtypes.

The shapes of the first test come from a case a random sweep once reported (Matern 3/2, fp32, 845 x 1280, d = 200,
70 right-hand sides, dmmv 2.0e-5 from the fp64 CPU path).  With d = 200 and the lengthscale used there every kernel
value lies within a few percent of 0.24, so K is close to a constant matrix and a column of the result is close to
(sum of v) * const: columns whose right-hand side sums to nearly nothing cancel a thousandfold (column norms from
1e2 to 2e5 in one call).  The reference's CPU path in fp32 is 2e-6 ... 2.3e-5 from its own fp64 twin on the worst
column of such calls, so the distance of two fp32 results is governed by the cancellation, not by either summation.
Two bars are applied: ``check_parity`` (1e-5 against the CPU path in the same dtype, with its bounded relaxation where
that path has itself drifted from fp64) and the error against the scale of the summed terms, which does not know about
cancellation and must stay at fp32 rounding level (falkon/mmv_ops/fmmv.py:740-762 is the summation being matched,
falkon/kernels/distance_kernel.py:225-269 the kernel functions).
"""
import numpy as np
import pytest
import torch

from falkon_amd import GaussianKernel, LaplacianKernel, MaternKernel
from oracle import mmv_ref
from conftest import check_parity, rel_err, scaled_err

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.float64: 1e-11}
# error against the scale of the terms: a few units of the dtype's rounding error
SCALED = {torch.float32: 1.5e-6, torch.float64: 5e-15}
NAMES = ["gaussian", "laplacian", "1.5-matern", "2.5-matern"]


def _kernel(name, sigma):
    return {"gaussian": lambda: GaussianKernel(sigma), "laplacian": lambda: LaplacianKernel(sigma),
            "1.5-matern": lambda: MaternKernel(sigma, 1.5), "2.5-matern": lambda: MaternKernel(sigma, 2.5)}[name]()


def _case(n, m, d, t, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(n, d, dtype=dtype, generator=g) * 0.7
    C = torch.randn(m, d, dtype=dtype, generator=g) * 0.7
    v = torch.randn(m, t, dtype=dtype, generator=g)
    w = torch.randn(n, t, dtype=dtype, generator=g)
    return X, C, v, w


def _check(dev, name, X, C, v, w, sigma, f_order_x=False, f_order_v=False):
    dtype = X.dtype
    k = _kernel(name, sigma)
    Xg, Cg, vg = X.to(dev), C.to(dev), v.to(dev)
    wg = None if w is None else w.to(dev)
    if f_order_x:
        Xg = Xg.T.contiguous().T
    if f_order_v:
        vg = vg.T.contiguous().T
    got_m = k.mmv(Xg, Cg, vg).cpu()
    got_d = k.dmmv(Xg, Cg, vg, wg).cpu()
    Xd, Cd, vd = X.double(), C.double(), v.double()
    wd = None if w is None else w.double()
    ref_m64 = mmv_ref.fmmv_ref(Xd, Cd, vd, sigma, kernel_name=name)
    ref_d64 = mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma, kernel_name=name)
    if dtype == torch.float64:
        ref_m, ref_d = ref_m64, ref_d64
    else:
        ref_m = mmv_ref.fmmv_ref(X, C, v, sigma, kernel_name=name)
        ref_d = mmv_ref.fdmmv_ref(X, C, v, w, sigma, kernel_name=name)
    check_parity(got_m, ref_m, ref_m64, TOL[dtype])
    check_parity(got_d, ref_d, ref_d64, TOL[dtype])
    # the same products with every term replaced by its absolute value (K is positive)
    abs_m = mmv_ref.fmmv_ref(Xd, Cd, vd.abs(), sigma, kernel_name=name)
    abs_d = mmv_ref.fdmmv_ref(Xd, Cd, vd.abs(), None if wd is None else wd.abs(), sigma, kernel_name=name)
    s_m, s_d = scaled_err(got_m, ref_m64, abs_m), scaled_err(got_d, ref_d64, abs_d)
    assert s_m < SCALED[dtype] and s_d < SCALED[dtype], (s_m, s_d)
    return {"gpu_vs_f64": (rel_err(got_m, ref_m64), rel_err(got_d, ref_d64)),
            "cpu_same_dtype_vs_f64": (rel_err(ref_m, ref_m64), rel_err(ref_d, ref_d64)),
            "gpu_vs_scale_of_terms": (s_m, s_d)}


@pytest.mark.parametrize("t", [65, 70, 129])
@pytest.mark.parametrize("d", [100, 200])
@pytest.mark.parametrize("name", ["gaussian", "1.5-matern", "2.5-matern"])
def test_many_columns_beyond_64_features(dev, name, d, t):
    """The LDS-tiled kernel's passes of 64 columns followed by a short pass, on nearly constant kernel matrices."""
    sigma = float(0.6 * np.sqrt(d) + 0.4)
    X, C, v, w = _case(845, 1280, d, t, torch.float32, seed=4 + d + t)
    figures = _check(dev, name, X, C, v, w, sigma)
    print(f"[many columns] {name} d={d} t={t} (mmv, dmmv) " + " ".join(f"{k}=({a:.2e}, {b:.2e})" for k, (a, b) in figures.items()))


def test_many_columns_beyond_64_features_fp64(dev):
    sigma = float(0.6 * np.sqrt(200) + 0.4)
    X, C, v, w = _case(845, 1280, 200, 70, torch.float64, seed=11)
    _check(dev, "1.5-matern", X, C, v, w, sigma)


FEATURES = [1, 2, 3, 5, 8, 9, 13, 15, 16, 17, 24, 25, 28, 29, 31, 32, 33, 40, 47, 49, 50, 52, 53, 56, 57, 61, 63, 64, 65,
            70, 97, 128, 200, 300]
COLUMNS = [1, 2, 3, 4, 5, 7, 8, 9, 12, 13, 16, 17, 20, 31, 32, 33, 36, 37, 40, 45, 48, 49, 63, 64, 65, 70, 100, 129]


def test_fixed_seed_shape_sweep(dev):
    """300 shapes drawn from a fixed seed: every kernel function, both dtypes, both layouts of X and v, with and
    without w, feature and column counts on both sides of every dispatch boundary, sides down to a single row.
    Each case is named on stdout before it runs, so that a run that ends early names the case it ended in."""
    rng = np.random.default_rng(20240531)
    for it in range(300):
        dtype = torch.float32 if rng.random() < 0.5 else torch.float64
        d = int(rng.choice(FEATURES))
        t = int(rng.choice(COLUMNS))
        n = int(rng.integers(1, 2500))
        m = int(rng.integers(1, 1500))
        if rng.random() < 0.1:
            n = int(rng.integers(1, 40))
        if rng.random() < 0.1:
            m = int(rng.integers(1, 40))
        seed = int(rng.integers(1 << 30))
        fx, fv = bool(rng.random() < 0.3), bool(rng.random() < 0.3)
        name = NAMES[int(rng.integers(4))]
        use_w = bool(rng.random() < 0.7)
        sigma = float(0.6 * np.sqrt(d) + 0.4)
        print(f"[sweep {it}] {name} {dtype} n={n} m={m} d={d} t={t} seed={seed} Fx={fx} Fv={fv} w={use_w}", flush=True)
        X, C, v, w = _case(n, m, d, t, dtype, seed)
        _check(dev, name, X, C, v, w if use_w else None, sigma, fx, fv)
