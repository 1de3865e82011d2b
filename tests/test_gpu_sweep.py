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


def _laid_out(t, mode):
    """t in one of four layouts: C order, F order, a column band of a wider row-major matrix (row stride beyond the
    columns), a row band of a taller column-major matrix (column stride beyond the rows)."""
    if mode == 0 or t.shape[1] == 0:
        return t.contiguous()
    if mode == 1:
        return t.T.contiguous().T
    if mode == 2:
        big = torch.zeros(t.shape[0], t.shape[1] + 3, dtype=t.dtype, device=t.device)
        big[:, 1:1 + t.shape[1]] = t
        return big[:, 1:1 + t.shape[1]]
    big = torch.zeros(t.shape[1], t.shape[0] + 5, dtype=t.dtype, device=t.device)
    big[:, 2:2 + t.shape[0]] = t.T
    return big[:, 2:2 + t.shape[0]].T


def test_fixed_seed_sweep_of_call_variants(dev):
    """200 calls drawn from a fixed seed that vary what the host side has to get right: each operand in host or
    device memory (host rows are streamed), in four memory layouts, isotropic or per-dimension lengthscales, a given
    ``out`` (C or F order, on the side the reference would allocate it) or none, w or none, an empty X1, and memory
    budgets down to 8 MB (row blocks; a budget that is too small must raise MemoryError).  Results against the fp64
    CPU path, measured on the scale of the summed terms."""
    from falkon_amd import FalkonOptions
    rng = np.random.default_rng(20240601)
    for it in range(200):
        dtype = torch.float32 if rng.random() < 0.5 else torch.float64
        d = int(rng.choice([1, 3, 9, 28, 33, 64, 65, 100, 300]))
        t = int(rng.choice([1, 2, 3, 5, 10, 17, 40, 70]))
        n, m = int(rng.integers(1, 6000)), int(rng.integers(1, 2500))
        if rng.random() < 0.05:
            n = 0
        if rng.random() < 0.05:
            m = int(rng.integers(1, 20))
        seed = int(rng.integers(1 << 30))
        per_dim = bool(rng.random() < 0.4)
        scale = 0.6 * np.sqrt(d) + 0.4
        sigma = torch.tensor(rng.uniform(0.5, 2.0, d) * scale, dtype=torch.float64) if per_dim else float(scale)
        name = NAMES[int(rng.integers(4))]
        budget = float(rng.choice([np.inf, np.inf, 64e6, 8e6]))
        host = [bool(rng.random() < 0.25) for _ in range(4)]
        lay = [int(rng.integers(4)) for _ in range(4)]
        use_w, use_out = bool(rng.random() < 0.7), bool(rng.random() < 0.5)
        out_lay = [int(rng.integers(2)), int(rng.integers(2))]
        print(f"[variants {it}] {name} {dtype} n={n} m={m} d={d} t={t} seed={seed} per_dim={per_dim} budget={budget:g} "
              f"host={host} layouts={lay} w={use_w} out={use_out}", flush=True)
        X, C, v, w = _case(n, m, d, t, dtype, seed)
        Xa, Ca, va, wa = (_laid_out(a if h else a.to(dev), l) for a, h, l in zip((X, C, v, w), host, lay))
        kernel = _kernel(name, sigma)
        opt = FalkonOptions(max_gpu_mem=budget)
        try:
            where = "cpu" if any(host[:3]) else dev
            om = _laid_out(torch.full((n, t), 7.0, dtype=dtype, device=where), out_lay[0]) if use_out else None
            got_m = kernel.mmv(Xa, Ca, va, out=om, opt=opt)
            where = "cpu" if any(host[:3]) or (use_w and host[3]) else dev
            od = _laid_out(torch.full((m, t), 7.0, dtype=dtype, device=where), out_lay[1]) if use_out else None
            got_d = kernel.dmmv(Xa, Ca, va, wa if use_w else None, out=od, opt=opt)
        except MemoryError:
            assert budget <= 8e6, "only the 8 MB budget may be too small for these sizes"
            continue
        if use_out:
            assert got_m.data_ptr() == om.data_ptr() and got_d.data_ptr() == od.data_ptr()
        assert got_m.shape == (n, t) and got_d.shape == (m, t)
        if n == 0:
            assert bool((got_d == 0).all())
            continue
        Xd, Cd, vd, wd = X.double(), C.double(), v.double(), (w.double() if use_w else None)
        ref_m = mmv_ref.fmmv_ref(Xd, Cd, vd, sigma, kernel_name=name)
        ref_d = mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma, kernel_name=name)
        abs_m = mmv_ref.fmmv_ref(Xd, Cd, vd.abs(), sigma, kernel_name=name)
        abs_d = mmv_ref.fdmmv_ref(Xd, Cd, vd.abs(), None if wd is None else wd.abs(), sigma, kernel_name=name)
        tol = 3e-6 if dtype == torch.float32 else 1e-12
        assert scaled_err(got_m, ref_m, abs_m) < tol and scaled_err(got_d, ref_d, abs_d) < tol
