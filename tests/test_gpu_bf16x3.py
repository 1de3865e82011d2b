"""The bf16x3 mode of the fp32 products (``FalkonOptions(bf16x3_cross_term=True)``, dtype code FLK_F32_BF16X3 of the
C ABI): the cross term of the squared distance on the bfloat16 matrix cores from an exact three-way bfloat16 split
of the scaled rows.  It must meet the same bar as the plain fp32 kernels (1e-5 relative, norm-wise per column,
against the CPU oracle) and must not be less accurate than they are against the fp64 result.
"""
import numpy as np
import pytest
import torch

from falkon_amd import Falkon, FalkonOptions, GaussianKernel, LaplacianKernel, MaternKernel
from oracle import brute, inputs, mmv_ref
from conftest import check_parity, rel_err

pytestmark = pytest.mark.gpu

SPLIT = FalkonOptions(bf16x3_cross_term=True)
PLAIN = FalkonOptions(bf16x3_cross_term=False)


def _data(n, m, d, t, seed, scale=1.0):
    g = np.random.default_rng(seed)
    mk = lambda *shape: torch.from_numpy(g.standard_normal(shape).astype(np.float32))     # noqa: E731
    return mk(n, d) * scale, mk(m, d) * scale, mk(m, t), mk(n, t)


@pytest.mark.parametrize("d", [1, 2, 9, 13, 14, 15, 28, 30, 31, 46, 47, 62])
@pytest.mark.parametrize("t", [1, 2, 3, 4, 5, 8, 10])
def test_products_vs_oracle(dev, d, t):
    n, m = 700 + 3 * d, 190 + d
    X, C, v, w = _data(n, m, d, t, seed=d + 100 * t)
    sigma = torch.tensor([0.9 * np.sqrt(d)], dtype=torch.float64)
    k = GaussianKernel(sigma, opt=FalkonOptions(bf16x3_cross_term=True, many_rhs_stored_blocks=True))
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    Xd, Cd, vd, wd = (a.double() for a in (X, C, v, w))
    check_parity(k.mmv(Xg, Cg, vg), mmv_ref.fmmv_ref(X, C, v, sigma), mmv_ref.fmmv_ref(Xd, Cd, vd, sigma), 1e-5)
    check_parity(k.dmmv(Xg, Cg, vg, wg), mmv_ref.fdmmv_ref(X, C, v, w, sigma),
                 mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma), 1e-5)
    check_parity(k.dmmv(Xg, Cg, vg, None), mmv_ref.fdmmv_ref(X, C, v, None, sigma),
                 mmv_ref.fdmmv_ref(Xd, Cd, vd, None, sigma), 1e-5)


@pytest.mark.parametrize("d", [9, 14, 28, 30, 31, 46, 47, 62])
@pytest.mark.parametrize("t", [7, 16, 17, 24, 33, 48, 64, 66, 70])
def test_many_right_hand_sides_on_the_register_resident_kernel(dev, d, t):
    """Five and more right-hand sides at up to 62 features (one to four k-steps): the bf16x3 chain for the cross term, the contraction of
    8 to 64 columns per pass on the fp32 matrix-core steps (every form, a second pass beyond 64 columns, which the
    per-lane FMA kernel takes when it has four columns or fewer); repeatable
    bit for bit, Fortran-ordered operands included."""
    n, m = 650 + 5 * d, 300 + t
    X, C, v, w = _data(n, m, d, t, seed=3 * d + 7 * t)
    sigma = torch.tensor([0.9 * np.sqrt(d)], dtype=torch.float64)
    k = GaussianKernel(sigma, opt=SPLIT)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    Xd, Cd, vd, wd = (a.double() for a in (X, C, v, w))
    check_parity(k.mmv(Xg, Cg, vg), mmv_ref.fmmv_ref(X, C, v, sigma), mmv_ref.fmmv_ref(Xd, Cd, vd, sigma), 1e-5)
    got = k.dmmv(Xg, Cg, vg, wg)
    check_parity(got, mmv_ref.fdmmv_ref(X, C, v, w, sigma), mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma), 1e-5)
    f = lambda a: a.T.contiguous().T                                                      # noqa: E731
    assert torch.equal(k.dmmv(f(Xg), f(Cg), f(vg), f(wg)), got)
    # the same numbers as the fp32 kernels give, to rounding
    plain = GaussianKernel(sigma).dmmv(Xg, Cg, vg, wg)
    assert rel_err(got, plain) < 5e-6


def test_layouts_sigma_per_dimension_and_repeatability(dev):
    X, C, v, w = _data(1500, 333, 11, 2, seed=7)
    sigma = torch.from_numpy(np.random.default_rng(3).uniform(1.0, 4.0, 11))
    k = GaussianKernel(sigma, opt=SPLIT)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    ref = k.dmmv(Xg, Cg, vg, wg)
    check_parity(ref, mmv_ref.fdmmv_ref(X, C, v, w, sigma),
                 mmv_ref.fdmmv_ref(X.double(), C.double(), v.double(), w.double(), sigma), 1e-5)
    # Fortran-ordered operands, an `out` buffer, a second call: bit-identical
    f = lambda a: a.T.contiguous().T                                                      # noqa: E731
    out = torch.empty(333, 2, dtype=torch.float32, device=dev)
    res = k.dmmv(f(Xg), f(Cg), f(vg), f(wg), out=out)
    assert res.data_ptr() == out.data_ptr() and torch.equal(res, ref)
    assert torch.equal(k.dmmv(Xg, Cg, vg, wg), ref)
    # host data goes through the same kernels
    assert torch.equal(k.dmmv(X, C, v, w).to(dev), ref)


@pytest.mark.parametrize("d", [63, 100, 300])
@pytest.mark.parametrize("t", [17, 32, 33, 48, 64, 65, 100])
def test_many_right_hand_sides_on_the_lds_tiled_kernel(dev, d, t):
    """Beyond 62 features the LDS-tiled kernel of the mode takes up to 64 columns per pass: 16 with the 16x16x1 step, 32
    and 64 with one or two groups of 32x32x2 steps (their right-hand sides swizzled in LDS, two operand stages instead
    of three), a second pass beyond 64 columns; ragged tiles on both sides, several reduction tiles per workgroup,
    Fortran-ordered operands, repeatable bit for bit."""
    n, m = 900 + 3 * d + t, 280 + t
    X, C, v, w = _data(n, m, d, t, seed=5 * d + 11 * t)
    sigma = torch.tensor([0.9 * np.sqrt(d)], dtype=torch.float64)
    k = GaussianKernel(sigma, opt=SPLIT)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    Xd, Cd, vd, wd = (a.double() for a in (X, C, v, w))
    check_parity(k.mmv(Xg, Cg, vg), mmv_ref.fmmv_ref(X, C, v, sigma), mmv_ref.fmmv_ref(Xd, Cd, vd, sigma), 1e-5)
    got = k.dmmv(Xg, Cg, vg, wg)
    check_parity(got, mmv_ref.fdmmv_ref(X, C, v, w, sigma), mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma), 1e-5)
    f = lambda a: a.T.contiguous().T                                                      # noqa: E731
    assert torch.equal(k.dmmv(f(Xg), f(Cg), f(vg), f(wg)), got)
    plain = GaussianKernel(sigma).dmmv(Xg, Cg, vg, wg)
    assert rel_err(got, plain) < 5e-6
    # fewer rows than one tile on either side.  (With so few rows of X single output columns are one cancelling sum
    # times a vector, whatever kernel computes them: the error is taken over the whole result here.)
    for nn, mm in ((40, m), (n, 1)):
        g1 = k.dmmv(Xg[:nn], Cg[:mm], vg[:mm], wg[:nn]).cpu().double()
        r1 = mmv_ref.fdmmv_ref(Xd[:nn], Cd[:mm], vd[:mm], wd[:nn], sigma)
        assert float((g1 - r1).norm() / r1.norm()) < 1e-5


@pytest.mark.parametrize("n,m,d,t", [(400, 150, 63, 2), (300, 257, 65, 1), (129, 64, 200, 10), (64, 300, 784, 5),
                                     (700, 129, 100, 4), (513, 260, 130, 16), (260, 513, 96, 17)])
def test_lds_tiled_kernel_vs_oracle(dev, n, m, d, t):
    """Feature counts beyond 62 run the LDS-tiled kernel of the mode: both epilogues, ragged tiles."""
    X, C, v, w = _data(n, m, d, t, seed=n + d)
    sigma = torch.tensor([0.9 * np.sqrt(d)], dtype=torch.float64)
    k = GaussianKernel(sigma, opt=FalkonOptions(bf16x3_cross_term=True, many_rhs_stored_blocks=True))
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    Xd, Cd, vd, wd = (a.double() for a in (X, C, v, w))
    check_parity(k.mmv(Xg, Cg, vg), mmv_ref.fmmv_ref(X, C, v, sigma), mmv_ref.fmmv_ref(Xd, Cd, vd, sigma), 1e-5)
    check_parity(k.dmmv(Xg, Cg, vg, wg), mmv_ref.fdmmv_ref(X, C, v, w, sigma),
                 mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma), 1e-5)
    assert torch.equal(k.dmmv(Xg, Cg, vg, wg), k.dmmv(Xg, Cg, vg, wg))


def test_fp64_data_is_not_affected_by_the_option(dev):
    X, C, v, _ = _data(300, 140, 40, 3, seed=6)
    Xd, Cd, vd = X.double().to(dev), C.double().to(dev), v.double().to(dev)
    assert torch.equal(GaussianKernel(15.0, opt=SPLIT).mmv(Xd, Cd, vd), GaussianKernel(15.0, opt=PLAIN).mmv(Xd, Cd, vd))


def test_config4_shape_reduced(dev):
    X, C, sigma, v, w = inputs.make_config("C4", N=20_000, M=2_000)
    k = GaussianKernel(sigma, opt=SPLIT)
    got = k.dmmv(X.to(dev), C.to(dev), v.to(dev), w.to(dev))
    check_parity(got, mmv_ref.fdmmv_ref(X, C, v, w, sigma, max_cpu_mem=2 * 2**30),
                 mmv_ref.fdmmv_ref(X.double(), C.double(), v.double(), w.double(), sigma, max_cpu_mem=4 * 2**30), 1e-5)
    exact = brute.radial_brute(X[:3000], C, sigma, "gaussian") @ v.double().numpy()
    e_split = rel_err(k.mmv(X[:3000].to(dev), C.to(dev), v.to(dev)), exact)
    e_plain = rel_err(GaussianKernel(sigma, opt=PLAIN).mmv(X[:3000].to(dev), C.to(dev), v.to(dev)), exact)
    assert e_split <= 1.5 * e_plain + 2e-7, (e_split, e_plain)


@pytest.mark.parametrize("name,make", [("laplacian", lambda s: LaplacianKernel(s, opt=SPLIT)),
                                       ("1.5-matern", lambda s: MaternKernel(s, 1.5, opt=SPLIT)),
                                       ("2.5-matern", lambda s: MaternKernel(s, 2.5, opt=SPLIT))])
def test_other_kernel_functions(dev, name, make):
    X, C, v, w = _data(900, 260, 20, 2, seed=9)
    sigma = torch.tensor([4.0], dtype=torch.float64)
    k = make(sigma)
    got = k.dmmv(X.to(dev), C.to(dev), v.to(dev), w.to(dev))
    check_parity(got, mmv_ref.fdmmv_ref(X, C, v, w, sigma, kernel_name=name),
                 mmv_ref.fdmmv_ref(X.double(), C.double(), v.double(), w.double(), sigma, kernel_name=name), 1e-5)
    K = brute.radial_brute(X, C, sigma, name)
    assert rel_err(k.mmv(X.to(dev), C.to(dev), v.to(dev)), K @ v.double().numpy()) < 5e-6


@pytest.mark.parametrize("scale", [1e-3, 1.0, 30.0])
def test_accuracy_is_that_of_the_fp32_kernels(dev, scale):
    """Against the fp64 closed form the split mode may not be further away than the plain fp32 kernels (small slack):
    data far from the origin (large norms, where the expanded squared distance cancels most) included."""
    X, C, v, _ = _data(4000, 500, 28, 1, seed=11, scale=scale)
    X, C = X + 2.0 * scale, C + 2.0 * scale
    sigma = torch.tensor([3.8 * scale], dtype=torch.float64)
    exact = brute.radial_brute(X, C, sigma, "gaussian") @ v.double().numpy()
    Xg, Cg, vg = X.to(dev), C.to(dev), v.to(dev)
    e_split = rel_err(GaussianKernel(sigma, opt=SPLIT).mmv(Xg, Cg, vg), exact)
    e_plain = rel_err(GaussianKernel(sigma, opt=PLAIN).mmv(Xg, Cg, vg), exact)
    assert e_split <= 1.5 * e_plain + 2e-7, (e_split, e_plain)


@pytest.mark.parametrize("d,t", [(28, 32), (28, 64), (40, 33), (9, 64), (46, 100)])
def test_cancelling_columns_with_many_right_hand_sides(dev, d, t):
    """Columns whose terms cancel two hundredfold (a nearly constant kernel matrix against right-hand sides that sum to
    almost nothing), at the widths of the 32- and 64-column passes: the mode may not be further from the fp64 result
    than the plain fp32 kernels are (the same bound as above, on the worst column), for K v and for K^T(K v)."""
    g = np.random.default_rng(300 + d + t)
    n, m = 3000, 2048
    X = torch.from_numpy(g.standard_normal((n, d)).astype(np.float32))
    C = torch.from_numpy(g.standard_normal((m, d)).astype(np.float32))
    z = g.standard_normal((m, t))
    v = torch.from_numpy((z - z.mean(0) * (1 - 1 / 200)).astype(np.float32))
    sigma = torch.tensor([12.0 * np.sqrt(d)], dtype=torch.float64)             # K within a few percent of 1
    K = brute.radial_brute(X, C, sigma, "gaussian")
    exact_m = K @ v.double().numpy()
    exact_d = K.T @ exact_m
    cancel = np.abs(exact_m).sum(0) / (np.abs(K) @ np.abs(v.double().numpy())).sum(0)
    assert cancel.max() < 0.05                                                   # the columns do cancel
    Xg, Cg, vg = X.to(dev), C.to(dev), v.to(dev)
    ks, kp = GaussianKernel(sigma, opt=SPLIT), GaussianKernel(sigma, opt=PLAIN)
    e_split, e_plain = rel_err(ks.mmv(Xg, Cg, vg), exact_m), rel_err(kp.mmv(Xg, Cg, vg), exact_m)
    assert e_split <= 1.5 * e_plain + 2e-7, ("mmv", e_split, e_plain)
    e_split, e_plain = rel_err(ks.dmmv(Xg, Cg, vg, None), exact_d), rel_err(kp.dmmv(Xg, Cg, vg, None), exact_d)
    assert e_split <= 1.5 * e_plain + 2e-7, ("dmmv", e_split, e_plain)


def test_config2_and_config3_shapes_reduced(dev):
    for name, N, M in (("C2", 100_000, 5_000), ("C3", 200_000, 5_000)):
        X, C, sigma, v, w = inputs.make_config(name, N=N, M=M)
        k = GaussianKernel(sigma, opt=SPLIT)
        got = k.dmmv(X.to(dev), C.to(dev), v.to(dev), None if w is None else w.to(dev))
        wd = None if w is None else w.double()
        check_parity(got, mmv_ref.fdmmv_ref(X, C, v, w, sigma, max_cpu_mem=2 * 2**30),
                     mmv_ref.fdmmv_ref(X.double(), C.double(), v.double(), wd, sigma, max_cpu_mem=4 * 2**30), 1e-5)


def test_falkon_fit_predict_with_the_option(dev):
    """End to end: the same model with and without the option (the preconditioner does not depend on it)."""
    g = np.random.default_rng(21)
    X = torch.from_numpy(g.standard_normal((20_000, 10)).astype(np.float32))
    a = g.standard_normal(10) / np.sqrt(10)
    y = torch.from_numpy(np.sign(np.sin(X.numpy() @ a) + 0.3 * g.standard_normal(20_000)).astype(np.float32)).reshape(-1, 1)
    preds = []
    for opt in (SPLIT, PLAIN):
        model = Falkon(GaussianKernel(2.5, opt=opt), penalty=1e-6, M=1_000, maxiter=15, seed=3, options=opt)
        model.fit(X.to(dev), y.to(dev))
        preds.append(model.predict(X[:4000].to(dev)).cpu())
    mse = [float(((p - y[:4000]) ** 2).mean()) for p in preds]
    assert abs(mse[0] - mse[1]) <= 1e-3 * mse[1]
    assert rel_err(preds[0], preds[1]) < 1e-3


@pytest.mark.parametrize("d", [9, 100])
def test_degenerate_shapes(dev, d):
    """No centres, no data rows, a single row on either side, in both kernels of the mode."""
    k = GaussianKernel(1.5 * np.sqrt(d), opt=SPLIT)
    X, C, v, w = _data(70, 9, d, 2, seed=3)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    r = k.mmv(Xg, Cg[:0], vg[:0])
    assert r.shape == (70, 2) and float(r.abs().max()) == 0.0
    assert k.dmmv(Xg, Cg[:0], vg[:0], wg).shape == (0, 2)
    r = k.dmmv(Xg[:0], Cg, vg, wg[:0])
    assert r.shape == (9, 2) and float(r.abs().max()) == 0.0
    assert k.mmv(Xg[:0], Cg, vg).shape == (0, 2)
    for n, m in ((1, 9), (70, 1), (1, 1)):
        got = k.dmmv(Xg[:n], Cg[:m], vg[:m], wg[:n])
        assert rel_err(got, mmv_ref.fdmmv_ref(X[:n], C[:m], v[:m], w[:n], k.sigma)) < 1e-5


@pytest.mark.parametrize("d,t", [(28, 2), (200, 2), (28, 40), (200, 12), (200, 40)])
def test_dmmv_replays_from_a_hip_graph(dev, d, t):
    """As for the fp32 kernels: nothing is allocated, cleared with a memset or synchronised, so a call can be captured
    into a HIP graph; every replay reproduces the eager result bit for bit.  With few and with many right-hand sides."""
    X, C, v, w = _data(20_000, 1_200, d, t, seed=21)
    k = GaussianKernel(0.7 * np.sqrt(d), opt=SPLIT)
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    out = torch.empty(1_200, t, device=dev)
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
    for _ in range(3):
        vg.copy_(torch.from_numpy(g.standard_normal((1_200, t)).astype(np.float32)))
        wg.copy_(torch.from_numpy(g.standard_normal((20_000, t)).astype(np.float32)))
        graph.replay()
        torch.cuda.synchronize()
        replayed = out.clone()
        eager = k.dmmv(Xg, Cg, vg, wg)
        torch.cuda.synchronize()
        assert torch.equal(replayed, eager)
    assert rel_err(eager, mmv_ref.fdmmv_ref(X, C, vg.cpu(), wg.cpu(), k.sigma)) < 1e-5


@pytest.mark.parametrize("n,m,d", [(600, 700, 130), (257, 513, 65), (64, 300, 110), (50, 45, 784), (1, 300, 100), (300, 1, 97)])
def test_kernel_matrix_in_the_mode(dev, n, m, d):
    """Beyond 64 features the option also serves the kernel matrix evaluated in fp32 (``no_single_kernel=False``): as
    close to the fp64 closed form as the fp32 kernels, both memory orders, a NaN row stays a NaN row, other kernel
    functions; with ``no_single_kernel=True`` (fp64 evaluation) the option changes nothing."""
    from oracle import brute
    g = np.random.default_rng(n + d)
    X = torch.from_numpy(g.standard_normal((n, d)).astype(np.float32) * 0.6)
    C = torch.from_numpy(g.standard_normal((m, d)).astype(np.float32) * 0.6)
    sigma = torch.from_numpy(g.uniform(0.8, 1.6, d) * np.sqrt(d))
    exact = torch.from_numpy(brute.gaussian_brute(X, C, sigma))
    split_opt = FalkonOptions(bf16x3_cross_term=True, no_single_kernel=False)
    k = GaussianKernel(sigma, opt=split_opt)
    Xg, Cg = X.to(dev), C.to(dev)
    got = k(Xg, Cg).cpu()
    plain = GaussianKernel(sigma, opt=FalkonOptions(no_single_kernel=False))(Xg, Cg).cpu()
    err, err_plain = float((got.double() - exact).abs().max()), float((plain.double() - exact).abs().max())
    assert got.dtype == torch.float32 and err <= 1.5 * err_plain + 2e-7
    out = torch.empty(m, n, dtype=torch.float32, device=dev).T                       # F-ordered result
    assert k(Xg, Cg, out=out).data_ptr() == out.data_ptr()      # operands change roles: same terms, another order
    assert float((out.cpu().double() - exact).abs().max()) <= 1.5 * err_plain + 2e-7
    Xb = X.clone()
    Xb[n // 2, 3] = float("nan")
    bad = k(Xb.to(dev), Cg).cpu()
    keep = torch.arange(n) != n // 2
    assert torch.isnan(bad[n // 2]).all() and torch.equal(bad[keep], got[keep])
    lap = LaplacianKernel(float(np.sqrt(d)), opt=split_opt)(Xg, Cg).cpu()
    want = torch.from_numpy(brute.radial_brute(X, C, torch.tensor([np.sqrt(d)]), "laplacian"))
    assert float((lap.double() - want).abs().max()) < 5e-6
    both = GaussianKernel(sigma, opt=FalkonOptions(bf16x3_cross_term=True, no_single_kernel=True))(Xg, Cg)
    assert torch.equal(both, GaussianKernel(sigma, opt=FalkonOptions(no_single_kernel=True))(Xg, Cg))


def test_stored_block_route_in_the_mode(dev):
    """Many right-hand sides beyond 64 features with the option: the stored blocks of K come from the bf16x3 kernel."""
    n, m, d, t = 700, 300, 100, 40
    X, C, v, w = _data(n, m, d, t, seed=11)
    sigma = torch.tensor([0.9 * np.sqrt(d)], dtype=torch.float64)
    k = GaussianKernel(sigma, opt=FalkonOptions(bf16x3_cross_term=True, many_rhs_stored_blocks=True))
    Xg, Cg, vg, wg = (a.to(dev) for a in (X, C, v, w))
    Xd, Cd, vd, wd = (a.double() for a in (X, C, v, w))
    check_parity(k.mmv(Xg, Cg, vg), mmv_ref.fmmv_ref(X, C, v, sigma), mmv_ref.fmmv_ref(Xd, Cd, vd, sigma), 1e-5)
    check_parity(k.dmmv(Xg, Cg, vg, wg), mmv_ref.fdmmv_ref(X, C, v, w, sigma),
                 mmv_ref.fdmmv_ref(Xd, Cd, vd, wd, sigma), 1e-5)


def test_kernel_matrix_in_the_mode_blocking_and_inputs(dev):
    """The drivers' row blocking of X1 under a small memory budget, F-ordered inputs (F-ordered result) and host inputs
    (result on the host) reach the same bf16x3 kernel: the blocked result equals the one-piece result bitwise, the
    others agree with the fp64 closed form like it."""
    from oracle import brute
    n, m, d = 900, 410, 150
    g = np.random.default_rng(3)
    X = torch.from_numpy(g.standard_normal((n, d)).astype(np.float32) * 0.5)
    C = torch.from_numpy(g.standard_normal((m, d)).astype(np.float32) * 0.5)
    exact = torch.from_numpy(brute.gaussian_brute(X, C, torch.tensor([9.0], dtype=torch.float64)))
    opt = FalkonOptions(bf16x3_cross_term=True, no_single_kernel=False)
    k = GaussianKernel(9.0, opt=opt)
    Xg, Cg = X.to(dev), C.to(dev)
    whole = k(Xg, Cg).cpu()
    err = float((whole.double() - exact).abs().max())
    assert err < 4e-7
    blocked = k(Xg, Cg, opt=FalkonOptions(bf16x3_cross_term=True, no_single_kernel=False, max_gpu_mem=2_500_000))
    assert torch.equal(blocked.cpu(), whole)
    Xf = torch.empty_strided(X.shape, (1, n), dtype=X.dtype).copy_(X).to(dev)
    Cf = torch.empty_strided(C.shape, (1, m), dtype=C.dtype).copy_(C).to(dev)
    got_f = k(Xf, Cf)
    assert got_f.stride(0) == 1 and float((got_f.cpu().double() - exact).abs().max()) < 4e-7
    host = k(X, C)
    assert host.device.type == "cpu" and float((host.double() - exact).abs().max()) < 4e-7
