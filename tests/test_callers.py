"""The callers of the hot path: conjugate gradient, preconditioner, Falkon estimator.

CPU part: the oracle's restatement of the pipeline is pinned against the closed-form solution of the
linear system (the reference's own check, falkon/tests/test_conjgrad.py:74-131), the product's CG and
preconditioner algebra are checked without a GPU.  GPU part: ``Falkon.fit`` / ``predict`` with the HIP
products against the CPU pipeline.
"""
import numpy as np
import pytest
import torch

from falkon_amd import Falkon, FalkonOptions, GaussianKernel
from falkon_amd.center_selection import FixedSelector, UniformSelector
from falkon_amd.optim import ConjugateGradient
from falkon_amd.preconditioner import FalkonPreconditioner
from oracle import falkon_ref, gaussian_ref, inputs


def _conjgrad_problem(dtype=np.float64):
    """falkon/tests/test_conjgrad.py:74-99: N=500, M=10, D=1000, sigma=100, lambda=10; gen_random seeds 10 / 9,
    centres chosen with default_rng(2)."""
    N, M, D = 500, 10, 1000
    X = torch.from_numpy(inputs.gen_random(N, D, dtype, F=False, seed=10))
    Y = torch.from_numpy(inputs.gen_random(N, 1, dtype, F=False, seed=9))
    idx = np.random.default_rng(2).choice(N, M, replace=False)
    return X, Y, X[idx].clone(), 100.0, 10.0


def test_oracle_pipeline_solves_the_normal_equations():
    X, Y, C, sigma, lam = _conjgrad_problem()
    alpha = falkon_ref.falkon_fit_ref(X, Y, C, sigma, lam, maxiter=200, cg_tolerance=1e-10)
    expected = falkon_ref.nystrom_krr_direct(X, Y, C, sigma, lam)
    np.testing.assert_allclose(alpha.numpy(), expected, rtol=1e-5)


def test_oracle_pipeline_multiple_rhs_and_prediction():
    X, Y, C, sigma, lam = _conjgrad_problem()
    Y10 = torch.from_numpy(inputs.gen_random(500, 10, np.float64, seed=9))
    alpha = falkon_ref.falkon_fit_ref(X, Y10, C, sigma, lam, maxiter=200, cg_tolerance=1e-10)
    expected = falkon_ref.nystrom_krr_direct(X, Y10, C, sigma, lam)
    np.testing.assert_allclose(alpha.numpy(), expected, rtol=1e-5)
    Knm = gaussian_ref.rbf_core_ref(X, C, None, torch.tensor([sigma]))
    torch.testing.assert_close(falkon_ref.falkon_predict_ref(X, C, alpha, sigma), Knm @ alpha, rtol=1e-10, atol=1e-12)


def test_conjugate_gradient_on_dense_spd_system():
    g = np.random.default_rng(0)
    Q = g.standard_normal((30, 30))
    A = torch.from_numpy(Q @ Q.T + 30 * np.eye(30))
    B = torch.from_numpy(g.standard_normal((30, 3)))
    cg = ConjugateGradient(FalkonOptions(cg_tolerance=1e-9))
    X = cg.solve(None, B, lambda v: A @ v, max_iter=100)
    torch.testing.assert_close(A @ X, B, rtol=1e-9, atol=1e-9)
    assert cg.num_iter < 60
    X2 = cg.solve(X.clone(), B, lambda v: A @ v, max_iter=5)          # warm start stays converged
    torch.testing.assert_close(X2, X, rtol=1e-9, atol=1e-9)


class _DenseKernel:
    """Stands in for the GPU kernel object so the preconditioner algebra can run on the host."""

    def __init__(self, sigma):
        self.sigma = torch.tensor([float(sigma)])

    def __call__(self, X1, X2, opt=None):
        return gaussian_ref.rbf_core_ref(X1.double(), X2.double(), None, self.sigma).to(X1.dtype)


def test_preconditioner_invariants():
    """falkon/tests/test_chol_prec.py:17-67: T^T T = K + eps M I, A^T A = T T^T / M + lambda I, solves invert."""
    g = np.random.default_rng(1)
    C = torch.from_numpy(g.standard_normal((40, 5)))
    lam, M = 1e-3, 40
    pc = FalkonPreconditioner(lam, _DenseKernel(2.0), FalkonOptions())
    with pytest.raises(RuntimeError):
        pc.invA(torch.ones(40, 1, dtype=torch.float64))
    pc.init(C)
    K = _DenseKernel(2.0)(C, C)
    T, A = pc.LT.T, pc.LA.T
    torch.testing.assert_close(T.T @ T, K + 1e-13 * M * torch.eye(M, dtype=torch.float64), rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(A.T @ A, T @ T.T / M + lam * torch.eye(M, dtype=torch.float64), rtol=1e-10, atol=1e-10)
    v = torch.from_numpy(g.standard_normal((40, 3)))
    torch.testing.assert_close(A @ pc.invA(v), v, rtol=1e-8, atol=1e-8)
    torch.testing.assert_close(A.T @ pc.invAt(v), v, rtol=1e-8, atol=1e-8)
    torch.testing.assert_close(T @ pc.invT(v), v, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(T.T @ pc.invTt(v), v, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(pc.apply(v), pc.invT(pc.invA(v)), rtol=0, atol=0)
    torch.testing.assert_close(pc.apply_t(v), pc.invAt(pc.invTt(v)), rtol=0, atol=0)
    # and the oracle's scipy restatement builds the same factors
    ref = falkon_ref.PrecondRef(C, torch.tensor([2.0]), lam)
    np.testing.assert_allclose(ref.T, T.numpy(), rtol=1e-8, atol=1e-10)
    np.testing.assert_allclose(ref.A, A.numpy(), rtol=1e-8, atol=1e-10)


def test_blocked_triangular_solves_match_lapack():
    """The block solver behind invT / invTt / invA / invAt against scipy's triangular solve, ragged last
    block, several right-hand sides; the two directions are exact transposes of each other."""
    import scipy.linalg as sla
    from falkon_amd.preconditioner import _BlockedTriangular
    g = np.random.default_rng(3)
    for M, blk in ((1, 4), (37, 8), (64, 16), (130, 32)):
        B = g.standard_normal((M, M))
        L = np.linalg.cholesky(B @ B.T + M * np.eye(M))
        for order in ("row-major", "column-major"):          # torch.linalg.cholesky returns column-major factors
            Lt = torch.from_numpy(L.copy()) if order == "row-major" else torch.from_numpy(L.T.copy()).T
            bt = _BlockedTriangular(Lt, block=blk, min_size=0)
            assert len(bt.bounds) == -(-M // blk) and bt.row_major == (order == "row-major" or M < 2)
            for t in (1, 3):
                rhs = g.standard_normal((M, t))
                np.testing.assert_allclose(bt.solve(torch.from_numpy(rhs)).numpy(),
                                           sla.solve_triangular(L, rhs, lower=True), rtol=1e-10, atol=1e-12)
                np.testing.assert_allclose(bt.solve_t(torch.from_numpy(rhs)).numpy(),
                                           sla.solve_triangular(L, rhs, lower=True, trans=1), rtol=1e-10, atol=1e-12)
            u, v = torch.from_numpy(g.standard_normal((M, 1))), torch.from_numpy(g.standard_normal((M, 1)))
            assert abs(float((u * bt.solve(v)).sum() - (bt.solve_t(u) * v).sum())) < 1e-12
    from falkon_amd.preconditioner import _gram_of_lower_factor
    for M, blk in ((5, 8), (37, 8), (64, 16)):
        L = torch.from_numpy(np.tril(g.standard_normal((M, M))))
        G = _gram_of_lower_factor(L, block=blk)
        torch.testing.assert_close(torch.tril(G), torch.tril(L.T @ L), rtol=1e-12, atol=1e-12)
    from falkon_amd.preconditioner import _cholesky_lower_
    for M, blk in ((40, 8), (37, 16), (64, 64)):
        B = g.standard_normal((M, M))
        A = torch.from_numpy(B @ B.T + M * np.eye(M))
        ref = torch.linalg.cholesky(A)
        low = torch.tril(A) + torch.triu(torch.full_like(A, float("nan")), 1)      # the upper triangle is never read
        torch.testing.assert_close(_cholesky_lower_(low, block=blk, min_size=0), ref, rtol=1e-11, atol=1e-11)
    with pytest.raises(torch.linalg.LinAlgError):
        _cholesky_lower_(-torch.eye(20, dtype=torch.float64), block=8, min_size=0)
    # small factors go straight to the library routine
    assert _BlockedTriangular(torch.eye(10, dtype=torch.float64)).bounds == []


def test_center_selection_is_seeded_uniform_without_replacement():
    X = torch.arange(200, dtype=torch.float32).reshape(100, 2)
    sel = UniformSelector(np.random.default_rng(7), num_centers=10)
    C, idx = sel.select_indices(X, None)
    expect = np.random.default_rng(7).choice(100, size=10, replace=False)
    assert np.array_equal(idx.numpy(), expect) and torch.equal(C, X[expect])
    assert len(set(idx.tolist())) == 10
    Xf = torch.empty_strided((100, 2), (1, 100)).copy_(X)
    assert UniformSelector(0, 5).select(Xf, None).stride(0) == 1          # memory order is kept
    with pytest.warns(UserWarning):
        assert UniformSelector(0, 500).select(X, None).shape[0] == 100
    fs = FixedSelector(X[:3])
    assert fs.select(X, None) is not None
    with pytest.raises(RuntimeError):
        fs.select_indices(X, None)


def test_falkon_constructor_errors():
    k = GaussianKernel(1.0)
    with pytest.raises(ValueError):
        Falkon(k, 1e-3, None)
    with pytest.raises(ValueError):
        Falkon(k, 1e-3, 10, center_selection="kmeans")
    f = Falkon(k, 1e-3, 10)
    with pytest.raises(RuntimeError):
        f.predict(torch.zeros(3, 2))
    with pytest.raises(ValueError):
        f.fit(torch.zeros(5, 2), torch.zeros(4))
    with pytest.raises(TypeError):
        f.fit(torch.zeros(5, 2), torch.zeros(5, dtype=torch.float64))
    assert f.get_params()["M"] == 10                                       # sklearn surface


# --------------------------------------------------------------------------------------------------
@pytest.mark.gpu
def test_falkon_cg_matches_direct_solve_on_gpu(dev):
    """The reference's conjugate-gradient test (tests/test_conjgrad.py:100-131) through the HIP products."""
    X, Y, C, sigma, lam = _conjgrad_problem()
    model = Falkon(GaussianKernel(sigma), lam, M=10, center_selection=FixedSelector(C), maxiter=200,
                   options=FalkonOptions(cg_tolerance=1e-10))
    model.fit(X.to(dev), Y.to(dev))
    expected = falkon_ref.nystrom_krr_direct(X, Y, C, sigma, lam)
    np.testing.assert_allclose(model.alpha_.cpu().numpy(), expected, rtol=1e-5)
    Y10 = torch.from_numpy(inputs.gen_random(500, 10, np.float64, seed=9))
    model.fit(X.to(dev), Y10.to(dev))
    np.testing.assert_allclose(model.alpha_.cpu().numpy(), falkon_ref.nystrom_krr_direct(X, Y10, C, sigma, lam), rtol=1e-5)


@pytest.mark.gpu
def test_falkon_with_matern_and_laplacian_kernels_on_gpu(dev):
    """The same conjugate-gradient test with the other distance kernels: preconditioner (kernel matrix), CG
    (dfmmv) and prediction (fmmv) all run the kernel's own function."""
    from falkon_amd import LaplacianKernel, MaternKernel
    X, Y, C, sigma, lam = _conjgrad_problem()
    for kernel, name in ((LaplacianKernel(sigma), "laplacian"), (MaternKernel(sigma, 1.5), "1.5-matern"),
                         (MaternKernel(sigma, 2.5), "2.5-matern")):
        model = Falkon(kernel, lam, M=10, center_selection=FixedSelector(C), maxiter=200,
                       options=FalkonOptions(cg_tolerance=1e-10))
        model.fit(X.to(dev), Y.to(dev))
        expected = falkon_ref.nystrom_krr_direct(X, Y, C, sigma, lam, kernel_name=name)
        np.testing.assert_allclose(model.alpha_.cpu().numpy(), expected, rtol=1e-5)
        pred = model.predict(X[:50].to(dev)).cpu()
        from oracle import brute
        np.testing.assert_allclose(pred.numpy(), brute.radial_brute(X[:50], C, torch.tensor([sigma]), name) @ expected,
                                   rtol=1e-5, atol=1e-8)


def _config5(N, Nts, seed=1005, d=28):
    rng = np.random.default_rng(seed)
    X = rng.standard_normal((N, d)).astype(np.float32)
    Xts = rng.standard_normal((Nts, d)).astype(np.float32)
    a = rng.standard_normal(d) / np.sqrt(d)
    y = np.sign(np.sin(X @ a) + 0.3 * rng.standard_normal(N)).astype(np.float32)
    yts = np.sign(np.sin(Xts @ a) + 0.3 * rng.standard_normal(Nts)).astype(np.float32)
    return tuple(torch.from_numpy(t) for t in (X, y.reshape(-1, 1), Xts, yts.reshape(-1, 1)))


@pytest.mark.gpu
def test_config5_reduced_end_to_end(dev, monkeypatch):
    """Config 5 at N=40000, M=2000, test 8000: sigma=3.8, penalty=1e-6, 20 CG iterations, fp32.
    Test MSE of the GPU fit must be within 0.1 % (relative) of the CPU pipeline's on the same centres."""
    X, Y, Xts, Yts = _config5(40_000, 8_000)
    M, sigma, lam = 2_000, 3.8, 1e-6
    model = Falkon(GaussianKernel(sigma), lam, M=M, maxiter=20, seed=12)
    model.fit(X, Y)                                                        # host data, GPU compute, host results
    assert model.alpha_.device.type == "cpu" and model.alpha_.shape == (M, 1)
    pred = model.predict(Xts)
    mse_gpu = float(((pred - Yts) ** 2).mean())
    C = model.ny_points_
    alpha_ref = falkon_ref.falkon_fit_ref(X, Y, C, sigma, lam, maxiter=20)
    mse_ref = float(((falkon_ref.falkon_predict_ref(Xts, C, alpha_ref, sigma) - Yts) ** 2).mean())
    assert abs(mse_gpu - mse_ref) / mse_ref < 1e-3, (mse_gpu, mse_ref)
    assert mse_gpu < 0.9                                                   # it learned something (labels are +-1)
    # resident-data variant gives the same model
    model2 = Falkon(GaussianKernel(sigma), lam, M=M, maxiter=20, center_selection=FixedSelector(C))
    model2.fit(X.to(dev), Y.to(dev))
    assert model2.alpha_.is_cuda
    mse2 = float(((model2.predict(Xts.to(dev)).cpu() - Yts) ** 2).mean())
    assert abs(mse2 - mse_gpu) / mse_gpu < 1e-3
    # the blocked triangular solves (used from M = 4096 on) and factorisation give the same model
    import falkon_amd.preconditioner as pcm
    monkeypatch.setattr(pcm, "TRSV_BLOCK", 256)
    monkeypatch.setattr(pcm, "TRSV_MIN_SIZE", 512)
    monkeypatch.setattr(pcm, "CHOL_BLOCK", 512)              # and the blocked Cholesky (host matrices from M = 16384 on;
    monkeypatch.setattr(pcm, "CHOL_BLOCK_DEVICE", 512)       # device matrices beyond one block column of 2048)
    monkeypatch.setattr(pcm, "CHOL_MIN_SIZE", 1024)
    model4 = Falkon(GaussianKernel(sigma), lam, M=M, maxiter=20, center_selection=FixedSelector(C))
    model4.fit(X.to(dev), Y.to(dev))
    assert len(model4.precond._T.bounds) == 8
    mse4 = float(((model4.predict(Xts.to(dev)).cpu() - Yts) ** 2).mean())
    assert abs(mse4 - mse_ref) / mse_ref < 1e-3, (mse4, mse_ref)
    monkeypatch.undo()
    # warm start from the preconditioned solution resumes instead of restarting
    model3 = Falkon(GaussianKernel(sigma), lam, M=M, maxiter=2, center_selection=FixedSelector(C))
    model3.fit(X.to(dev), Y.to(dev), warm_start=model2.beta_.clone())
    mse3 = float(((model3.predict(Xts.to(dev)).cpu() - Yts) ** 2).mean())
    assert abs(mse3 - mse_gpu) / mse_gpu < 5e-3


# --------------------------------------------------------------------------------------------------
# The reference's estimator tests (tests/test_falkon.py:20-123,126-149,271-304): same sklearn data sets
# (random_state=11), same kernels, penalties, M, seeds and accuracy thresholds, fitted through the HIP products.
# --------------------------------------------------------------------------------------------------
def _cls_data():
    from sklearn import datasets
    X, Y = datasets.make_classification(1000, 10, n_classes=2, random_state=11)
    Y = Y.astype(np.float64).reshape(-1, 1)
    Y[Y == 0] = -1
    return torch.from_numpy(X.astype(np.float64)), torch.from_numpy(Y)


def _multicls_data():
    from sklearn import datasets
    X, Y = datasets.make_classification(2000, 30, n_classes=20, n_informative=6, random_state=11)
    return torch.from_numpy(X.astype(np.float64)), torch.from_numpy(np.eye(20, dtype=np.float64)[Y.astype(np.int32), :])


def _reg_data():
    from sklearn import datasets
    X, Y = datasets.make_regression(1000, 30, random_state=11)
    X, Y = X.astype(np.float64), Y.astype(np.float64).reshape(-1, 1)
    return tuple(torch.from_numpy(a) for a in (X[:800], Y[:800], X[800:], Y[800:]))


def _c_err(t, p):
    return 100 * torch.sum(t * p <= 0).to(torch.float32) / t.shape[0], "c-err"


def _rmse(t, p):
    return torch.sqrt(torch.mean((t - p) ** 2)).item(), "RMSE"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_reference_accuracy_thresholds(dev, dtype):
    """Binary classification error below 5 %, 20-class error below 0.23, regression test RMSE below 2.5 and above
    the training RMSE (tests/test_falkon.py:62-123), with host tensors as there (the fit moves them to the GPU)."""
    X, Y = (a.to(dtype) for a in _cls_data())
    flk = Falkon(kernel=GaussianKernel(2.0), penalty=1e-6, M=500, seed=10, maxiter=10).fit(X, Y)
    assert float(_c_err(flk.predict(X), Y)[0]) < 5

    X, Y = (a.to(dtype) for a in _multicls_data())
    flk = Falkon(kernel=GaussianKernel(10.0), penalty=1e-6, M=500, seed=10, maxiter=10).fit(X, Y)
    preds = flk.predict(X)
    assert preds.shape == Y.shape and preds.device == X.device
    assert float((preds.argmax(1) != Y.argmax(1)).double().mean()) < 0.23

    Xtr, Ytr, Xts, Yts = (a.to(dtype) for a in _reg_data())
    flk = Falkon(kernel=GaussianKernel(20.0), penalty=1e-6, M=Xtr.shape[0] // 2, seed=10, maxiter=10)
    flk.fit(Xtr, Ytr, Xts=Xts, Yts=Yts)
    assert flk.predict(Xts).shape == (Yts.shape[0], 1)
    ts_err, tr_err = _rmse(flk.predict(Xts), Yts)[0], _rmse(flk.predict(Xtr), Ytr)[0]
    assert tr_err < ts_err < 2.5


@pytest.mark.gpu
def test_reference_gpu_predict_and_validation_callback(dev, capsys):
    """tests/test_falkon.py:126-149: fit on host data with a validation set and an error function, move the model to
    the GPU, predict there."""
    Xtr, Ytr, Xts, Yts = _reg_data()
    flk = Falkon(kernel=GaussianKernel(20.0), penalty=1e-6, M=500, seed=10, error_fn=_rmse)
    flk.fit(Xtr, Ytr, Xts=Xts, Yts=Yts)
    assert "validation RMSE" in capsys.readouterr().out and len(flk.val_errors_) > 0
    flk.to("cuda:0")
    ts_preds, tr_preds = flk.predict(Xts.to(dev)), flk.predict(Xtr.to(dev))
    assert ts_preds.device.type == "cuda" and ts_preds.shape == (Yts.shape[0], 1)
    ts_err, tr_err = _rmse(ts_preds.cpu(), Yts)[0], _rmse(tr_preds.cpu(), Ytr)[0]
    assert tr_err < ts_err < 2.5


@pytest.mark.gpu
def test_reference_incore_falkon(dev):
    """tests/test_falkon.py:271-304: InCoreFalkon refuses host tensors in fit and predict, and classifies the GPU
    copy of the data with less than 5 % error."""
    from falkon_amd import InCoreFalkon
    X, Y = _cls_data()
    flk = InCoreFalkon(kernel=GaussianKernel(2.0), penalty=1e-6, M=500, seed=10)
    with pytest.raises(ValueError):
        flk.fit(X, Y)
    flk.fit(X.to(dev), Y.to(dev))
    with pytest.raises(ValueError):
        flk.predict(X)
    flkc = InCoreFalkon(kernel=GaussianKernel(2.0), penalty=1e-6, M=500, seed=10, maxiter=20, error_fn=_c_err)
    flkc.fit(X.to(dev), Y.to(dev))
    preds = flkc.predict(X.to(dev))
    assert preds.device == X.to(dev).device
    assert float(_c_err(preds, Y.to(dev))[0]) < 5


def test_falkon_cg_refuses_to_run_outside_inference_mode():
    """tests/test_conjgrad.py:133-143: RuntimeError naming InferenceMode (checked before anything touches the GPU)."""
    from falkon_amd.optim import FalkonConjugateGradient
    X, Y, C, sigma, lam = _conjgrad_problem()
    solver = FalkonConjugateGradient(GaussianKernel(sigma), FalkonPreconditioner(lam, GaussianKernel(sigma), FalkonOptions()),
                                     FalkonOptions())
    with pytest.raises(RuntimeError, match="InferenceMode"):
        solver.solve(X=X, M=C, Y=Y, _lambda=lam, initial_solution=None, max_iter=100)


@pytest.mark.gpu
def test_falkon_cg_restarts(dev):
    """tests/test_conjgrad.py:145-166: thirty solves of six iterations each, every one started from the last
    solution, reach the direct solution of the normal equations."""
    from falkon_amd.optim import FalkonConjugateGradient
    X, Y, C, sigma, lam = _conjgrad_problem()
    kernel = GaussianKernel(sigma)
    opt = FalkonOptions(cg_tolerance=1e-10)
    Xd, Yd, Cd = X.to(dev), Y.to(dev), C.to(dev)
    with torch.inference_mode():
        prec = FalkonPreconditioner(lam, kernel, opt)
        prec.init(Cd)
        solver = FalkonConjugateGradient(kernel, prec, opt)
        sol = None
        for _ in range(30):
            sol = solver.solve(X=Xd, M=Cd, Y=Yd, _lambda=lam, initial_solution=sol, max_iter=6)
        alpha = prec.apply(sol)
    np.testing.assert_allclose(alpha.cpu().numpy(), falkon_ref.nystrom_krr_direct(X, Y, C, sigma, lam), rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("order", ["C", "F"])
@pytest.mark.parametrize("dtype,la,tol", [(torch.float32, 100.0, 1e-2), (torch.float64, 100.0, 1e-10),
                                          (torch.float64, 0.0, 1e-10)])
def test_reference_preconditioner_invariants_on_gpu(dev, order, dtype, la, tol):
    """The reference's preconditioner test on the GPU (tests/test_chol_prec.py:17-67,99-163): 100 uniform points,
    GaussianKernel(10), penalty 100 and 0; with T = chol(K_MM) and A = chol(T T^T / M + la I), solving T^T x = K_MM
    gives T, solving A^T x = A^T A gives A, invT(invTt(K_MM)) = I, and the preconditioner inverts
    n/M K_MM^T K_MM + la n K_MM (tolerances as there).  The Gram matrix comes from the HIP kernel-matrix path."""
    M, N = 100, 50_000
    mat = torch.from_numpy(inputs.gen_random(M, M, "float64", F=True, seed=10)).to(dtype)
    mat = (mat.T.contiguous().T if order == "F" else mat.contiguous()).to(dev)
    kernel = GaussianKernel(10.0)
    opt = FalkonOptions(no_single_kernel=True)
    with torch.inference_mode():
        gram = kernel(mat, mat, opt=opt)
        prec = FalkonPreconditioner(la, kernel, opt)
        prec.init(mat)
        eye = torch.eye(M, dtype=dtype, device=dev)
        T = prec.invTt(gram)
        assert T.dtype == dtype
        np.testing.assert_allclose((T.T @ T).cpu().numpy(), gram.cpu().numpy(), rtol=tol, atol=tol)
        ATA = (1.0 / M) * T @ T.T + la * eye
        A = prec.invAt(ATA)
        np.testing.assert_allclose((A.T @ A).cpu().numpy(), ATA.cpu().numpy(), rtol=tol, atol=tol)
        np.testing.assert_allclose(prec.invT(prec.invTt(gram)).cpu().numpy(), eye.cpu().numpy(), rtol=10 * tol, atol=10 * tol)
        desired = (N / M) * gram.T @ gram + la * N * gram
        out = (1 / N) * prec.invT(prec.invA(prec.invAt(prec.invTt(desired))))
        prec_tol = 10 * tol if la else 100 * tol            # test_chol_prec.py:117,133
        np.testing.assert_allclose(out.cpu().numpy(), eye.cpu().numpy(), rtol=prec_tol, atol=prec_tol)


def test_center_selection_with_targets():
    """tests/test_nysel.py:109-125: centres and their targets come back together, orders, dtypes and devices kept."""
    M, D, num = 10_000, 20, 100
    X = torch.from_numpy(inputs.gen_random(M, D, "float64", F=True, seed=0))
    Y = torch.empty(M, 1, dtype=X.dtype)
    sel = UniformSelector(np.random.default_rng(0), num_centers=num)
    centers, cY = sel.select(X, Y)
    assert centers.stride() == (1, num) and centers.size() == (num, D) and cY.size() == (num, 1)
    assert centers.dtype == X.dtype and cY.dtype == Y.dtype and centers.device == X.device
    centers, cY, idx = sel.select_indices(X, Y)
    assert idx.dtype == torch.long and len(idx) == centers.shape[0] == cY.shape[0]
    assert torch.equal(centers, X[idx])


@pytest.mark.gpu
def test_center_selection_on_gpu_tensors(dev):
    """tests/test_nysel.py:37-55: GPU data gives GPU centres (and indices) with the input's strides."""
    M, D, num = 10_000, 20, 100
    X = torch.from_numpy(inputs.gen_random(M, D, "float64", F=False, seed=0)).to(dev)
    sel = UniformSelector(np.random.default_rng(0), num_centers=num)
    centers = sel.select(X, None)
    assert centers.stride() == (D, 1) and centers.size() == (num, D)
    assert centers.dtype == X.dtype and centers.device == X.device
    centers, idx = sel.select_indices(X, None)
    assert centers.device == idx.device and idx.dtype == torch.long and len(idx) == num


# --------------------------------------------------------------------------------------------------
# weighted least squares (falkon/optim/conjgrad.py:258-300, flk_preconditioner.py:94-160, models/falkon.py:258-275)
# --------------------------------------------------------------------------------------------------
def _two_to_one(y, x, indices):
    """The reference's test weights: class -1 counts twice (tests/test_falkon.py:212-216)."""
    weight = torch.empty_like(y)
    weight[y == 1] = 1
    weight[y == -1] = 2
    return weight


@pytest.mark.gpu
def test_weighted_falkon_solves_the_weighted_normal_equations(dev):
    """alpha = (K_nm^T W K_nm + lambda n K_mm)^-1 K_nm^T W y, from the definition in fp64, for weights that depend on
    the targets; centres are rows of the data, so that the preconditioner gets their weights."""
    X, Y, _, sigma, lam = _conjgrad_problem()
    Y = torch.sign(Y - 0.5)
    idx = torch.from_numpy(np.random.default_rng(2).choice(X.shape[0], 10, replace=False))
    C = X[idx].clone()
    model = Falkon(GaussianKernel(sigma), lam, M=10, center_selection=FixedSelector(C, idx_centers=idx), maxiter=200,
                   weight_fn=_two_to_one, options=FalkonOptions(cg_tolerance=1e-10))
    model.fit(X.to(dev), Y.to(dev))
    Knm = gaussian_ref.rbf_core_ref(X, C, None, torch.tensor([sigma])).numpy()
    Kmm = gaussian_ref.rbf_core_ref(C, C, None, torch.tensor([sigma])).numpy()
    W = _two_to_one(Y, X, None).numpy()
    expected = np.linalg.solve(Knm.T @ (W * Knm) + lam * X.shape[0] * Kmm, Knm.T @ (W * Y.numpy()))
    np.testing.assert_allclose(model.alpha_.cpu().numpy(), expected, rtol=1e-5)
    # the preconditioner's second factor is that of T W_M T^T / M + lambda I
    T = model.precond.LT.T.cpu().numpy()
    Wm = _two_to_one(Y[idx], None, None).numpy().reshape(-1)
    A = model.precond.LA.T.cpu().numpy()
    np.testing.assert_allclose(A.T @ A, T @ (Wm[:, None] * T.T) / 10 + lam * np.eye(10), rtol=1e-9, atol=1e-12)


@pytest.mark.gpu
@pytest.mark.parametrize("where", ["incore", "mixed"])
def test_reference_weighted_falkon_classification(dev, where):
    """tests/test_falkon.py:191-244: weighting class -1 twice lowers its error and does not lower the other's."""
    from falkon_amd import InCoreFalkon
    X, Y = _cls_data()
    cls = Falkon
    if where == "incore":
        X, Y, cls = X.to(dev), Y.to(dev), InCoreFalkon
    errs = {}
    for name, wf in (("weighted", _two_to_one), ("plain", None)):
        flk = cls(kernel=GaussianKernel(2.0), penalty=1e-6, M=500, seed=10, weight_fn=wf).fit(X, Y)
        preds = flk.predict(X)
        errs[name] = (float(_c_err(preds[Y == -1], Y[Y == -1])[0]), float(_c_err(preds[Y == 1], Y[Y == 1])[0]))
    assert errs["weighted"][0] < errs["plain"][0], "Error of weighted class is higher than without weighting"
    assert errs["weighted"][1] >= errs["plain"][1], "Error of unweighted class is lower than in flk with no weights"


@pytest.mark.gpu
@pytest.mark.parametrize("incore", [False, True])
def test_reference_precomputed_kernel_fit(dev, incore):
    """tests/test_falkon.py:167-189,306-340: with ``store_kernel_d_threshold`` below the feature count the fit keeps
    K(X, centres) in memory and runs its products on it; same accuracy bounds, and the same coefficients as the fit
    that evaluates the kernel in every iteration."""
    from falkon_amd import InCoreFalkon
    Xtr, Ytr, Xts, Yts = _reg_data()
    if incore:
        Xtr, Ytr, Xts, Yts = (a.to(dev) for a in (Xtr, Ytr, Xts, Yts))
    cls = InCoreFalkon if incore else Falkon
    opt = FalkonOptions(never_store_kernel=False, store_kernel_d_threshold=Xtr.shape[1] - 1)
    flk = cls(kernel=GaussianKernel(20.0), penalty=1e-6, M=Xtr.shape[0] // 2, seed=10, options=opt, maxiter=10)
    assert flk._can_store_knm(Xtr.to(dev), Xtr[:400].to(dev))
    flk.fit(Xtr, Ytr, Xts=Xts, Yts=Yts)
    assert flk.predict(Xts).shape == (Yts.shape[0], 1)
    ts_err, tr_err = _rmse(flk.predict(Xts), Yts)[0], _rmse(flk.predict(Xtr), Ytr)[0]
    assert tr_err < ts_err < 2.5
    plain = cls(kernel=GaussianKernel(20.0), penalty=1e-6, M=Xtr.shape[0] // 2, seed=10, maxiter=10,
                options=FalkonOptions(never_store_kernel=True, store_kernel_d_threshold=Xtr.shape[1] - 1))
    assert not plain._can_store_knm(Xtr.to(dev), Xtr[:400].to(dev))
    plain.fit(Xtr, Ytr)
    # (penalty 1e-6, ten iterations: the coefficients feel the different summation order of the two routes)
    a, b = flk.alpha_.cpu().numpy(), plain.alpha_.cpu().numpy()
    np.testing.assert_allclose(a, b, rtol=1e-4, atol=1e-6 * np.abs(b).max())


@pytest.mark.gpu
@pytest.mark.parametrize("weighted", [False, True])
def test_fit_with_operands_packed_once_is_the_same_fit(dev, weighted):
    """``cg_pack_once`` (the default: X and the centres packed once for the solve) changes no result: the coefficients of
    a GPU fit are bit for bit those of a fit whose every product packs its operands itself; also with a weight function."""
    X, Y, _, _ = _config5(20_000, 10)
    Xg, Yg = X.to(dev), Y.to(dev)
    C = X[:700].clone()
    weight_fn = (lambda Y, X, idx: torch.where(Y > 0, 2.0, 1.0).to(Y.dtype)) if weighted else None
    fits = []
    for once in (True, False):
        opt = FalkonOptions(cg_pack_once=once)
        model = Falkon(GaussianKernel(3.8, opt=opt), 1e-6, M=700, maxiter=10, options=opt, weight_fn=weight_fn,
                       center_selection=FixedSelector(C.to(dev), idx_centers=torch.arange(700)))
        model.fit(Xg, Yg)
        fits.append(model.alpha_.clone())
    assert torch.equal(fits[0], fits[1])
