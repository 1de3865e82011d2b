"""Hyperparameter-optimisation objectives (falkon_amd/hopt) on the MI355X kernels.

Pinned against the definitions evaluated densely in fp64 with numpy (hat matrix H = K_nm (K_mn K_nm + v K_mm)^-1 K_mn
from brute-force kernel matrices; leave-one-out by actually refitting n times), not against the factorised formulas
the module uses; then the reference's own test (falkon/tests/test_hopt.py:31-70): Adam on every objective.
"""
import numpy as np
import pytest
import torch

from falkon_amd import GaussianKernel
from falkon_amd.hopt import GCV, LOOCV, SGPR, CompReg, HoldOut, NystromCompReg, PositiveTransform
from oracle import brute

pytestmark = pytest.mark.gpu


def _small_problem(dev, n=60, m=12, d=4, seed=3):
    g = np.random.default_rng(seed)
    X = torch.from_numpy(g.standard_normal((n, d)))
    Y = torch.from_numpy(np.sin(X.numpy() @ g.standard_normal((d, 1))) + 0.1 * g.standard_normal((n, 1)))
    C = X[:m].clone() + 0.05 * torch.from_numpy(g.standard_normal((m, d)))
    sigma = torch.tensor([1.5, 2.0, 2.5, 1.8], dtype=torch.float64)
    return X, Y, C, sigma, 1e-2


def _dense(X, Y, C, sigma, v, jitter=1e-8):
    """K_nm, K_mm (+ the module's first jitter), hat matrix and coefficients from the definitions."""
    Knm, Kmm = brute.gaussian_brute(X, C, sigma), brute.gaussian_brute(C, C, sigma) + jitter * np.eye(C.shape[0])
    inner = np.linalg.solve(Knm.T @ Knm + v * Kmm, Knm.T)
    return Knm, Kmm, Knm @ inner, inner @ Y.numpy()


def _build(cls, C, sigma, penalty, dev, **kw):
    kernel = GaussianKernel(sigma.clone().requires_grad_())
    return cls(kernel, C.clone().to(dev), torch.tensor(penalty, dtype=torch.float64, device=dev), True, True, **kw)


def test_positive_transform_round_trip():
    t = PositiveTransform(1e-8)
    y = torch.tensor([1e-7, 1e-5, 1e-3, 0.1, 1.0, 10.0, 50.0, 1e3], dtype=torch.float64)
    assert float(((t(t.inv(y)) - y) / y).abs().max()) < 1e-12
    assert float(t(torch.tensor(-1e3, dtype=torch.float64))) >= 1e-8


def test_objectives_match_their_definitions(dev):
    X, Y, C, sigma, penalty = _small_problem(dev)
    n, Yn = X.shape[0], Y.numpy()
    Xg, Yg = X.to(dev), Y.to(dev)
    v = penalty * n
    Knm, Kmm, H, alpha = _dense(X, Y, C, sigma, v)
    resid = Yn - H @ Yn

    got = _build(GCV, C, sigma, penalty, dev)(Xg, Yg).item()
    assert abs(got - np.mean(resid ** 2) / (1 - np.trace(H) / n) ** 2) < 1e-6 * abs(got)

    got = _build(CompReg, C, sigma, penalty, dev)(Xg, Yg).item()
    assert abs(got - (np.trace(H) + (Yn.T @ resid).item())) < 1e-6 * abs(got)

    Knn_trace = float(n)                                               # Gaussian kernel: unit diagonal
    Q = Knm @ np.linalg.solve(Kmm, Knm.T)
    data_fit = (Yn.T @ resid).item()
    want = np.trace(H) + data_fit + (Knn_trace - np.trace(Q)) * data_fit / (v * n)
    got = _build(NystromCompReg, C, sigma, penalty, dev)(Xg, Yg).item()
    assert abs(got - want) < 1e-5 * abs(want)

    cov = Q + v * np.eye(n)
    want = 0.5 * np.linalg.slogdet(cov)[1] + 0.5 * (Yn.T @ np.linalg.solve(cov, Yn)).item() + 0.5 * (Knn_trace - np.trace(Q)) / v
    got = _build(SGPR, C, sigma, penalty, dev)(Xg, Yg).item()
    assert abs(got - want) < 1e-5 * abs(want)

    # leave-one-out by refitting without each point in turn (variance penalty * (n - 1), as the closed form assumes)
    v1, errs = penalty * (n - 1), []
    for i in range(n):
        keep = np.arange(n) != i
        _, _, _, a = _dense(X[keep], Y[keep], C, sigma, v1)
        errs.append((Yn[i] - brute.gaussian_brute(X[i:i + 1], C, sigma) @ a).item() ** 2)
    got = _build(LOOCV, C, sigma, penalty, dev)(Xg, Yg).item()
    assert abs(got - np.mean(errs)) < 1e-5 * abs(got)

    model = _build(HoldOut, C, sigma, penalty, dev, val_pct=0.25, per_iter_split=False)
    got = model(Xg, Yg).item()
    tr, va = model.tr_indices.cpu().numpy(), model.val_indices.cpu().numpy()
    _, _, _, a = _dense(X[tr], Y[tr], C, sigma, penalty * len(tr))
    want = np.mean((Yn[va] - brute.gaussian_brute(X[va], C, sigma) @ a) ** 2)
    assert abs(got - want) < 1e-6 * abs(want)
    # predictions use the coefficients of the whole training set
    pred = model.predict(Xg[:7]).cpu().numpy()
    np.testing.assert_allclose(pred, Knm[:7] @ alpha, rtol=1e-6, atol=1e-9)


@pytest.mark.parametrize("cls", [CompReg, NystromCompReg, SGPR, GCV, LOOCV, HoldOut])
def test_reference_exact_objectives_optimise(dev, cls):
    """falkon/tests/test_hopt.py:31-70: 1000 synthetic points in 10 dimensions, 100 centres, lengthscales (one per
    feature), centres and penalty optimised by 50 Adam steps on each objective; the loss must stay finite and the
    error on the test points must end below that of the initial hyperparameters."""
    torch.manual_seed(12)
    n, d, dtype = 1000, 10, torch.float64
    X = torch.randn((n, d), dtype=dtype)
    Y = X @ torch.arange(d, dtype=dtype).reshape(-1, 1) + torch.randn((n, 1), dtype=dtype) * 0.3
    ntr = int(n * 0.8)
    xm, xs, ym, ys = X[:ntr].mean(0, keepdim=True), X[:ntr].std(0, keepdim=True), Y[:ntr].mean(), Y[:ntr].std()
    X, Y = ((X - xm) / xs).to(dev), ((Y - ym) / ys).to(dev)
    Xtr, Ytr, Xts, Yts = X[:ntr], Y[:ntr], X[ntr:], Y[ntr:]
    kernel = GaussianKernel(sigma=torch.tensor([5.0] * d, dtype=torch.float32, requires_grad=True))
    extra = dict(val_pct=0.8, per_iter_split=False) if cls is HoldOut else {}
    model = cls(kernel, Xtr[:100].clone(), torch.tensor(1e-5, dtype=dtype, device=dev), True, True, **extra)
    params = list(model.parameters())
    assert len(params) == 3 and any(p is kernel.sigma for p in params)
    optimiser = torch.optim.Adam(params, lr=0.1)
    model(Xtr, Ytr)
    before = float(torch.mean((model.predict(Xts) - Yts) ** 2))
    for _ in range(50):
        optimiser.zero_grad()
        loss = model(Xtr, Ytr)
        assert torch.isfinite(loss)
        loss.backward()
        optimiser.step()
    after = float(torch.mean((model.predict(Xts) - Yts) ** 2))
    assert np.isfinite(after) and after < max(before, 0.05)


def test_stochastic_objective_equals_the_exact_one_for_exact_traces(dev):
    """With the Hutchinson vectors replaced by sqrt(n) e_1 .. sqrt(n) e_n the trace estimates are exact, and with the
    solver run to convergence the matrix-free objective and its gradient (lengthscales, centres, penalty) must equal
    those of ``NystromCompReg``, whose gradient is plain autograd through the factorised formula."""
    from falkon_amd import FalkonOptions
    from falkon_amd.hopt import StochasticNystromCompReg
    X, Y, C, sigma, penalty = _small_problem(dev, n=80, m=10)
    Xg, Yg = X.to(dev), Y.to(dev)
    exact = _build(NystromCompReg, C, sigma, penalty, dev)
    stoch = _build(StochasticNystromCompReg, C, sigma, penalty, dev, flk_maxiter=300,
                   flk_opt=FalkonOptions(cg_tolerance=1e-13, pc_epsilon_64=1e-8, cg_full_gradient_every=5))
    stoch.trace_vectors = (np.sqrt(80.0) * torch.eye(80, dtype=torch.float64)).to(dev)
    values, grads = [], []
    for model in (exact, stoch):
        loss = model(Xg, Yg)
        loss.backward()
        values.append(loss.item())
        grads.append([model.kernel.sigma.grad.cpu(), model.centers_.grad.cpu(), model.penalty_.grad.cpu()])
    assert abs(values[0] - values[1]) < 1e-6 * abs(values[0])
    for a, b in zip(*grads):
        np.testing.assert_allclose(b.double().numpy(), a.double().numpy(), rtol=2e-4, atol=1e-6 * float(a.abs().max()))


def test_reference_stochastic_objective_optimises(dev):
    """falkon/tests/test_hopt.py:73-115: fp32, 100 centres, 10 trace vectors, 100 solver iterations to 1e-4; 60 Adam
    steps; the test error must end far below the reference's bound of 60 (targets are standardised)."""
    from falkon_amd import FalkonOptions
    from falkon_amd.hopt import StochasticNystromCompReg
    torch.manual_seed(12)
    n, d, dtype = 1000, 10, torch.float32
    X = torch.randn((n, d), dtype=dtype)
    Y = X @ torch.arange(d, dtype=dtype).reshape(-1, 1) + torch.randn((n, 1), dtype=dtype) * 0.1
    ntr = int(n * 0.8)
    xm, xs, ym, ys = X[:ntr].mean(0, keepdim=True), X[:ntr].std(0, keepdim=True), Y[:ntr].mean(), Y[:ntr].std()
    X, Y = ((X - xm) / xs).to(dev), ((Y - ym) / ys).to(dev)
    kernel = GaussianKernel(sigma=torch.tensor([5.0] * d, dtype=torch.float32, requires_grad=True))
    model = StochasticNystromCompReg(kernel, X[:100].clone(), torch.tensor(1e-1, dtype=dtype, device=dev), True, True,
                                     flk_opt=FalkonOptions(pc_epsilon_32=1e-4, cg_tolerance=1e-4), flk_maxiter=100,
                                     num_trace_est=10)
    optimiser = torch.optim.Adam(model.parameters(), lr=0.1)
    for _ in range(60):
        optimiser.zero_grad()
        loss = model(X[:ntr], Y[:ntr])
        assert torch.isfinite(loss)
        loss.backward()
        optimiser.step()
    ts_err = float(torch.mean((model.predict(X[ntr:]) - Y[ntr:]) ** 2))
    assert ts_err < 0.5
