"""Backward pass of the kernel-vector product and of the kernel matrix on the MI355X (closed form on the library's
kernels, falkon_amd/mmv_ops/fmmv_grad.py) against what the reference computes: autograd through the kernel's core
function (oracle/grad_ref.py, following falkon/mmv_ops/fmmv.py:405-485 and falkon/mmv_ops/fmm.py:391-438), and
``torch.autograd.gradcheck`` as in the reference's own tests (falkon/tests/test_kernels.py:92-171,240-261).

Tolerances: gradients in fp64 within 1e-9, in fp32 within 1e-4 (relative, norm-wise per column) of the CPU result
in the same dtype; where the CPU fp32 gradient itself is further than that from its fp64 twin (the differences
x * sum_j W_ij - sum_j W_ij c_j cancel), the GPU gradient has to be as close to the fp64 one as the CPU's is.
"""
import numpy as np
import pytest
import torch

from falkon_amd import FalkonOptions, GaussianKernel, LaplacianKernel, MaternKernel
from oracle import grad_ref, inputs
from conftest import check_parity, rel_err

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.float64: 1e-9}
KERNELS = {
    "gaussian": lambda s: GaussianKernel(s),
    "laplacian": lambda s: LaplacianKernel(s),
    "1.5-matern": lambda s: MaternKernel(s, 1.5),
    "2.5-matern": lambda s: MaternKernel(s, 2.5),
}


def _data(n, m, d, t, dtype, seed, per_dim=False):
    g = np.random.default_rng(seed)
    np_dt = np.float32 if dtype == torch.float32 else np.float64
    mk = lambda *shape: torch.from_numpy(g.standard_normal(shape).astype(np_dt))     # noqa: E731
    sigma = torch.from_numpy(g.uniform(0.8, 1.3, d if per_dim else 1) * np.sqrt(d))
    return mk(n, d) + 0.5, mk(m, d) + 0.5, mk(m, t), sigma, mk(n, t)


def _gpu_grads(name, X1, X2, v, sigma, G, dev, needs=(True, True, True, True), data_dev=None):
    data_dev = dev if data_dev is None else data_dev
    leaves = [t.clone().to(data_dev).requires_grad_(n) for t, n in zip((X1, X2, v), needs[:3])]
    sg = sigma.clone().requires_grad_(needs[3])
    kernel = KERNELS[name](sg)
    out = kernel.mmv(*leaves)
    wanted = [t for t in leaves + list(kernel.diff_params.values()) if t.requires_grad]
    got = iter(torch.autograd.grad(out, wanted, grad_outputs=G.to(out.device)))
    return out, tuple(next(got) if n else None for n in needs)


@pytest.mark.parametrize("name", sorted(KERNELS))
@pytest.mark.parametrize("per_dim", [False, True])
def test_gradcheck_mmv_and_kernel_matrix(dev, name, per_dim):
    """The reference's own check (test_kernels.py:133-171) on its test matrices: n = 20, m = 5, d = 3, t = 2, fp64."""
    A, B, v, _ = inputs.reference_test_mats(20, 5, 3, 2, np.float64)
    m1, m2, vv = (t.to(dev).requires_grad_() for t in (A, B, v))
    sigma = (torch.tensor([3.0, 2.0, 4.0]) if per_dim else torch.tensor([3.0])).double().requires_grad_()
    kernel = KERNELS[name](sigma)
    assert torch.autograd.gradcheck(lambda a, b, c, *p: kernel.mmv(a, b, c),
                                    inputs=(m1, m2, vv, *kernel.diff_params.values()))
    assert torch.autograd.gradcheck(lambda a, b, *p: kernel(a, b), inputs=(m1, m2, *kernel.diff_params.values()))


def test_gradcheck_not_all_grads(dev):
    """falkon/tests/test_kernels.py:240-261: only X2 and sigma want gradients."""
    A, B, v, _ = inputs.reference_test_mats(20, 5, 3, 2, np.float64)
    m1, vv = A.to(dev), v.to(dev)
    m2 = B.to(dev).requires_grad_()
    kernel = GaussianKernel(torch.tensor([3.0], dtype=torch.float64).requires_grad_())
    assert torch.autograd.gradcheck(lambda a, b, *p: kernel(a, b), inputs=(m1, m2, *kernel.diff_params.values()))
    assert torch.autograd.gradcheck(lambda a, b, c, *p: kernel.mmv(a, b, c),
                                    inputs=(m1, m2, vv, *kernel.diff_params.values()))
    out = kernel.mmv(m1, m2, vv)
    g2, gs = torch.autograd.grad(out.sum(), [m2, kernel.sigma])
    assert g2.shape == m2.shape and gs.shape == kernel.sigma.shape and m1.grad is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("name", sorted(KERNELS))
@pytest.mark.parametrize("n,m,d,t,per_dim", [
    (300, 131, 28, 1, False), (257, 100, 9, 3, True),       # register-resident kernels: 29 and 10 columns per column of v
    (129, 70, 100, 2, False),                               # LDS-tiled kernel, 101 right-hand sides per column of v
])
def test_mmv_gradients_vs_oracle(dev, dtype, name, n, m, d, t, per_dim):
    X1, X2, v, sigma, G = _data(n, m, d, t, dtype, seed=n + d, per_dim=per_dim)
    out, got = _gpu_grads(name, X1, X2, v, sigma, G, dev)
    same = grad_ref.fmmv_grads_ref(X1, X2, v, sigma, G, name)
    wide = grad_ref.fmmv_grads_ref(X1.double(), X2.double(), v.double(), sigma, G.double(), name)
    for g_gpu, g_cpu, g_64, like in zip(got, same, wide, (X1, X2, v, sigma)):
        assert g_gpu.shape == like.shape and g_gpu.dtype == like.dtype
        check_parity(g_gpu.reshape(g_64.shape[0], -1), g_cpu.reshape(g_64.shape[0], -1),
                     g_64.reshape(g_64.shape[0], -1), TOL[dtype])
    # the forward value is the plain product
    plain = KERNELS[name](sigma).mmv(X1.to(dev), X2.to(dev), v.to(dev))
    assert torch.equal(out.detach(), plain)


@pytest.mark.parametrize("name", ["gaussian", "2.5-matern"])
def test_host_inputs_out_argument_and_subsets(dev, name):
    X1, X2, v, sigma, G = _data(400, 90, 12, 2, torch.float32, seed=4)
    _, full = _gpu_grads(name, X1, X2, v, sigma, G, dev)
    # data on the host: gradients come back on the host, same values
    _, host = _gpu_grads(name, X1, X2, v, sigma, G, dev, data_dev=torch.device("cpu"))
    for a, b in zip(full[:3], host[:3]):
        assert b.device.type == "cpu"
        assert rel_err(b, a) < 1e-6
    assert rel_err(host[3].reshape(-1, 1), full[3].reshape(-1, 1)) < 1e-5
    # only some inputs want gradients
    _, part = _gpu_grads(name, X1, X2, v, sigma, G, dev, needs=(True, False, False, True))
    assert part[1] is None and part[2] is None
    assert rel_err(part[0], full[0]) < 1e-6 and rel_err(part[3].reshape(-1, 1), full[3].reshape(-1, 1)) < 1e-6
    # `out` is written in place and carries the graph (falkon/tests/test_kernels.py:144-153)
    x1 = X1.to(dev).requires_grad_()
    kernel = KERNELS[name](sigma)
    buf = torch.empty(400, 2, dtype=torch.float32, device=dev)
    res = kernel.mmv(x1, X2.to(dev), v.to(dev), out=buf)
    assert res.data_ptr() == buf.data_ptr() and res.requires_grad
    (g1,) = torch.autograd.grad(res, [x1], grad_outputs=G.to(dev))
    assert rel_err(g1, full[0]) < 1e-6
    # dmmv has no backward pass (falkon/mmv_ops/fmmv.py:1028-1031)
    with pytest.raises(NotImplementedError):
        kernel.dmmv(x1, X2.to(dev), v.to(dev), None)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("name", sorted(KERNELS))
def test_kernel_matrix_gradients_vs_oracle(dev, dtype, name):
    X1, X2, _, sigma, _ = _data(210, 77, 15, 1, dtype, seed=8, per_dim=True)
    G = torch.from_numpy(np.random.default_rng(2).standard_normal((210, 77))).to(dtype)
    x1, x2 = X1.to(dev).requires_grad_(), X2.to(dev).requires_grad_()
    kernel = KERNELS[name](sigma.clone().requires_grad_())
    K = kernel(x1, x2, opt=FalkonOptions(no_single_kernel=False))
    got = torch.autograd.grad(K, [x1, x2, kernel.sigma], grad_outputs=G.to(dev))
    same = grad_ref.fmm_grads_ref(X1, X2, sigma, G, name)
    wide = grad_ref.fmm_grads_ref(X1.double(), X2.double(), sigma, G.double(), name)
    for g_gpu, g_cpu, g_64 in zip(got, same, wide):
        check_parity(g_gpu.reshape(g_64.shape[0], -1), g_cpu.reshape(g_64.shape[0], -1),
                     g_64.reshape(g_64.shape[0], -1), TOL[dtype])
    # the diagonal under autograd (stock torch ops): Gaussian of two different matrices
    if name == "gaussian":
        diag = kernel(x1[:77], x2, diag=True)
        (gd,) = torch.autograd.grad(diag.sum(), [x1])
        want = -((X1[:77].double() - X2.double()) / sigma ** 2) * torch.exp(
            -0.5 * (((X1[:77].double() - X2.double()) / sigma) ** 2).sum(-1, keepdim=True))
        assert rel_err(gd[:77], want) < 10 * TOL[dtype] and float(gd[77:].abs().max()) == 0.0


def test_config2_shape_reduced_gradients(dev):
    """Config 2's shape (d = 28, sigma = 3.8, fp32, T = 1, centres drawn from the data) at N = 20k, M = 2k: the
    lengthscale and centre gradients a hyper-parameter optimiser asks for."""
    X, C, sigma, v, w = inputs.make_config("C2", N=20_000, M=2_000)
    G = w[:, :1]
    _, got = _gpu_grads("gaussian", X, C, v, sigma, G, dev, needs=(False, True, True, True))
    wide = grad_ref.fmmv_grads_ref(X.double(), C.double(), v.double(), sigma, G.double(), "gaussian",
                                   needs=(False, True, True, True))
    same = grad_ref.fmmv_grads_ref(X, C, v, sigma, G, "gaussian", needs=(False, True, True, True))
    for g_gpu, g_cpu, g_64 in zip(got[1:], same[1:], wide[1:]):
        check_parity(g_gpu.reshape(g_64.shape[0], -1), g_cpu.reshape(g_64.shape[0], -1),
                     g_64.reshape(g_64.shape[0], -1), 1e-4)


@pytest.mark.parametrize("name", ["laplacian", "1.5-matern"])
def test_gradients_with_centres_from_the_data(dev, name):
    """Coincident points in fp32.  The Laplacian's derivative weight exp(-D)/D is unbounded there (its backward pass
    runs in fp64 for that reason); the GPU gradients must be at least as close to the fp64 ones as the CPU's."""
    X1, _, v, sigma, G = _data(3000, 500, 28, 1, torch.float32, seed=12)
    X2 = X1[:500].clone()
    _, got = _gpu_grads(name, X1, X2, v, sigma, G, dev)
    same = grad_ref.fmmv_grads_ref(X1, X2, v, sigma, G, name)
    wide = grad_ref.fmmv_grads_ref(X1.double(), X2.double(), v.double(), sigma, G.double(), name)
    for g_gpu, g_cpu, g_64 in zip(got, same, wide):
        shape = (g_64.shape[0], -1)
        assert torch.isfinite(g_gpu).all()
        assert rel_err(g_gpu.reshape(shape), g_64.reshape(shape)) <= max(1e-5, rel_err(g_cpu.reshape(shape), g_64.reshape(shape)))


def _hopt_data(dtype, n=1000, d=10):
    """The synthetic regression set of the reference's hyperparameter-optimisation tests
    (falkon/tests/test_hopt.py:31-50): linear targets with noise, standardised, 80 % for training."""
    g = torch.Generator().manual_seed(12)
    X = torch.randn((n, d), dtype=dtype, generator=g)
    Y = X @ torch.arange(d, dtype=dtype).reshape(-1, 1) + torch.randn((n, 1), dtype=dtype, generator=g) * 0.3
    ntr = int(n * 0.8)
    xm, xs, ym, ys = X[:ntr].mean(0, keepdim=True), X[:ntr].std(0, keepdim=True), Y[:ntr].mean(), Y[:ntr].std()
    X, Y = (X - xm) / xs, (Y - ym) / ys
    return X[:ntr], Y[:ntr], X[ntr:], Y[ntr:]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_gradient_descent_on_a_holdout_objective(dev, dtype):
    """What the backward pass is for (the reference's ``falkon.hopt`` objectives, e.g.
    falkon/hopt/objectives/exact_objectives/holdout.py:37-83): lengthscales (one per feature), centres and penalty
    are optimised by Adam on the hold-out error of the Nystroem estimator, every kernel matrix and its gradient
    coming from the MI355X kernels.  The hold-out error must drop, and so must the error on unseen data."""
    Xtr, Ytr, Xts, Yts = (a.to(dev) for a in _hopt_data(dtype))
    fit_idx, val_idx = torch.arange(0, 600, device=dev), torch.arange(600, 800, device=dev)
    kernel = GaussianKernel(torch.full((10,), 5.0, dtype=torch.float32).requires_grad_())
    centres = Xtr[:100].clone().requires_grad_()
    log_penalty = torch.tensor(np.log(1e-3), dtype=dtype, device=dev, requires_grad=True)

    def coefficients(Xf, Yf):
        kmn, kmm = kernel(centres, Xf), kernel(centres, centres)
        reg = torch.exp(log_penalty) * Xf.shape[0]
        lhs = kmn @ kmn.T + reg * kmm + 1e-6 * reg * torch.eye(100, dtype=dtype, device=dev)
        return torch.linalg.solve(lhs, kmn @ Yf)

    def holdout():
        alpha = coefficients(Xtr[fit_idx], Ytr[fit_idx])
        return torch.mean((Ytr[val_idx] - kernel(Xtr[val_idx], centres) @ alpha) ** 2)

    def test_error():
        with torch.no_grad():
            return float(torch.mean((Yts - kernel(Xts, centres) @ coefficients(Xtr, Ytr)) ** 2))

    optimiser = torch.optim.Adam([kernel.sigma, centres, log_penalty], lr=0.1)
    first, before = None, test_error()
    for _ in range(40):
        optimiser.zero_grad()
        loss = holdout()
        loss.backward()
        assert all(torch.isfinite(p.grad).all() for p in (kernel.sigma, centres, log_penalty))
        optimiser.step()
        first = float(loss.detach()) if first is None else first
    assert float(holdout().detach()) < 0.5 * first
    assert test_error() < 0.7 * before


def test_gradient_descent_through_the_kernel_vector_product(dev):
    """The same through ``kernel.mmv`` (K is never stored, forward or backward): lengthscale, centres and
    coefficients of ``f(x) = K(x, C) v`` are fitted to the training targets by Adam; the squared error must fall by
    an order of magnitude."""
    Xtr, Ytr, _, _ = (a.to(dev) for a in _hopt_data(torch.float32))
    kernel = GaussianKernel(torch.tensor([4.0]).requires_grad_())
    centres = Xtr[:64].clone().requires_grad_()
    v = torch.zeros(64, 1, device=dev, requires_grad=True)
    optimiser = torch.optim.Adam([kernel.sigma, centres, v], lr=0.05)
    losses = []
    for _ in range(150):
        optimiser.zero_grad()
        loss = torch.mean((kernel.mmv(Xtr, centres, v) - Ytr) ** 2)
        loss.backward()
        optimiser.step()
        losses.append(float(loss.detach()))
    assert losses[-1] < 0.1 * losses[0] and np.isfinite(losses).all()
