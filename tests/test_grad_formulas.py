"""The closed-form backward pass (falkon_amd/mmv_ops/fmmv_grad.py) checked on the CPU: the two library calls it is
built from are replaced by dense stand-ins that evaluate the same kernel functions from their definitions, so that
what is tested is the algebra (derivative kernels, weights, centring, the lengthscale identity), against autograd
through the reference's arithmetic (oracle/grad_ref.py).  The real kernels are tested on the GPU."""
import numpy as np
import pytest
import torch

from falkon_amd import _backend
from oracle import grad_ref

NAMES = {_backend.FLK_GAUSSIAN: "gaussian", _backend.FLK_LAPLACIAN: "laplacian",
         _backend.FLK_MATERN32: "1.5-matern", _backend.FLK_MATERN52: "2.5-matern"}


def _dense_kernel(Xa, Xb, sigma, kernel_fn):
    if kernel_fn == _backend.FLK_LAPLACIAN_DU:
        diff = (Xa[:, None, :] - Xb[None, :, :]) / sigma
        d2 = (diff * diff).sum(-1)
        dist = d2.clamp_min(1e-20).sqrt()
        return torch.where(d2 > 1e-20, torch.exp(-dist) / dist, torch.zeros_like(dist))
    return grad_ref.radial_kernel_difference_form(Xa, Xb, sigma, NAMES[kernel_fn])


@pytest.fixture()
def grad_module(monkeypatch):
    import importlib
    mod = importlib.import_module("falkon_amd.mmv_ops.fmmv_grad")

    def fmmv_stub(Xa, Xb, sigma_dev, rhs, out, kernel_fn=_backend.FLK_GAUSSIAN):
        out.copy_(_dense_kernel(Xa, Xb, sigma_dev, kernel_fn) @ rhs)

    def fmm_stub(Xa, Xb, sigma_dev, out, compute_f64, kernel_fn=_backend.FLK_GAUSSIAN):
        out.copy_(_dense_kernel(Xa, Xb, sigma_dev, kernel_fn))

    monkeypatch.setattr(mod, "gauss_fmmv_native", fmmv_stub)
    monkeypatch.setattr(mod, "gauss_fmm_native", fmm_stub)
    monkeypatch.setattr(mod, "_compute_device", lambda opt, devs: torch.device("cpu"))
    return mod


def _data(n, m, d, t, seed, per_dim):
    g = np.random.default_rng(seed)
    mk = lambda *s: torch.from_numpy(g.standard_normal(s))                       # noqa: E731
    sigma = torch.from_numpy(g.uniform(1.0, 2.5, d if per_dim else 1))
    return mk(n, d) + 3.0, mk(m, d) + 3.0, mk(m, t), sigma, mk(n, t)            # off-centre on purpose


@pytest.mark.parametrize("kernel_fn", sorted(NAMES))
@pytest.mark.parametrize("per_dim", [False, True])
@pytest.mark.parametrize("n,m,d,t", [(23, 11, 3, 2), (8, 30, 5, 1), (17, 17, 12, 60)])
def test_fmmv_backward_formulas(grad_module, kernel_fn, per_dim, n, m, d, t):
    X1, X2, v, sigma, G = _data(n, m, d, t, seed=n + d, per_dim=per_dim)
    want = grad_ref.fmmv_grads_ref(X1, X2, v, sigma, G, NAMES[kernel_fn])
    got = grad_module.fmmv_backward(kernel_fn, X1, X2, v, sigma, G, (True, True, True, True))
    for w, g_ in zip(want, got):
        assert g_.shape == w.shape
        assert float((g_ - w).abs().max()) <= 1e-10 * max(1.0, float(w.abs().max()))
    # a subset of the gradients: the others are not computed, the requested ones do not change
    only = grad_module.fmmv_backward(kernel_fn, X1, X2, v, sigma, G, (False, True, False, True))
    assert only[0] is None and only[2] is None
    torch.testing.assert_close(only[1], got[1], rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(only[3], got[3], rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("kernel_fn", sorted(NAMES))
@pytest.mark.parametrize("per_dim", [False, True])
def test_fmm_backward_formulas(grad_module, kernel_fn, per_dim):
    X1, X2, _, sigma, _ = _data(19, 14, 4, 1, seed=5, per_dim=per_dim)
    G = torch.from_numpy(np.random.default_rng(6).standard_normal((19, 14)))
    want = grad_ref.fmm_grads_ref(X1, X2, sigma, G, NAMES[kernel_fn])
    got = grad_module.fmm_backward(kernel_fn, X1, X2, sigma, G, (True, True, True))
    for w, g_ in zip(want, got):
        assert float((g_ - w).abs().max()) <= 1e-10 * max(1.0, float(w.abs().max()))


def test_coincident_points_have_no_laplacian_gradient(grad_module):
    """Centres that are data points: the reference's clamp stops the gradient of those pairs, the derivative
    weight is zero there, and nothing is infinite."""
    X1, _, v, sigma, G = _data(12, 5, 3, 2, seed=9, per_dim=False)
    X2 = X1[:5].clone()
    want = grad_ref.fmmv_grads_ref(X1, X2, v, sigma, G, "laplacian", kernel_fn=grad_ref.radial_kernel_difference_form)
    got = grad_module.fmmv_backward(_backend.FLK_LAPLACIAN, X1, X2, v, sigma, G, (True, True, True, True))
    for w, g_ in zip(want, got):
        assert torch.isfinite(g_).all()
        assert float((g_ - w).abs().max()) <= 1e-9 * max(1.0, float(w.abs().max()))
