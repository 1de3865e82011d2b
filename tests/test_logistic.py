"""Logistic Falkon and its losses: the reference's tests (falkon/tests/test_gsc_losses.py:9-65,
falkon/tests/test_logistic_falkon.py:12-45) on this build's restatement, whose kernel products are the MI355X ``mmv``."""
import numpy as np
import pytest
import torch

from falkon_amd import GaussianKernel, LogisticFalkon
from falkon_amd.gsc_losses import LogisticLoss, WeightedCrossEntropyLoss


def _check_derivatives(closed_form, loss, pred, true):
    """Value, first and second derivative in ``pred`` against autograd through the textbook expression."""
    value = closed_form(true, pred)
    first = torch.autograd.grad(value.sum(), pred, create_graph=True)[0]
    second = torch.autograd.grad(first.sum(), pred)[0]
    p = pred.detach()
    np.testing.assert_allclose(loss(true, p).numpy(), value.detach().numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(loss.df(true, p).numpy(), first.detach().numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(loss.ddf(true, p).numpy(), second.numpy(), rtol=1e-10, atol=1e-12)


def test_logistic_loss_derivatives():
    pred = torch.linspace(-10, 10, 10, dtype=torch.float64).requires_grad_()
    true = torch.bernoulli(torch.full_like(pred, 0.5).detach(), generator=torch.Generator().manual_seed(1)) * 2 - 1
    _check_derivatives(lambda t, p: torch.log(1 + torch.exp(-t * p)), LogisticLoss(GaussianKernel(3)), pred, true)


@pytest.mark.parametrize("neg_weight", [1.0, 0.5])
def test_weighted_cross_entropy_derivatives(neg_weight):
    pred = torch.linspace(-10, 10, 10, dtype=torch.float64).requires_grad_()
    true = torch.bernoulli(torch.full_like(pred, 0.5).detach(), generator=torch.Generator().manual_seed(2))
    naive = lambda t, p: -(t * torch.log(torch.sigmoid(p)) + neg_weight * (1 - t) * torch.log(1 - torch.sigmoid(p)))  # noqa: E731
    _check_derivatives(naive, WeightedCrossEntropyLoss(GaussianKernel(3), neg_weight=neg_weight), pred, true)


def test_losses_do_not_overflow():
    loss = LogisticLoss(GaussianKernel(3))
    y, p = torch.tensor([1.0, -1.0]), torch.tensor([-1e4, -1e4])
    assert torch.isfinite(loss(y, p)).all() and torch.isfinite(loss.df(y, p)).all() and torch.isfinite(loss.ddf(y, p)).all()


def test_logistic_falkon_constructor_checks():
    with pytest.raises(ValueError, match="same length"):
        LogisticFalkon(GaussianKernel(3.0), [1e-1, 1e-3], [3], LogisticLoss(GaussianKernel(3.0)), M=10)


@pytest.mark.gpu
@pytest.mark.parametrize("incore", [False, True])
def test_reference_logistic_falkon(dev, incore, capsys):
    """falkon/tests/test_logistic_falkon.py:22-45: eight Newton steps on the sklearn classification set, training error
    below 0.1 %; and every Newton step lowers the regularised objective's loss term."""
    from sklearn import datasets
    X, Y = datasets.make_classification(1000, 10, n_classes=2, random_state=11)
    X, Y = torch.from_numpy(X.astype(np.float64)), torch.from_numpy(Y.astype(np.float64).reshape(-1, 1))
    Y[Y == 0] = -1
    if incore:
        X, Y = X.to(dev), Y.to(dev)
    kernel = GaussianKernel(3.0)

    def error_fn(t, p):
        return float(100 * torch.sum(t * p <= 0)) / t.shape[0], "c-err"

    model = LogisticFalkon(kernel=kernel, loss=LogisticLoss(kernel=kernel),
                           penalty_list=[1e-1, 1e-3, 1e-5, 1e-8, 1e-8, 1e-8, 1e-8, 1e-8],
                           iter_list=[3, 3, 3, 3, 8, 8, 8, 8], M=500, seed=10, error_fn=error_fn)
    model.fit(X, Y)
    preds = model.predict(X)
    assert preds.device == X.device and error_fn(preds, Y)[0] < 0.1
    losses = [float(line.split("training loss")[1].split()[0]) for line in capsys.readouterr().out.splitlines()
              if "training loss" in line]
    assert len(losses) == 8 and all(b < a for a, b in zip(losses, losses[1:]))
