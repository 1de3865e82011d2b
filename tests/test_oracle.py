"""Pins the CPU oracle (test infrastructure) before anything is checked against it.

Witnesses, all independent of the oracle's expanded-norm route:
  * ``oracle.brute``   closed form, fp64 difference form (numpy)
  * ``oracle.brute_c`` the same closed form in C with long-double accumulation
  * ``torch.cdist``    the reference's own naive oracle (falkon/tests/naive_kernels.py:23-25)
plus what the mathematics fixes: unit diagonal, sigma -> inf, adjoint identity, linearity,
one-hot vectors, blocked == unblocked, C order == F order.
"""
import numpy as np
import pytest
import torch

from oracle import brute, brute_c, gaussian_ref, grad_ref, inputs, mmv_ref


def _cdist_kernel(X, C, sigma):
    s = sigma.to(X.dtype) if isinstance(sigma, torch.Tensor) else sigma
    return torch.exp(-0.5 * torch.cdist(X / s, C / s, compute_mode="donot_use_mm_for_euclid_dist") ** 2)


@pytest.mark.parametrize("order", ["C", "F"])
@pytest.mark.parametrize("sigma", [torch.tensor([3.0]), torch.tensor([3.0, 3.0, 3.0]), torch.tensor([0.7, 2.0, 5.0])])
def test_rbf_core_reference_fixture(order, sigma):
    """n=20 m=5 d=3 fp64, seeds 92/93, rtol=atol=1e-8 (falkon/tests/test_kernels.py:32-35,75-89,304-319)."""
    A, B, _, _ = inputs.reference_test_mats(20, 5, 3, 2, np.float64, order)
    K = gaussian_ref.rbf_core_ref(A, B, None, sigma)
    np.testing.assert_allclose(K.numpy(), brute.gaussian_brute(A, B, sigma), rtol=1e-8, atol=1e-8)
    torch.testing.assert_close(K, _cdist_kernel(A, B, sigma), rtol=1e-8, atol=1e-8)
    out = torch.empty(20, 5, dtype=torch.float64)
    K2 = gaussian_ref.rbf_core_ref(A, B, out, sigma)
    assert K2.data_ptr() == out.data_ptr()
    torch.testing.assert_close(K2, K, rtol=0, atol=0)


def test_rbf_core_special_cases():
    g = np.random.default_rng(0)
    X = torch.from_numpy(g.standard_normal((50, 7)))
    K = gaussian_ref.rbf_core_ref(X, X, None, torch.tensor([1.3]))
    torch.testing.assert_close(torch.diagonal(K), torch.ones(50, dtype=torch.float64), rtol=0, atol=1e-12)
    torch.testing.assert_close(K, K.T, rtol=1e-13, atol=1e-13)
    assert float(K.max()) <= 1.0                     # clamp at 1e-20 keeps K <= 1
    Kinf = gaussian_ref.rbf_core_ref(X, X[:9], None, torch.tensor([1e9]))
    torch.testing.assert_close(Kinf, torch.ones(50, 9, dtype=torch.float64), rtol=0, atol=1e-12)
    # per-dimension sigma == isotropic sigma=1 on pre-divided data (distance_kernel.py:151-152)
    s = torch.from_numpy(g.uniform(0.5, 2.0, 7))
    torch.testing.assert_close(gaussian_ref.rbf_core_ref(X, X[:9], None, s),
                               gaussian_ref.rbf_core_ref(X / s, X[:9] / s, None, torch.tensor([1.0])),
                               rtol=1e-13, atol=1e-13)
    # a single far pair has a textbook value: |x-c|^2 = 4 d, sigma = 2 -> exp(-d/2)
    a, b = torch.ones(1, 6, dtype=torch.float64), -torch.ones(1, 6, dtype=torch.float64)
    assert abs(float(gaussian_ref.rbf_core_ref(a, b, None, torch.tensor([2.0]))) - np.exp(-3.0)) < 1e-15


def test_wrong_sigma_length_is_runtime_error():
    """falkon/tests/test_kernels.py:338-358."""
    A, B, v, _ = inputs.reference_test_mats(20, 5, 3, 2, np.float64)
    with pytest.raises(RuntimeError):
        mmv_ref.fmmv_ref(A, B, v, torch.tensor([2.0, 2.0], dtype=torch.float64))


def test_validate_sigma():
    assert gaussian_ref.validate_sigma_ref(3).dtype == torch.float64
    assert gaussian_ref.validate_sigma_ref(torch.ones(4, 1)).shape == (4,)
    with pytest.raises(ValueError):
        gaussian_ref.validate_sigma_ref(torch.ones(3, 3))
    with pytest.raises(TypeError):
        gaussian_ref.validate_sigma_ref(None)


@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-8), (np.float32, 1e-4)])
@pytest.mark.parametrize("n,m,d,t", [(20, 5, 3, 2), (1500, 250, 3, 2), (100, 250, 110, 2)])
def test_mmv_dmmv_against_both_brutes(dtype, tol, n, m, d, t):
    """Reference shapes (i)-(iii) (tests/test_kernels.py:32-35,529-535,594-601) and tolerances (:75-81)."""
    A, B, v, w = inputs.reference_test_mats(n, m, d, t, dtype)
    sigma = torch.tensor([3.0])
    mm = mmv_ref.fmmv_ref(A, B, v, sigma)
    dm = mmv_ref.fdmmv_ref(A, B, v, w, sigma)
    for ref_mm, ref_dm in ((brute.mmv_brute(A, B, sigma, v), brute.dmmv_brute(A, B, sigma, v, w)),
                           (brute_c.mmv_brute_c(A, B, sigma, v), brute_c.dmmv_brute_c(A, B, sigma, v, w))):
        np.testing.assert_allclose(mm.double().numpy(), ref_mm, rtol=tol, atol=tol)
        np.testing.assert_allclose(dm.double().numpy(), ref_dm, rtol=tol * max(1, n / 100), atol=tol * max(1, n / 100))
    assert mm.dtype == A.dtype and dm.dtype == A.dtype


def test_brutes_agree_and_have_closed_form_values():
    g = np.random.default_rng(3)
    X, C = g.standard_normal((40, 5)), g.standard_normal((30, 5))
    s = g.uniform(0.5, 2.0, 5)
    v, w = g.standard_normal((30, 3)), g.standard_normal((40, 3))
    np.testing.assert_allclose(brute.mmv_brute(X, C, s, v), brute_c.mmv_brute_c(X, C, s, v), rtol=1e-13, atol=1e-13)
    np.testing.assert_allclose(brute.dmmv_brute(X, C, s, v, w), brute_c.dmmv_brute_c(X, C, s, v, w), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(brute.dmmv_brute(X, C, s, None, w), brute_c.dmmv_brute_c(X, C, s, None, w), rtol=1e-12, atol=1e-12)
    # two points at distance 2 with sigma 1: K = exp(-2); mmv with v = [1] returns it
    out = brute_c.mmv_brute_c(np.array([[0.0, 0.0]]), np.array([[2.0, 0.0]]), np.array([1.0]), np.array([[1.0]]))
    assert abs(out[0, 0] - np.exp(-2.0)) < 1e-16


def test_mmv_algebraic_invariants():
    g = np.random.default_rng(11)
    X = torch.from_numpy(g.standard_normal((300, 6)))
    C = torch.from_numpy(g.standard_normal((70, 6)))
    v = torch.from_numpy(g.standard_normal((70, 3)))
    v2 = torch.from_numpy(g.standard_normal((70, 3)))
    w = torch.from_numpy(g.standard_normal((300, 3)))
    u = torch.from_numpy(g.standard_normal((300, 3)))
    s = torch.tensor([1.7])
    mm = lambda a, b, x: mmv_ref.fmmv_ref(a, b, x, s)
    # linearity, column independence, one-hot -> column of K
    torch.testing.assert_close(mm(X, C, 2 * v + v2), 2 * mm(X, C, v) + mm(X, C, v2), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(mm(X, C, v)[:, 1:2], mm(X, C, v[:, 1:2].contiguous()), rtol=1e-13, atol=1e-13)
    e = torch.zeros(70, 1, dtype=torch.float64); e[13] = 1
    torch.testing.assert_close(mm(X, C, e)[:, 0], gaussian_ref.rbf_core_ref(X, C, None, s)[:, 13], rtol=1e-13, atol=1e-13)
    # adjoint identity ties the two orientations together: u.T (K v) == (K.T u).T v
    lhs = (u * mm(X, C, v)).sum(0)
    rhs = (mm(C, X, u) * v).sum(0)
    torch.testing.assert_close(lhs, rhs, rtol=1e-11, atol=1e-11)
    # fdmmv == mmv(C, X, mmv(X, C, v) + w)   (falkon/kernels/keops_helpers.py:189-213)
    torch.testing.assert_close(mmv_ref.fdmmv_ref(X, C, v, w, s), mm(C, X, mm(X, C, v) + w), rtol=1e-11, atol=1e-11)
    torch.testing.assert_close(mmv_ref.fdmmv_ref(X, C, v, None, s), mm(C, X, mm(X, C, v)), rtol=1e-11, atol=1e-11)
    # row permutation of X permutes fmmv and leaves fdmmv unchanged
    p = torch.from_numpy(g.permutation(300))
    torch.testing.assert_close(mm(X[p], C, v), mm(X, C, v)[p], rtol=1e-13, atol=1e-13)
    torch.testing.assert_close(mmv_ref.fdmmv_ref(X[p], C, v, w[p], s), mmv_ref.fdmmv_ref(X, C, v, w, s), rtol=1e-11, atol=1e-11)


def test_blocked_equals_unblocked_and_orders():
    """A 1 MiB budget forces many blocks (reference TestLargeComputations, tests/test_kernels.py:529-573)."""
    A, B, v, w = inputs.reference_test_mats(1500, 250, 3, 2, np.float32)
    s = torch.tensor([3.0])
    budget = 2**20 + mmv_ref.EXTRA_MM_RAM_BYTES
    bn, bm, _ = mmv_ref.mmv_blk_sizes_ref(1500, 3, 250, 2, budget / 4, torch.float32)
    assert bn < 1500 or bm < 250
    torch.testing.assert_close(mmv_ref.fmmv_ref(A, B, v, s, max_cpu_mem=budget), mmv_ref.fmmv_ref(A, B, v, s), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(mmv_ref.fdmmv_ref(A, B, v, w, s, max_cpu_mem=budget), mmv_ref.fdmmv_ref(A, B, v, w, s), rtol=1e-4, atol=1e-4)
    Af, Bf, vf, wf = inputs.reference_test_mats(1500, 250, 3, 2, np.float32, "F")
    of = mmv_ref.fmmv_ref(Af, Bf, vf, s)
    assert of.stride(0) == 1                      # output follows X1's order (mmv_ops/utils.py:124-155)
    torch.testing.assert_close(of, mmv_ref.fmmv_ref(A, B, v, s), rtol=1e-5, atol=1e-5)
    out = torch.empty(250, 2)
    res = mmv_ref.fdmmv_ref(A, B, v, w, s, out=out)
    assert res.data_ptr() == out.data_ptr()


@pytest.mark.parametrize("avail", [2.8e6, 3.5e6, 4e6, 5e7, 1e9])
def test_block_solvers_respect_budget(avail):
    """Properties of falkon/tests/test_dim_selectors.py:12-90: never over budget, never over the maxima."""
    n, d, m, t = 100_000, 28, 20_000, 3
    extra0 = mmv_ref.EXTRA_MM_RAM_BYTES / 4
    bn = mmv_ref.dmmv_blk_sizes_ref(n, d, m, t, avail, torch.float32)[0]
    assert 1 <= bn <= n
    assert bn * (m + d + t + 1) + m * d + m + extra0 <= avail
    bn, bm, _ = mmv_ref.mmv_blk_sizes_ref(n, d, m, t, avail, torch.float32)
    assert 1 <= bn <= n and 1 <= bm <= m
    assert bn * bm + bn * (d + 1) + bm * (d + 1) + extra0 <= avail * (1 + 1e-9)
    with pytest.raises(MemoryError):
        mmv_ref.dmmv_blk_sizes_ref(n, d, m, t, extra0, torch.float32)


def test_errors_match_reference_types():
    A, B, v, w = inputs.reference_test_mats(20, 5, 3, 2, np.float64)
    s = torch.tensor([3.0])
    with pytest.raises(ValueError):
        mmv_ref.fmmv_ref(A[None], B, v, s)
    with pytest.raises(ValueError):
        mmv_ref.fmmv_ref(A, B, v[:4], s)
    with pytest.raises(TypeError):
        mmv_ref.fmmv_ref(A, B.float(), v, s)
    big = torch.zeros(40, 6, dtype=torch.float64)[::2, ::2]          # no unit stride
    with pytest.raises(ValueError):
        mmv_ref.fmmv_ref(big, B, v, s)
    with pytest.raises(ValueError):
        mmv_ref.fdmmv_ref(A, B, v, w, s, out=torch.empty(4, 2, dtype=torch.float64))


def test_config_generators_are_seeded():
    X, C, sigma, v, w = inputs.make_config("C2", N=2000, M=100)
    X2, C2, _, v2, w2 = inputs.make_config("C2", N=2000, M=100)
    assert torch.equal(X, X2) and torch.equal(C, C2) and torch.equal(v, v2) and torch.equal(w, w2)
    assert X.dtype == torch.float32 and X.shape == (2000, 28) and C.shape == (100, 28) and w.shape == (2000, 1)
    assert float(sigma) == 3.8
    X, C, sigma, v, w = inputs.make_config("C3", N=1000, M=50)
    assert sigma.shape == (9,) and w is None and float(X.abs().max()) <= 1.0
    X, C, sigma, v, w = inputs.make_config("C4", N=300, M=20)
    assert X.shape == (300, 784) and v.shape == (20, 10) and 0.1 < float((X != 0).float().mean()) < 0.3
    X, C, sigma, v, w = inputs.make_config("C1", N=500, M=20)
    assert X.dtype == torch.float64 and w is None


# --------------------------------------------------------------------------------------------------
# Laplacian and Matern cores (falkon/kernels/distance_kernel.py:182-269)
# --------------------------------------------------------------------------------------------------
KERNEL_NAMES = ("laplacian", "0.5-matern", "1.5-matern", "2.5-matern", "inf-matern")


def _cdist_radial(X, C, sigma, name):
    """The reference's naive oracles (falkon/tests/naive_kernels.py:28-31,48-61) on torch.cdist distances."""
    s = sigma.to(X.dtype)
    D = torch.cdist(X / s, C / s, compute_mode="donot_use_mm_for_euclid_dist")
    if name in ("laplacian", "0.5-matern"):
        return torch.exp(-D)
    if name == "1.5-matern":
        return (1.0 + D * 3 ** 0.5) * torch.exp(-D * 3 ** 0.5)
    if name == "2.5-matern":
        S = D * 5 ** 0.5
        return (1.0 + S + S ** 2 / 3.0) * torch.exp(-S)
    return torch.exp(-D ** 2 / 2.0)


@pytest.mark.parametrize("name", KERNEL_NAMES)
@pytest.mark.parametrize("sigma", [torch.tensor([3.0]), torch.tensor([0.7, 2.0, 5.0])])
def test_radial_cores_reference_fixture(name, sigma):
    """The reference's kernel-test shape (n=20 m=5 d=3 fp64, seeds 92/93, falkon/tests/test_kernels.py:32-35,75-89)
    against the closed forms in difference form (numpy) and on torch.cdist, rtol = atol = 1e-8."""
    A, B, _, _ = inputs.reference_test_mats(20, 5, 3, 2, np.float64, "C")
    core = gaussian_ref.core_ref_for(name)
    K = core(A, B, None, sigma)
    np.testing.assert_allclose(K.numpy(), brute.radial_brute(A, B, sigma, name), rtol=1e-8, atol=1e-8)
    torch.testing.assert_close(K, _cdist_radial(A, B, sigma, name), rtol=1e-8, atol=1e-8)
    out = torch.empty(20, 5, dtype=torch.float64)
    assert core(A, B, out, sigma).data_ptr() == out.data_ptr()
    torch.testing.assert_close(out, K, rtol=0, atol=0)


def test_radial_cores_special_cases():
    g = np.random.default_rng(4)
    X = torch.from_numpy(g.standard_normal((30, 6)))
    C = torch.from_numpy(g.standard_normal((12, 6)))
    sig = torch.tensor([1.7], dtype=torch.float64)
    lap = gaussian_ref.laplacian_core_ref(X, C, None, sig)
    # nu = 1/2 is the Laplacian and nu = inf the Gaussian (falkon/kernels/distance_kernel.py:235-238)
    torch.testing.assert_close(gaussian_ref.matern_core_ref(X, C, None, sig, 0.5), lap, rtol=0, atol=0)
    torch.testing.assert_close(gaussian_ref.matern_core_ref(X, C, None, sig, float("inf")),
                               gaussian_ref.rbf_core_ref(X, C, None, sig), rtol=0, atol=0)
    # textbook form of the Laplacian on a single pair
    d01 = float(((X[0] - C[1]) / 1.7).norm())
    assert abs(float(lap[0, 1]) - np.exp(-d01)) < 1e-12
    for nu in (0.5, 1.5, 2.5):
        K = gaussian_ref.matern_core_ref(X, C, None, sig, nu)
        assert float(K.max()) <= 1.0 and float(K.min()) > 0.0
        # coincident points: K = 1 up to the clamp of the squared distance at 1e-20 and the sqrt of rounding noise
        Kxx = gaussian_ref.matern_core_ref(X, X, None, sig, nu)
        assert float((Kxx.diagonal() - 1).abs().max()) < 1e-6
        # smoother kernels decay more slowly near zero distance: at small D, 1 - K ~ D, D^2 * 3/2 ... ordering at D -> 0
    near = X[:1] + 1e-3
    k05, k15, k25 = (float(gaussian_ref.matern_core_ref(X[:1], near, None, sig, nu)) for nu in (0.5, 1.5, 2.5))
    assert k05 < k15 < k25 < 1.0
    # per-dimension lengthscales are a rescaling of the inputs
    per_dim = torch.tensor([0.5, 1.0, 1.5, 2.0, 2.5, 3.0], dtype=torch.float64)
    one = torch.tensor([1.0])
    for name in KERNEL_NAMES:
        core = gaussian_ref.core_ref_for(name)
        torch.testing.assert_close(core(X, C, None, per_dim), core(X / per_dim, C / per_dim, None, one),
                                   rtol=1e-12, atol=1e-14)
    with pytest.raises(ValueError):
        gaussian_ref.matern_core_ref(X, C, None, sig, 3.5)


@pytest.mark.parametrize("name", KERNEL_NAMES)
def test_radial_products_against_brute(name):
    """fmmv / fdmmv of the block loops with another kernel's core against K from the closed form."""
    g = np.random.default_rng(9)
    X = torch.from_numpy(g.standard_normal((150, 7)))
    C = torch.from_numpy(g.standard_normal((40, 7)))
    v = torch.from_numpy(g.standard_normal((40, 3)))
    w = torch.from_numpy(g.standard_normal((150, 3)))
    sig = torch.tensor([2.2], dtype=torch.float64)
    K = brute.radial_brute(X, C, sig, name)
    np.testing.assert_allclose(mmv_ref.fmmv_ref(X, C, v, sig, kernel_name=name, max_cpu_mem=2**24).numpy(),
                               K @ v.numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(mmv_ref.fdmmv_ref(X, C, v, w, sig, kernel_name=name, max_cpu_mem=2**24).numpy(),
                               K.T @ (K @ v.numpy() + w.numpy()), rtol=1e-10, atol=1e-12)


# ---- gradients (oracle/grad_ref.py) -------------------------------------------------------------------
def _grad_case(per_dim: bool, seed: int = 21, n: int = 14, m: int = 9, d: int = 4, t: int = 2):
    g = np.random.default_rng(seed)
    mk = lambda *s: torch.from_numpy(g.standard_normal(s))                        # noqa: E731
    sigma = torch.from_numpy(g.uniform(1.0, 2.0, d if per_dim else 1))
    return mk(n, d), mk(m, d), mk(m, t), sigma, mk(n, t)


@pytest.mark.parametrize("name", KERNEL_NAMES)
def test_autograd_restatement_is_the_core(name):
    """The out-of-place graph evaluates to what the in-place core functions give."""
    X, C, _, sigma, _ = _grad_case(per_dim=True)
    torch.testing.assert_close(grad_ref.radial_kernel_autograd(X, C, sigma, name),
                               gaussian_ref.core_ref_for(name)(X, C, None, sigma), rtol=1e-14, atol=1e-15)
    torch.testing.assert_close(grad_ref.radial_kernel_difference_form(X, C, sigma, name),
                               torch.from_numpy(brute.radial_brute(X, C, sigma, name)), rtol=1e-13, atol=1e-15)


@pytest.mark.parametrize("name", KERNEL_NAMES)
@pytest.mark.parametrize("per_dim", [False, True])
def test_gradients_against_difference_form_and_finite_differences(name, per_dim):
    X, C, v, sigma, G = _grad_case(per_dim)
    got = grad_ref.fmmv_grads_ref(X, C, v, sigma, G, name)
    exact = grad_ref.fmmv_grads_ref(X, C, v, sigma, G, name, kernel_fn=grad_ref.radial_kernel_difference_form)
    for a, b in zip(got, exact):
        torch.testing.assert_close(a, b, rtol=1e-9, atol=1e-11)

    # central differences of L = sum(G * (K v)) built on the closed form, a few coordinates of every input
    def loss(x, c, vv, sg):
        return float((G.numpy() * (brute.radial_brute(x, c, sg, name) @ vv.numpy())).sum())

    h = 1e-6
    args = [X, C, v, sigma]
    for which, grad in enumerate(got):
        flat = grad.reshape(-1)
        for idx in range(0, flat.numel(), max(1, flat.numel() // 5)):
            up = [a.clone() for a in args]
            dn = [a.clone() for a in args]
            up[which].view(-1)[idx] += h
            dn[which].view(-1)[idx] -= h
            fd = (loss(*up) - loss(*dn)) / (2 * h)
            assert abs(fd - float(flat[idx])) <= 1e-6 * max(1.0, abs(fd)), (which, idx)
    # the kernel matrix: L = sum(G2 * K)
    G2 = torch.from_numpy(np.random.default_rng(3).standard_normal((X.shape[0], C.shape[0])))
    got_mm = grad_ref.fmm_grads_ref(X, C, sigma, G2, name)
    exact_mm = grad_ref.fmm_grads_ref(X, C, sigma, G2, name, kernel_fn=grad_ref.radial_kernel_difference_form)
    for a, b in zip(got_mm, exact_mm):
        torch.testing.assert_close(a, b, rtol=1e-9, atol=1e-11)
    # K @ v with v = e_j and G = e_i picks the gradient of a single kernel entry: same as the matrix form
    E = torch.zeros_like(G2)
    E[2, 3] = 1.0
    vj = torch.zeros((C.shape[0], 1), dtype=torch.float64)
    vj[3] = 1.0
    Gi = torch.zeros((X.shape[0], 1), dtype=torch.float64)
    Gi[2] = 1.0
    one_mm = grad_ref.fmm_grads_ref(X, C, sigma, E, name)
    one_mv = grad_ref.fmmv_grads_ref(X, C, vj, sigma, Gi, name)
    for a, b in zip(one_mm, (one_mv[0], one_mv[1], one_mv[3])):
        torch.testing.assert_close(a, b, rtol=1e-12, atol=1e-14)
