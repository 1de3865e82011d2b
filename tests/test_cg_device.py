"""The device-resident conjugate-gradient iteration (``flk_cg_update``) and the solver built on it.

Checked against the same iteration written in torch ops on the host (``ConjugateGradient._solve_in_torch_ops``, the
restatement of falkon/optim/conjgrad.py:53-185), against the exact solution of dense systems, and, for the Falkon
solver, against the direct solution of the normal equations (falkon/tests/test_conjgrad.py:100-131).
"""
import numpy as np
import pytest
import torch

from conftest import rel_err
from falkon_amd import Falkon, FalkonOptions, GaussianKernel
from falkon_amd.center_selection import FixedSelector
from falkon_amd.optim import ConjugateGradient
from oracle import falkon_ref, inputs


def _spd(n, t, seed, dtype=torch.float64, cond_shift=None):
    g = np.random.default_rng(seed)
    Q = g.standard_normal((n, n))
    A = torch.from_numpy(Q @ Q.T + (cond_shift if cond_shift is not None else n) * np.eye(n)).to(dtype)
    B = torch.from_numpy(g.standard_normal((n, t))).to(dtype)
    return A, B


def test_differential_convergence_freezes_converged_columns_on_host():
    """Columns of very different difficulty: with differential convergence each column stops at the iterate at which
    its own residual fell below the tolerance (the value a single-column solve of it returns), without it all columns
    run until the last one has converged; both solve the system."""
    A, B = _spd(40, 3, seed=1)
    B[:, 0] = A[:, 3]                       # exact solution e_3: converges fast
    opt = FalkonOptions(cg_tolerance=1e-8, cg_differential_convergence=True)
    X = ConjugateGradient(opt).solve(None, B.clone(), lambda v: A @ v, max_iter=200)
    assert rel_err(A @ X, B) < 1e-7
    for c in range(3):
        alone = ConjugateGradient(FalkonOptions(cg_tolerance=1e-8)).solve(None, B[:, c:c + 1].clone(), lambda v: A @ v, 200)
        torch.testing.assert_close(X[:, c:c + 1], alone, rtol=1e-12, atol=1e-14)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("order", ["C", "F"])
@pytest.mark.parametrize("t", [1, 3])
def test_cg_update_kernel_is_one_reference_iteration(dev, dtype, order, t):
    """One call in mode 0, and the pair mode 1 + mode 2, against the reference's formulas evaluated in fp64."""
    from falkon_amd import _backend
    lib = _backend.load()
    code = _backend.FLK_F32 if dtype == torch.float32 else _backend.FLK_F64
    m = 5000 + 37
    g = torch.Generator().manual_seed(t)

    def mat():
        a = torch.randn(m, t, generator=g, dtype=torch.float64).to(dtype)
        a = torch.empty_strided((m, t), (1, m), dtype=dtype).copy_(a) if order == "F" else a
        return a.to(dev)

    X, R, P, Q, B = (mat() for _ in range(5))
    eps, tol2 = 1e-7, 1e-14
    rsold = (R.double() ** 2).sum(0).to(dtype)
    stream = torch.cuda.current_stream(dev).cuda_stream
    tol = 2e-6 if dtype == torch.float32 else 1e-14

    def call(mode, X, R, P, Q, rs, state, it):
        rc = lib.flk_cg_update(mode, X.data_ptr(), R.data_ptr(), P.data_ptr(), Q.data_ptr(), B.data_ptr(), m, t,
                               X.stride(0), X.stride(1), rs.data_ptr(), state.data_ptr(), it, eps, tol2, 0, code, stream)
        _backend.raise_for_status(rc, "flk_cg_update")

    # mode 0
    Xd, Rd, Pd, Qd, rso = X.double(), R.double(), P.double(), Q.double(), rsold.double()
    alpha = rso / ((Pd * Qd).sum(0) + eps)
    X_ref, R_ref = Xd + Pd * alpha, Rd - Qd * alpha
    rsn = (R_ref ** 2).sum(0)
    P_ref = R_ref + Pd * (rsn / (rso + eps))
    X0, R0, P0, rs0 = X.clone(), R.clone(), P.clone(), rsold.clone()
    state = torch.zeros(int(lib.flk_cg_state_ints(t)), dtype=torch.int32, device=dev)
    call(0, X0, R0, P0, Q, rs0, state, 0)
    assert rel_err(X0, X_ref) < tol and rel_err(R0, R_ref) < tol and rel_err(P0, P_ref) < tol
    assert rel_err(rs0.reshape(1, -1), rsn.reshape(1, -1)) < tol
    st = state.cpu()
    assert int(st[0]) == 0 and int(st[1]) == 1 and not bool(st[2:2 + 2 * t].any())
    # mode 1 then mode 2 (Q2 plays A X)
    Q2 = mat()
    X1, R1, P1, rs1 = X.clone(), R.clone(), P.clone(), rsold.clone()
    state.zero_()
    call(1, X1, R1, P1, Q, rs1, state, 3)
    assert rel_err(X1, X_ref) < tol and torch.equal(R1, R) and torch.equal(P1, P) and torch.equal(rs1, rsold)
    call(2, X1, R1, P1, Q2, rs1, state, 3)
    R2_ref = B.double() - Q2.double()
    rsn2 = (R2_ref ** 2).sum(0)
    P2_ref = R2_ref + Pd * (rsn2 / (rso + eps))
    assert rel_err(R1, R2_ref) < tol and rel_err(P1, P2_ref) < tol and rel_err(X1, X_ref) < tol
    assert int(state[1]) == 1


@pytest.mark.gpu
@pytest.mark.parametrize("graph", [False, True], ids=["eager", "graph"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_device_solver_equals_host_solver(dev, dtype, graph):
    """Dense SPD system, three right-hand sides: the GPU solve follows the host solve iterate for iterate (same number
    of iterations, same solution to rounding), stops when every column has converged although the host only looks at
    the flags every few iterations, and solves the system.  With the iterations replayed from HIP graphs as well."""
    A, B = _spd(300, 3, seed=2, dtype=dtype)
    opt = FalkonOptions(cg_tolerance=1e-4 if dtype == torch.float32 else 1e-9, cg_capture_graph=graph)
    host = ConjugateGradient(opt)
    Xh = host._solve_in_torch_ops(None, B.clone(), lambda v: A @ v, 200, None)
    Ag, Bg = A.to(dev), B.to(dev)
    devs = ConjugateGradient(opt)
    with torch.inference_mode():
        Xg = devs.solve(None, Bg.clone(), lambda v: Ag @ v, 200)
    assert devs.num_iter == host.num_iter and 3 < host.num_iter < 150
    assert rel_err(Xg, Xh) < (5e-4 if dtype == torch.float32 else 1e-9)
    assert rel_err(Ag @ Xg, Bg) < (1e-4 if dtype == torch.float32 else 1e-8)
    # the residual is recomputed from scratch every 10 iterations (mode 1 + 2): fewer iterations than that, and more
    for max_iter in (4, 25):
        Xh = host._solve_in_torch_ops(None, B.clone(), lambda v: A @ v, max_iter, None)
        with torch.inference_mode():
            Xg = devs.solve(None, Bg.clone(), lambda v: Ag @ v, max_iter)
        assert devs.num_iter == host.num_iter and (max_iter > 4 or host.num_iter == 3)
        assert rel_err(Xg, Xh) < (1e-4 if dtype == torch.float32 else 1e-10)


@pytest.mark.gpu
def test_device_solver_warm_start_callback_and_layouts(dev):
    """Warm start updates the given tensor in place (also an F-ordered one next to a C-ordered right-hand side), the
    callback sees every iteration's solution and can stop the solve, differential convergence freezes columns."""
    from falkon_amd.optim import StopOptimizationException
    A, B = _spd(200, 4, seed=3)
    Ag, Bg = A.to(dev), B.to(dev)
    opt = FalkonOptions(cg_tolerance=1e-9)
    exact = torch.linalg.solve(A, B)
    with torch.inference_mode():
        X0 = torch.zeros(4, 200, dtype=torch.float64, device=dev).T            # F-ordered start
        for _ in range(40):
            out = ConjugateGradient(opt).solve(X0, Bg, lambda v: Ag @ v, 5)
            assert out is X0
        assert rel_err(X0, exact) < 1e-8
        seen = []

        def cb(it, sol, elapsed):
            seen.append((it, sol.clone()))
            if it == 7:
                raise StopOptimizationException("enough")
        X = ConjugateGradient(opt).solve(None, Bg, lambda v: Ag @ v, 50, cb)
        assert [it for it, _ in seen] == list(range(1, 8)) and torch.equal(seen[-1][1], X)
        host = ConjugateGradient(opt)._solve_in_torch_ops(None, B.clone(), lambda v: A @ v, 7, None)
        assert rel_err(X, host) < 1e-10
        # differential convergence: as on the host, column by column
        B2 = B.clone()
        B2[:, 1] = A[:, 5]
        dopt = FalkonOptions(cg_tolerance=1e-8, cg_differential_convergence=True)
        Xd = ConjugateGradient(dopt).solve(None, B2.to(dev), lambda v: Ag @ v, 300)
        Xh = ConjugateGradient(dopt)._solve_in_torch_ops(None, B2.clone(), lambda v: A @ v, 300, None)
        assert rel_err(Xd, Xh) < 1e-9 and rel_err(Ag @ Xd, B2) < 1e-7


@pytest.mark.gpu
@pytest.mark.parametrize("graph", [False, True], ids=["eager", "graph"])
def test_falkon_solver_with_graph_replays_matches_direct_solve(dev, graph):
    """The reference's conjugate-gradient test (falkon/tests/test_conjgrad.py:100-131) with every iteration after the
    first replayed from a HIP graph (preconditioner solves + dfmmv + update in one graph per kind of iteration), one
    and ten right-hand sides, fp64 and fp32: the direct solution of the normal equations, and the eager solver's
    result."""
    X, Y, C, sigma, lam = _conjgrad_problem64()
    for Yk in (Y, torch.from_numpy(inputs.gen_random(500, 10, np.float64, seed=9))):
        opt = FalkonOptions(cg_tolerance=1e-10, cg_capture_graph=graph)
        model = Falkon(GaussianKernel(sigma), lam, M=10, center_selection=FixedSelector(C), maxiter=200, options=opt)
        model.fit(X.to(dev), Yk.to(dev))
        expected = falkon_ref.nystrom_krr_direct(X, Yk, C, sigma, lam)
        np.testing.assert_allclose(model.alpha_.cpu().numpy(), expected, rtol=1e-5)
    # a larger problem in fp32 whose preconditioner runs the blocked triangular solves, 20 iterations, against the CPU
    # pipeline; graph and eager agree to rounding
    n, m, d = 30_000, 4_500, 12
    g = np.random.default_rng(4)
    Xl = torch.from_numpy(g.standard_normal((n, d)).astype(np.float32))
    yl = torch.sign(torch.sin(Xl @ torch.from_numpy(g.standard_normal(d).astype(np.float32))).reshape(-1, 1))
    Cl = Xl[:m].clone()
    alphas = []
    for use in (graph, False):
        opt = FalkonOptions(cg_capture_graph=use)
        model = Falkon(GaussianKernel(2.5), 1e-6, M=m, center_selection=FixedSelector(Cl), maxiter=20, options=opt)
        model.fit(Xl.to(dev), yl.to(dev))
        alphas.append(model.predict(Xl[:2000].to(dev)).cpu())
    assert rel_err(alphas[0], alphas[1]) < 1e-4
    ref_alpha = falkon_ref.falkon_fit_ref(Xl, yl, Cl, 2.5, 1e-6, maxiter=20)
    ref_pred = falkon_ref.falkon_predict_ref(Xl[:2000], Cl, ref_alpha, 2.5)
    assert float(((alphas[0] - ref_pred) ** 2).mean() / (ref_pred ** 2).mean()) < 1e-3


def _conjgrad_problem64():
    N, M, D = 500, 10, 1000
    X = torch.from_numpy(inputs.gen_random(N, D, np.float64, F=False, seed=10))
    Y = torch.from_numpy(inputs.gen_random(N, 1, np.float64, F=False, seed=9))
    idx = np.random.default_rng(2).choice(N, M, replace=False)
    return X, Y, X[idx].clone(), 100.0, 10.0


@pytest.mark.gpu
def test_right_hand_sides_that_are_no_dense_matrix(dev):
    """Work buffers take the right-hand side's strides: an expanded view (columns aliasing each other) or a column
    slice of a wider matrix must be solved as a dense copy, column for column like their dense twins."""
    A, B = _spd(150, 3, seed=5)
    Ag = A.to(dev)
    opt = FalkonOptions(cg_tolerance=1e-9)
    one = B[:, :1].to(dev)
    expanded = one.expand(150, 3)
    assert expanded.stride() == (1, 0)
    wide = torch.zeros(150, 7, dtype=torch.float64, device=dev)
    wide[:, 2:5] = B.to(dev)
    sliced = wide[:, 2:5]
    assert not sliced.is_contiguous() and not sliced.T.is_contiguous()
    with torch.inference_mode():
        Xe = ConjugateGradient(opt).solve(None, expanded, lambda v: Ag @ v, 300)
        Xs = ConjugateGradient(opt).solve(None, sliced, lambda v: Ag @ v, 300)
    exact = torch.linalg.solve(A, B)
    assert rel_err(Xs, exact) < 1e-8
    assert rel_err(Xe, exact[:, :1].expand(150, 3)) < 1e-8
    assert wide[:, :2].abs().max() == 0 and wide[:, 5:].abs().max() == 0        # nothing written beside the slice


@pytest.mark.gpu
def test_graph_replay_with_a_callback(dev):
    """Graph replay together with a callback (the host then looks at the flags after every iteration): the callback
    sees the same iterates as in the eager solve, and the solution is the same."""
    A, B = _spd(250, 2, seed=6)
    Ag, Bg = A.to(dev), B.to(dev)
    seen = {}
    for graph in (False, True):
        opt = FalkonOptions(cg_tolerance=1e-9, cg_capture_graph=graph)
        trace = []
        with torch.inference_mode():
            X = ConjugateGradient(opt).solve(None, Bg.clone(), lambda v: Ag @ v, 60,
                                             callback=lambda it, sol, t: trace.append((it, sol.clone())))
        seen[graph] = (X, trace)
    (Xe, te), (Xg, tg) = seen[False], seen[True]
    assert len(te) == len(tg) > 5 and [i for i, _ in te] == [i for i, _ in tg]
    for (_, a), (_, b) in zip(te, tg):
        assert rel_err(b, a) < 1e-12
    assert rel_err(Xg, Xe) < 1e-12 and rel_err(Ag @ Xg, Bg) < 1e-8


@pytest.mark.gpu
def test_an_operator_that_cannot_be_captured_falls_back_to_eager_iterations():
    """An operator that waits for the device cannot be recorded into a graph: the solve warns, goes on eagerly and
    returns the eager result.  Run in a process of its own, so that a capture that fails cannot touch the state of the
    other tests' device context."""
    import subprocess
    import sys
    code = r'''
import warnings, numpy as np, torch
from falkon_amd import FalkonOptions
from falkon_amd.optim import ConjugateGradient
g = np.random.default_rng(8)
Q = g.standard_normal((120, 120))
A = torch.from_numpy(Q @ Q.T + 120 * np.eye(120)).cuda()
B = torch.from_numpy(g.standard_normal((120, 2))).cuda()
def waiting_operator(v):
    out = A @ v
    float(out[0, 0])            # a host wait: not allowed while a stream is capturing
    return out
with torch.inference_mode():
    want = ConjugateGradient(FalkonOptions(cg_tolerance=1e-9)).solve(None, B.clone(), lambda v: A @ v, 100)
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        got = ConjugateGradient(FalkonOptions(cg_tolerance=1e-9, cg_capture_graph=True)).solve(None, B.clone(), waiting_operator, 100)
torch.cuda.synchronize()
assert any("could not be captured" in str(w.message) for w in caught), [str(w.message) for w in caught]
err = float((got - want).norm() / want.norm())
assert err < 1e-10, err
print("fallback ok", err)
'''
    import os
    env = dict(os.environ, PYTHONPATH=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=240, env=env)
    assert res.returncode == 0 and "fallback ok" in res.stdout, res.stdout + res.stderr
