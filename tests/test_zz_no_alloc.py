"""``flk_gauss_fdmmv_noalloc``: the entry point whose workspace is an array inside the library's device code.

It enqueues the kernels of ``flk_gauss_fdmmv`` on the built-in array instead of a caller's workspace, so its results
must equal that entry point's bit for bit, call after call, whatever the previous call left in the array.
"""
import numpy as np
import pytest
import torch

from conftest import rel_err
from oracle import mmv_ref

pytestmark = pytest.mark.gpu


def _inputs(n, m, d, t, dtype, seed, dev):
    g = np.random.default_rng(seed)
    X = torch.from_numpy(g.standard_normal((n, d))).to(dtype)
    C = X[torch.from_numpy(g.choice(n, m, replace=False))].clone()
    v = torch.from_numpy(g.standard_normal((m, t))).to(dtype)
    w = torch.from_numpy(g.standard_normal((n, t))).to(dtype)
    return tuple(a.to(dev) for a in (X, C, v, w))


def _call(lib, name, X, C, sigma, v, w, out, code, stream, workspace=None):
    n, d = X.shape
    m, t = v.shape
    args = [X.data_ptr(), n, X.stride(0), X.stride(1), C.data_ptr(), m, C.stride(0), C.stride(1), d,
            sigma.data_ptr(), sigma.numel(), v.data_ptr(), v.stride(0), v.stride(1),
            w.data_ptr() if w is not None else None, w.stride(0) if w is not None else 0,
            w.stride(1) if w is not None else 0, t, out.data_ptr(), out.stride(0), out.stride(1), code]
    if workspace is not None:
        args += [workspace.data_ptr(), workspace.numel()]
    return getattr(lib, name)(*args, stream)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, "bf16x3"])
def test_noalloc_equals_fdmmv_on_consecutive_calls(dev, dtype):
    """Two calls in a row, the second on a smaller problem (different blocking, the first call's packed operands and
    partial sums still in the array): each equals ``flk_gauss_fdmmv`` bit for bit and the CPU oracle to tolerance; no
    device memory is allocated through torch during the calls."""
    from falkon_amd import _backend
    lib = _backend.load()
    # "bf16x3": fp32 data with the cross term on the bf16 matrix cores (dtype code FLK_F32_BF16X3)
    code = {torch.float32: _backend.FLK_F32, torch.float64: _backend.FLK_F64, "bf16x3": _backend.FLK_F32_BF16X3}[dtype]
    dtype = torch.float32 if dtype == "bf16x3" else dtype
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    stream = torch.cuda.current_stream(dev).cuda_stream
    sigma = torch.tensor([2.5], dtype=dtype, device=dev)
    # (n, m, d, t, with w): register-resident kernel with several splits, then a smaller ragged problem, then the
    # LDS-tiled kernel (d > 64) and a many-column call, all sharing the one array
    cases = [(60_000, 3_000, 28, 1, True), (1_237, 301, 9, 3, False), (5_000, 700, 100, 2, True),
             (3_000, 500, 12, 40, True), (33, 7, 5, 1, True)]
    for i, (n, m, d, t, with_w) in enumerate(cases):
        X, C, v, w = _inputs(n, m, d, t, dtype, 100 + i, dev)
        w = w if with_w else None
        need = lib.flk_gauss_fdmmv_workspace_bytes(n, m, d, t, code)
        assert 0 < need <= _backend.NOALLOC_SCRATCH_BYTES
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        want = torch.empty(m, t, dtype=dtype, device=dev)
        got = torch.full((m, t), float("nan"), dtype=dtype, device=dev)
        rc = _call(lib, "flk_gauss_fdmmv", X, C, sigma, v, w, want, code, stream, ws)
        _backend.raise_for_status(rc, "flk_gauss_fdmmv")
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
        rc = _call(lib, "flk_gauss_fdmmv_noalloc", X, C, sigma, v, w, got, code, stream)
        _backend.raise_for_status(rc, "flk_gauss_fdmmv_noalloc")
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before
        assert torch.equal(got, want), f"case {i}: not bit-identical to flk_gauss_fdmmv"
        exp = mmv_ref.fdmmv_ref(X.cpu(), C.cpu(), v.cpu(), w.cpu() if w is not None else None, sigma.cpu())
        assert rel_err(got, exp) < tol, f"case {i}"


def test_noalloc_captured_into_a_graph_and_replayed(dev):
    """What the entry point is for: after one eager call (which looks the array's address up) the call is captured
    into a HIP graph and replayed several times with other work and synchronisations in between; every replay gives
    the eager result bit for bit, also after the inputs have changed in place."""
    from falkon_amd import _backend
    lib = _backend.load()
    code = _backend.FLK_F32
    sigma = torch.tensor([2.5], device=dev)
    X, C, v, w = _inputs(20_000, 1_500, 28, 2, torch.float32, 7, dev)
    want = torch.empty(1_500, 2, device=dev)
    got = torch.empty_like(want)
    eager = torch.cuda.current_stream(dev).cuda_stream
    _backend.raise_for_status(_call(lib, "flk_gauss_fdmmv_noalloc", X, C, sigma, v, w, want, code, eager), "eager call")
    torch.cuda.synchronize()
    side = torch.cuda.Stream(dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = _call(lib, "flk_gauss_fdmmv_noalloc", X, C, sigma, v, w, got, code, side.cuda_stream)
    _backend.raise_for_status(rc, "captured call")
    for rep in range(4):
        got.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {rep}"
        # other work of the program between the replays: a different problem through the same array, new inputs
        X2, C2, v2, w2 = _inputs(3_000, 200, 9, 1, torch.float32, 50 + rep, dev)
        tmp = torch.empty(200, 1, device=dev)
        _backend.raise_for_status(_call(lib, "flk_gauss_fdmmv_noalloc", X2, C2, sigma, v2, w2, tmp, code, eager), "between")
        v.mul_(1.25)
        _backend.raise_for_status(_call(lib, "flk_gauss_fdmmv_noalloc", X, C, sigma, v, w, want, code, eager), "eager call")
        torch.cuda.synchronize()


def test_noalloc_rejects_problems_beyond_the_array(dev):
    """A problem whose workspace exceeds the built-in array is refused with FLK_ENOMEM (MemoryError on the Python side)
    and a message that names both sizes; nothing is launched, the output is untouched."""
    from falkon_amd import _backend
    lib = _backend.load()
    n, m, d, t = 2_000_000, 1_000, 28, 1
    assert lib.flk_gauss_fdmmv_workspace_bytes(n, m, d, t, _backend.FLK_F32) > _backend.NOALLOC_SCRATCH_BYTES
    X = torch.zeros(n, d, device=dev)
    C = torch.zeros(m, d, device=dev)
    v = torch.zeros(m, t, device=dev)
    out = torch.full((m, t), 7.0, device=dev)
    sigma = torch.ones(1, device=dev)
    rc = _call(lib, "flk_gauss_fdmmv_noalloc", X, C, sigma, v, None, out, _backend.FLK_F32,
               torch.cuda.current_stream(dev).cuda_stream)
    assert rc == _backend.FLK_ENOMEM
    msg = _backend.last_error()
    assert str(_backend.NOALLOC_SCRATCH_BYTES) in msg and "scratch" in msg
    with pytest.raises(MemoryError):
        _backend.raise_for_status(rc, "flk_gauss_fdmmv_noalloc")
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())
