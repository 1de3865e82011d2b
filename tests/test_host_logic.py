"""Host-side behaviour that needs no GPU: the C ABI surface, argument validation, options."""
import ctypes
import dataclasses
import os
import re

import numpy as np
import pytest
import torch

import falkon_amd
from falkon_amd import FalkonOptions, GaussianKernel, _backend
from falkon_amd.kernels.distance_kernel import validate_sigma
from falkon_amd.utils.tensor_helpers import create_same_stride, is_contig, is_f_contig

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "falkon_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(flk_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_backend.library_path()) if os.path.exists(_backend.library_path()) else _backend.load()
    names = _declared_symbols()
    assert len(names) >= 10
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/falkon_amd.h but not exported"
    assert set(names) == set(_backend._SIGNATURES), "ctypes signature table and header disagree"


def test_size_queries_need_no_gpu():
    lib = _backend.load()
    assert lib.flk_version() >= 100
    assert lib.flk_max_d(_backend.FLK_F32) >= 28 and lib.flk_max_d(_backend.FLK_F64) >= 28
    # packed fp32: 32-row blocks, features padded to a multiple of 2, plus half norms, 256-byte aligned parts
    assert lib.flk_gauss_packed_bytes(33, 3, _backend.FLK_F32) == 2 * 4 * 32 * 4 + 256
    assert lib.flk_gauss_packed_bytes(16, 5, _backend.FLK_F64) == 8 * 16 * 8 + 256
    small = lib.flk_gauss_fdmmv_workspace_bytes(1000, 100, 8, 1, _backend.FLK_F32)
    big = lib.flk_gauss_fdmmv_workspace_bytes(100000, 100, 8, 1, _backend.FLK_F32)
    assert 0 < small < big
    # config 2 stays far below 288 GB: nothing of size N x M is ever allocated
    assert lib.flk_gauss_fdmmv_workspace_bytes(1_000_000, 20_000, 28, 1, _backend.FLK_F32) < 512 * 2**20
    # what no call would accept has no size: negative shapes, unknown dtypes, shapes beyond the published limits
    too_wide, too_many = lib.flk_max_d(_backend.FLK_F32) + 1, lib.flk_max_t() + 1
    for query in (lib.flk_gauss_fmmv_workspace_bytes, lib.flk_gauss_fdmmv_workspace_bytes,
                  lib.flk_gauss_mmv_packed_workspace_bytes):
        assert query(100, 10, 3, 1, _backend.FLK_F32) > 0
        assert query(-1, 10, 3, 1, _backend.FLK_F32) == 0
        assert query(100, 10, 3, 1, 7) == 0
        assert query(100, 10, too_wide, 1, _backend.FLK_F32) == 0
        assert query(100, 10, 3, too_many, _backend.FLK_F32) == 0
    assert lib.flk_gauss_packed_bytes(10, 3, 7) == 0 and lib.flk_gauss_packed_bytes(10, too_wide, _backend.FLK_F32) == 0
    assert lib.flk_gauss_fmmv_workspace_bytes(100, 10, 3, 1, _backend.FLK_F32_BF16X3) > 0
    # the bf16x3 code belongs to the product entry points and the kernel matrix, not to the packed entry points
    assert lib.flk_gauss_mmv_packed_workspace_bytes(100, 10, 3, 1, _backend.FLK_F32_BF16X3) == 0
    # kernel matrix: the code has operands of its own beyond 64 features in fp32 arithmetic (three bfloat16 planes per
    # 16-feature step, 32-row blocks, fp32 half norms), and asks for what FLK_F32 asks otherwise
    fmm = lib.flk_gauss_fmm_workspace_bytes
    a256 = lambda b: (b + 255) // 256 * 256
    split_operand = lambda n, d: a256((n + 31) // 32 * ((d + 2 + 15) // 16) * 3 * 64 * 16) + a256((n + 31) // 32 * 32 * 4)
    assert fmm(1000, 300, 100, _backend.FLK_F32_BF16X3, 0) == split_operand(1000, 100) + split_operand(300, 100)
    assert fmm(1000, 300, 100, _backend.FLK_F32_BF16X3, 1) == fmm(1000, 300, 100, _backend.FLK_F32, 1)
    assert fmm(1000, 300, 64, _backend.FLK_F32_BF16X3, 0) == fmm(1000, 300, 64, _backend.FLK_F32, 0)
    assert fmm(1000, 300, 100, 7, 0) == 0 and fmm(-1, 300, 100, _backend.FLK_F32, 0) == 0


def test_bad_arguments_rejected_on_host_before_any_launch():
    lib = _backend.load()
    rc = lib.flk_gauss_pack(None, 10, 3, 3, 1, None, 1, _backend.FLK_F32, None, 0, None)
    assert rc == _backend.FLK_EINVAL and "null" in _backend.last_error()
    rc = lib.flk_gauss_pack(4096, 10, 3, 3, 1, 4096, 2, _backend.FLK_F32, 4096, 1 << 20, None)
    assert rc == _backend.FLK_EINVAL and "sigma" in _backend.last_error()
    rc = lib.flk_gauss_pack(4096, 10, 3, 6, 2, 4096, 1, _backend.FLK_F32, 4096, 1 << 20, None)
    assert rc == _backend.FLK_EINVAL and "stride" in _backend.last_error()
    rc = lib.flk_gauss_pack(4096, 10, 3, 3, 1, 4096, 1, 7, 4096, 1 << 20, None)
    assert rc == _backend.FLK_EINVAL
    too_wide = lib.flk_max_d(_backend.FLK_F32) + 1
    rc = lib.flk_gauss_fmmv(4096, 10, too_wide, 1, 4096, 5, too_wide, 1, too_wide, 4096, 1, 4096, 1, 1, 1, 4096, 1, 1,
                            _backend.FLK_F32, 4096, 1 << 20, None)
    assert rc == _backend.FLK_EUNSUPPORTED and "features" in _backend.last_error()
    rc = lib.flk_gauss_fmmv(4096, 10, 3, 1, 4096, 5, 3, 1, 3, 4096, 1, 4096, 1, 1, 1, 4096, 1, 1, _backend.FLK_F32,
                            4096, 16, None)
    assert rc == _backend.FLK_ENOMEM
    with pytest.raises(MemoryError):
        _backend.raise_for_status(rc, "flk_gauss_fmmv")
    rc = lib.flk_gauss_fdmmv(4096, 10, 3, 1, 4096, 5, 3, 1, 3, 4096, 1, None, 1, 1, None, 0, 0, 1, 4096, 1, 1,
                             _backend.FLK_F32, 4096, 1 << 30, None)
    assert rc == _backend.FLK_EINVAL and "v" in _backend.last_error()


def test_validate_sigma_and_kernel_object():
    assert validate_sigma(2).dtype == torch.float64 and validate_sigma(2).shape == (1,)
    assert validate_sigma(torch.ones(5, 1)).shape == (5,)
    with pytest.raises(ValueError):
        validate_sigma(torch.ones(2, 2))
    with pytest.raises(TypeError):
        validate_sigma(None)
    k = GaussianKernel(torch.tensor([1.0, 2.0]))
    assert list(k.diff_params) == ["sigma"] and not k.sigma.requires_grad
    assert k.kernel_name == "gaussian" and "GaussianKernel" in repr(k)
    assert isinstance(k.detach(), GaussianKernel)
    # compute() is the explicit kernel block (not on the mmv path) and follows the closed form
    X, C = torch.randn(6, 2, dtype=torch.float64), torch.randn(4, 2, dtype=torch.float64)
    K = k.compute(X, C, torch.empty(6, 4, dtype=torch.float64), diag=False)
    s = torch.tensor([1.0, 2.0], dtype=torch.float64)
    torch.testing.assert_close(K, torch.exp(-0.5 * torch.cdist(X / s, C / s) ** 2), rtol=1e-10, atol=1e-12)


def test_sigma_copy_follows_writes_through_data():
    """The copy of sigma the kernels read is refreshed when sigma's values change, also through ``sigma.data``,
    which leaves the tensor's version counter alone (manual hyper-parameter updates do that)."""
    cpu = torch.device("cpu")
    k = GaussianKernel(torch.tensor([1.0, 2.0, 3.0]))
    first = k._sigma_on(cpu, torch.float32)
    assert first.dtype == torch.float32 and first.tolist() == [1.0, 2.0, 3.0]
    assert k._sigma_on(cpu, torch.float32) is first                    # unchanged values: the same copy
    version = k.sigma._version
    k.sigma.data.mul_(2.0)
    assert k.sigma._version == version                                 # invisible to the version counter
    assert k._sigma_on(cpu, torch.float32).tolist() == [2.0, 4.0, 6.0]
    k.sigma.data.fill_(5.0)
    assert k._sigma_on(cpu, torch.float64).tolist() == [5.0, 5.0, 5.0]
    assert k._sigma_on(cpu, torch.float32).tolist() == [5.0, 5.0, 5.0]


def test_dimension_and_dtype_checks_match_reference():
    """falkon/kernels/kernel.py:44-105."""
    k = GaussianKernel(1.0)
    X, C, v, w = torch.randn(8, 3), torch.randn(4, 3), torch.randn(4, 2), torch.randn(8, 2)
    with pytest.raises(ValueError, match="X1 must be 2D"):
        k.mmv(X[0], C, v)
    with pytest.raises(ValueError, match="X2 must be 2D"):
        k.dmmv(X, C[0], v, w)
    with pytest.raises(ValueError, match="Dimensions of matrix v"):
        k.mmv(X, C, v[:3])
    with pytest.raises(ValueError, match="Dimensions of matrix w"):
        k.dmmv(X, C, v, w[:5])
    with pytest.raises(ValueError, match="Output dimension"):
        k.mmv(X, C, v, out=torch.empty(8, 3))
    with pytest.raises(ValueError, match="One of v and w"):
        k.dmmv(X, C, None, None)
    with pytest.raises(TypeError, match="Data types"):
        k.mmv(X, C.double(), v)
    with pytest.raises(ValueError, match="memory contiguous"):
        k.mmv(torch.randn(16, 6)[::2, ::2], C, v)
    with pytest.raises(NotImplementedError):
        k.dmmv(X.clone().requires_grad_(), C, v, w)
    # 1-D v is reshaped to a column before reaching the backend
    seen = {}
    k._decide_mmv_impl = lambda *a: (lambda **kw: seen.update(kw) or "ok")
    assert k.mmv(X, C, torch.randn(4)) == "ok" and seen["v"].shape == (4, 1) and seen["kernel"] is k


def test_no_cpu_fallback():
    k = GaussianKernel(1.0)
    X, C, v = torch.randn(8, 3), torch.randn(4, 3), torch.randn(4, 2)
    with pytest.raises(RuntimeError, match="no CPU compute path"):
        k.mmv(X, C, v, opt=FalkonOptions(use_cpu=True))
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="needs a ROCm GPU"):
            k.dmmv(X, C, v, None)


def test_options_merge_like_reference():
    """Per-call options replace the kernel's (falkon/kernels/kernel.py:283-285)."""
    k = GaussianKernel(1.0, opt=FalkonOptions(max_gpu_mem=123.0))
    assert k._merged(None).max_gpu_mem == 123.0
    assert k._merged(FalkonOptions(use_cpu=True)).use_cpu is True
    fields = {f.name for f in dataclasses.fields(FalkonOptions)}
    for name in ("use_cpu", "max_gpu_mem", "max_cpu_mem", "memory_slack", "keops_active", "cg_tolerance",
                 "cg_full_gradient_every", "pc_epsilon_32", "no_single_kernel", "num_fmm_streams"):
        assert name in fields
    assert FalkonOptions().cg_epsilon(torch.float32) == 1e-7 and FalkonOptions().pc_epsilon(torch.float64) == 1e-13


def test_stride_helpers():
    """falkon/utils/tensor_helpers.py:128-213."""
    c, f = torch.empty(5, 3), torch.empty(3, 5).T
    assert is_contig(c) and is_contig(f) and not is_contig(torch.empty(10, 6)[::2, ::2])
    assert is_f_contig(f) and not is_f_contig(c)
    # (n,1) columns: non-strict accepts them as column-major, strict wants stride(1) >= n
    col = torch.empty(5, 1)
    assert is_f_contig(col, strict=False) and not is_f_contig(col, strict=True)
    assert is_f_contig(torch.empty_strided((5, 1), (1, 5)), strict=True)
    assert create_same_stride((7, 2), f, torch.float32, "cpu").stride() == (1, 7)
    assert create_same_stride((7, 2), c, torch.float32, "cpu").stride() == (2, 1)
    with pytest.raises(ValueError):
        create_same_stride((7, 2), torch.empty(10, 6)[::2, ::2], torch.float32, "cpu")


def test_product_code_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "falkon_amd")
    for base, _, files in os.walk(pkg):
        for fn in files:
            if fn.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(base, fn)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), fn
                assert "/root/reference" not in text, fn


def test_bench_refuses_more_than_one_gpu_and_builds_seeded_inputs():
    """bench.py: one GPU only (a clear message and a non-zero exit otherwise); synthetic inputs are reproducible."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout.strip() == ""
    sys.path.insert(0, ROOT)
    import bench
    saved = dict(bench.WORKLOADS)
    try:
        bench.WORKLOADS["C2"] = (1002, 2000, 28, 50, 1, True)          # same generator, small draw
        X, C, sigma, v, w = bench.make_inputs("C2")
        X2, C2, _, v2, w2 = bench.make_inputs("C2")
    finally:
        bench.WORKLOADS.update(saved)
    assert X.shape == (2000, 28) and C.shape == (50, 28) and v.shape == (50, 1) and w.shape == (2000, 1)
    assert X.dtype == torch.float32 and float(sigma) == 3.8
    assert torch.equal(X, X2) and torch.equal(C, C2) and torch.equal(v, v2) and torch.equal(w, w2)
    assert all(bool((C[i] == X).all(1).any()) for i in range(5))        # centres are rows of X


def test_laplacian_and_matern_kernel_objects():
    """Names, parameter handling and errors of the other distance kernels
    (falkon/kernels/distance_kernel.py:435-507,510-648)."""
    from falkon_amd import LaplacianKernel, MaternKernel
    from falkon_amd.mmv_ops.fmmv import _kernel_fn
    lap = LaplacianKernel(2.0)
    assert lap.kernel_name == "laplacian" and lap.name == "laplacian" and _kernel_fn(lap) == _backend.FLK_LAPLACIAN
    assert lap.sigma.dtype == torch.float64 and "sigma" in lap.diff_params and lap.nondiff_params == {"nu": 0.5}
    names = {0.5: ("0.5-matern", _backend.FLK_LAPLACIAN), 1.5: ("1.5-matern", _backend.FLK_MATERN32),
             2.5: ("2.5-matern", _backend.FLK_MATERN52), float("inf"): ("inf-matern", _backend.FLK_GAUSSIAN)}
    for nu, (name, code) in names.items():
        k = MaternKernel(torch.tensor([1.0, 2.0]), nu)
        assert k.kernel_name == name and _kernel_fn(k) == code and k.nondiff_params["nu"] == nu
        assert k.detach().kernel_name == name and repr(k).startswith("MaternKernel(")
    assert MaternKernel(1.0, torch.tensor(1.5)).nondiff_params["nu"] == 1.5
    assert MaternKernel(1.0, 2.4999).nondiff_params["nu"] == 2.5            # rounded to two digits
    with pytest.raises(ValueError):
        MaternKernel(1.0, 2.0)
    with pytest.raises(TypeError):
        MaternKernel(1.0, 2)
    with pytest.raises(ValueError):
        MaternKernel(1.0, torch.tensor(1.5, requires_grad=True))
    # the stock-torch block of every kernel agrees with the oracle's restatement of the reference core
    from oracle import gaussian_ref
    g = np.random.default_rng(0)
    X, C = torch.from_numpy(g.standard_normal((9, 4))), torch.from_numpy(g.standard_normal((6, 4)))
    for k in (lap, MaternKernel(2.0, 0.5), MaternKernel(2.0, 1.5), MaternKernel(2.0, 2.5), MaternKernel(2.0, float("inf")),
              GaussianKernel(2.0)):
        got = k.compute(X, C, torch.empty(9, 6, dtype=torch.float64), diag=False)
        torch.testing.assert_close(got, gaussian_ref.core_ref_for(k.kernel_name)(X, C, None, k.sigma), rtol=1e-12, atol=1e-14)
        assert float((k.compute(X, X, None, diag=True) - 1).abs().max()) < 1e-12

    class Other:
        kernel_name = "polynomial"
    with pytest.raises(NotImplementedError):
        _kernel_fn(Other())


def test_three_way_bfloat16_split_is_exact():
    """The arithmetic claim behind the bf16x3 mode (falkon_amd/csrc/split_common.h), checked in numpy: an fp32 value
    is the exact sum of three round-to-nearest bfloat16 pieces, and the six partial products the kernels keep
    reproduce an fp32 product to about 2^-23 of |x||y|."""
    import numpy as np

    def bf16_rne(x):                                  # the conversion of pack_split.hip, bit for bit
        u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
        r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
        return (r & 0xFFFFFFFF).astype(np.uint32).view(np.float32)

    def split3(x):
        hi = bf16_rne(x)
        r1 = (x - hi).astype(np.float32)
        mid = bf16_rne(r1)
        lo = bf16_rne((r1 - mid).astype(np.float32))
        return hi, mid, lo

    g = np.random.default_rng(0)
    x = (g.standard_normal(200_000) * np.exp(g.uniform(-30, 30, 200_000))).astype(np.float32)
    y = (g.standard_normal(200_000) * np.exp(g.uniform(-30, 30, 200_000))).astype(np.float32)
    xh, xm, xl = split3(x)
    assert np.array_equal((xh.astype(np.float64) + xm + xl).astype(np.float32), x)
    assert np.array_equal(xh.astype(np.float64) + xm.astype(np.float64) + xl.astype(np.float64), x.astype(np.float64))
    yh, ym, yl = split3(y)
    f = np.float64
    kept = (xm.astype(f) * ym + xh.astype(f) * yl + xl.astype(f) * yh + xh.astype(f) * ym + xm.astype(f) * yh
            + xh.astype(f) * yh)
    exact = x.astype(f) * y.astype(f)
    assert float(np.max(np.abs(kept - exact) / np.abs(exact))) < 2.0 ** -22


def test_torch_ops_are_registered_and_refuse_host_tensors():
    """``torch.ops.falkon.kernel_fmmv / kernel_fdmmv`` exist once falkon_amd.torch_ops is imported (the reference
    reaches its native code the same way, falkon/c_ext/__init__.py:13-21); there is no CPU implementation."""
    import falkon_amd.torch_ops  # noqa: F401
    schema = str(torch.ops.falkon.kernel_fmmv.default._schema)
    assert "Tensor(a4!) out" in schema and "kernel_fn=0" in schema and "bf16x3=False" in schema
    assert "Tensor? w" in str(torch.ops.falkon.kernel_fdmmv.default._schema)
    X = torch.randn(4, 3)
    with pytest.raises(RuntimeError, match="GPU only"):
        torch.ops.falkon.kernel_fmmv(X, X, torch.ones(1), torch.randn(4, 1), torch.empty(4, 1))
    with pytest.raises(RuntimeError, match="GPU only"):
        torch.ops.falkon.kernel_fdmmv(X, X, torch.ones(1), torch.randn(4, 1), None, torch.empty(4, 1))


def test_stored_block_route_rules(monkeypatch):
    """When the drivers store blocks of K instead of re-evaluating it per pass (many right-hand sides), how large
    the blocks are, and the options that switch the route off or on."""
    import importlib
    drv = importlib.import_module("falkon_amd.mmv_ops.fmmv")
    f32, f64 = torch.float32, torch.float64
    # off by default, whatever the number of right-hand sides: every product is matrix-free unless the caller opts in
    assert not any(drv._explicit_blocks_pay(d, t, dt, FalkonOptions())
                   for d in (9, 28, 100, 784) for t in (1, 17, 97, 1000, 10**4) for dt in (f32, f64))
    opt = FalkonOptions(many_rhs_stored_blocks=True)
    # from the measured break-even on: later for one product than for the two of dmmv (which evaluates K twice on the
    # matrix-free route), later at small d and in fp64, where an evaluation of K is cheap next to storing it
    pays = drv._explicit_blocks_pay
    assert not pays(784, 32, f32, opt) and pays(784, 33, f32, opt)
    assert not pays(784, 16, f32, opt, two_products=True) and pays(784, 17, f32, opt, two_products=True)
    assert not pays(28, 96, f32, opt) and pays(28, 97, f32, opt)
    assert not pays(28, 64, f32, opt, two_products=True) and pays(28, 65, f32, opt, two_products=True)
    assert not pays(40, 64, f32, opt) and pays(40, 65, f32, opt) and pays(40, 33, f32, opt, two_products=True)
    assert not pays(28, 128, f64, opt) and pays(28, 129, f64, opt) and pays(28, 129, f64, opt, two_products=True)
    assert not pays(40, 96, f64, opt) and pays(40, 97, f64, opt) and pays(40, 65, f64, opt, two_products=True)
    assert not pays(100, 64, f64, opt, two_products=True) and pays(100, 65, f64, opt, two_products=True)
    assert pays(784, 17, f64, opt, two_products=True) and not pays(784, 64, f64, opt) and pays(784, 65, f64, opt)
    assert not drv._explicit_blocks_pay(784, 1000, f32, FalkonOptions(many_rhs_stored_blocks=True, never_store_kernel=True))
    # block rows: within the block size, within half of what the budget leaves, nothing below 32 rows
    monkeypatch.setattr(drv, "usable_gpu_memory", lambda dev, cap, slack, enough=float("inf"): 64 * 2**30)
    rows = drv._explicit_block_rows(10**6, 10_000, 784, 256, 4, None, opt, upload_bytes=0)
    assert 32 <= rows <= 10**6 and rows * (10_000 + 512 + 3 * 784) * 4 <= drv._EXPLICIT_BLOCK_BYTES
    assert drv._explicit_block_rows(500, 10_000, 784, 256, 4, None, opt, upload_bytes=0) == 500
    monkeypatch.setattr(drv, "usable_gpu_memory", lambda dev, cap, slack, enough=float("inf"): 2**20)
    assert drv._explicit_block_rows(10**6, 10_000, 784, 256, 4, None, opt, upload_bytes=0) == 0


def test_memory_budget_reuses_a_recent_driver_report(monkeypatch):
    """``usable_gpu_memory`` (falkon/mmv_ops/utils.py:47-58): ``slack * min(free, max_gpu_mem)``.  The driver's report is
    asked for again unless a call needs at most an eighth of what it said within the last 50 ms; the value handed to
    such a call is a lower bound that still covers it."""
    import importlib
    utils = importlib.import_module("falkon_amd.mmv_ops.utils")
    calls = []

    def report(dev):
        calls.append(dev)
        return 80 * 2**30, 288 * 2**30
    monkeypatch.setattr(torch.cuda, "mem_get_info", report)
    monkeypatch.setattr(torch.cuda, "memory_reserved", lambda dev: 0)
    monkeypatch.setattr(torch.cuda, "memory_allocated", lambda dev: 0)
    utils._recent_free.clear()
    monkeypatch.setattr(utils, "_FREE_MEMORY_TTL", 3600.0)      # (50 ms in the library: a loaded machine must not age the report here)
    dev = torch.device("cuda", 0)
    big = utils.usable_gpu_memory(dev, float("inf"), 0.9, enough=2**30)
    assert len(calls) == 1 and big == pytest.approx(0.9 * 80 * 2**30)
    small = utils.usable_gpu_memory(dev, float("inf"), 0.9, enough=2**30)          # 8 GiB <= 72 GiB: the report is reused
    assert len(calls) == 1 and 2**30 <= small <= big
    assert utils.usable_gpu_memory(dev, 2**29, 0.9, enough=2**30) == pytest.approx(0.9 * 2**29)   # the cap still binds
    assert len(calls) == 1
    utils.usable_gpu_memory(dev, float("inf"), 0.9, enough=20 * 2**30)             # too large a share: asked again
    assert len(calls) == 2
    monkeypatch.setattr(utils, "_FREE_MEMORY_TTL", 0.0)
    utils.usable_gpu_memory(dev, float("inf"), 0.9, enough=2**20)                  # too old: asked again
    assert len(calls) == 3
    utils._recent_free.clear()
    utils._reused.clear()


def test_out_of_memory_on_a_reused_report_is_planned_again(monkeypatch):
    """A plan made from a reused free-memory report can be stale (somebody allocated in between): a product that runs
    out of memory on such a plan runs once more on a fresh report; one that was planned on a fresh report fails."""
    import importlib
    utils = importlib.import_module("falkon_amd.mmv_ops.utils")
    calls, runs = [], []
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda dev: (calls.append(dev), (80 * 2**30, 288 * 2**30))[1])
    monkeypatch.setattr(utils, "_FREE_MEMORY_TTL", 3600.0)      # the reuse below must not depend on how fast this machine is
    utils._recent_free.clear()
    utils._reused.clear()
    dev = torch.device("cuda", 0)

    def product():
        runs.append(utils.usable_gpu_memory(dev, float("inf"), 0.9, enough=2**30))
        if len(runs) == 2:                                       # the plan from the reused report does not fit
            raise torch.cuda.OutOfMemoryError("simulated")
        return len(runs)

    assert utils.retry_with_fresh_memory_report(product) == 1 and len(calls) == 1
    assert utils.retry_with_fresh_memory_report(product) == 3    # second run reused the report, failed, ran again
    assert len(calls) == 2 and runs[2] == pytest.approx(0.9 * 80 * 2**30)

    def always_fails():
        utils.usable_gpu_memory(dev, float("inf"), 0.9, enough=70 * 2**30)     # too large a share: a fresh report
        raise torch.cuda.OutOfMemoryError("simulated")
    with pytest.raises(torch.cuda.OutOfMemoryError):
        utils.retry_with_fresh_memory_report(always_fails)
    utils._recent_free.clear()
    utils._reused.clear()


def test_bench_defaults_by_workload():
    """The C5 workload's step is a whole fit: it defaults to few of them; the others keep 50 timed steps."""
    import ast
    src = open(os.path.join(os.path.dirname(__file__), "..", "bench.py")).read()
    assert 'args.steps = 2 if args.workload == "C5" else 50' in src and ast.parse(src)
