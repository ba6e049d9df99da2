"""CPU tier: the host twins of the products and format helpers (libstk_amd_host.so), which serve tensors in host memory.

BASELINE configuration 1 as the reference states it - stk.random.mask(1024, 1024, 0.5, 128) from numpy seed 0, dense
operands 1024 x 1024 fp32 ~ N(0, 1), sdd / dsd / dds in all transposes against to_dense + torch.matmul masked, on the
CPU (stk/ops/linear_ops_test.py:83-96, 110-111) - runs here through stk.ops on host tensors, forward and backward,
and is also checked against the oracle and the committed known-answer topology.  No GPU is involved.
"""
import ctypes
import json
import os
import re
import subprocess

import numpy as np
import pytest
import torch

import stk_amd as stk
from oracle import stk_oracle as O
from stk_amd.backend import host_kernels
from tests import _util as U

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_TRANSPOSE = ((False, False), (False, True), (True, False), (True, True))


def test_host_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "stk_amd_host.h")).read()
    declared = set(re.findall(r"\b(stk_cpu_[a-z0-9_]+)\s*\(", header))
    assert declared == set(host_kernels.SIGNATURES), declared ^ set(host_kernels.SIGNATURES)
    assert os.path.exists(host_kernels.LIB_PATH), "build the library first: make -C stk_amd/csrc"
    lib = ctypes.CDLL(host_kernels.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    # plain C++: the host library must not pull in the HIP runtime
    needed = subprocess.run(["readelf", "-d", host_kernels.LIB_PATH], capture_output=True, text=True).stdout
    assert "amdhip" not in needed and "hsa" not in needed, needed


def _config1():
    np.random.seed(0)
    torch.manual_seed(0)
    s = stk.random.mask(1024, 1024, 0.5, 128)
    with open(os.path.join(ROOT, "tests", "golden", "config1_topology.json")) as f:
        golden = json.load(f)
    for name in ("row_indices", "column_indices", "offsets", "offsets_t", "column_indices_t", "block_offsets_t"):
        assert getattr(s, name).tolist() == golden[name], name
    values = torch.randn(s.data.shape)
    s = stk.Matrix(s.size(), values, s.row_indices, s.column_indices, s.offsets, s.column_indices_t, s.offsets_t, s.block_offsets_t)
    return s, torch.randn(1024, 1024), torch.randn(1024, 1024)


# fp32 sums of 1024 products of N(0, 1) values are ~32; two fp32 summation orders differ by a few 1e-5 of that
_F32 = dict(rtol=1e-4, atol=2e-3)


def test_config1_fp32_on_the_cpu_forward():
    s, a, b = _config1()
    assert s.data.dtype == torch.float32 and not s.is_cuda
    topo = U.topo_of(s)
    data32 = s.data.numpy()
    dense = stk.ops.to_dense(s)
    mask = stk.ops.to_dense(stk.ops.ones_like(s))
    assert dense.dtype == torch.float32 and int(mask.sum()) == 32 * 128 * 128
    for ta, tb in _TRANSPOSE:
        lhs, rhs = (a.t() if ta else a), (b.t() if tb else b)
        # the reference's comparator: to_dense + torch.matmul, the sdd result masked to the topology
        sd = dense.t() if ta else dense
        got = stk.ops.dsd(s.t() if ta else s, rhs)
        np.testing.assert_allclose(got.numpy(), (sd @ rhs).numpy(), **_F32, err_msg=f"dsd {ta} {tb} vs matmul")
        np.testing.assert_allclose(got.numpy(), O.dsd((1024, 1024), data32, topo, ta, rhs.numpy()), **_F32, err_msg=f"dsd {ta} {tb} vs oracle")
        sd = dense.t() if tb else dense
        got = stk.ops.dds(lhs, s.t() if tb else s)
        np.testing.assert_allclose(got.numpy(), (lhs @ sd).numpy(), **_F32, err_msg=f"dds {ta} {tb} vs matmul")
        np.testing.assert_allclose(got.numpy(), O.dds(lhs.numpy(), (1024, 1024), data32, topo, tb), **_F32, err_msg=f"dds {ta} {tb} vs oracle")
        got = stk.ops.sdd(lhs, rhs, s)
        assert got.data.dtype == torch.float32 and got.data.shape == s.data.shape
        np.testing.assert_allclose(stk.ops.to_dense(got).numpy(), ((lhs @ rhs) * mask).numpy(), **_F32, err_msg=f"sdd {ta} {tb} vs masked matmul")
        np.testing.assert_allclose(got.data.numpy(), O.sdd(lhs.numpy(), rhs.numpy(), topo), **_F32, err_msg=f"sdd {ta} {tb} vs oracle")


@pytest.mark.parametrize("ta,tb", _TRANSPOSE)
def test_config1_fp32_on_the_cpu_gradients(ta, tb):
    # the reference's test procedure (linear_ops_test.py:99-207) on host tensors: gradients of the three products against
    # torch autograd on the dense copy, sparse gradients after to_dense, dense gradients of sdd masked - with a seeded
    # N(0, 1) incoming gradient instead of ones, so that a gradient built from the wrong block or its transpose fails
    s, a, b = _config1()
    g = torch.Generator().manual_seed(17)
    dense = stk.ops.to_dense(s)
    mask = stk.ops.to_dense(stk.ops.ones_like(s))
    tol = dict(rtol=1e-4, atol=4e-3)

    # dsd
    sp = stk.Matrix(s.size(), s.data.clone(), s.row_indices, s.column_indices, s.offsets, s.column_indices_t, s.offsets_t, s.block_offsets_t)
    sp.requires_grad_(True)
    rhs, rhs_ref, d_ref = b.clone().requires_grad_(True), b.clone().requires_grad_(True), dense.clone().requires_grad_(True)
    out = stk.ops.dsd(sp.t() if ta else sp, rhs.t() if tb else rhs)
    ref = (d_ref.t() if ta else d_ref) @ (rhs_ref.t() if tb else rhs_ref)
    dy = torch.randn(out.shape, generator=g)
    out.backward(dy)
    ref.backward(dy)
    np.testing.assert_allclose(stk.ops.to_dense(sp.grad).numpy(), (d_ref.grad * mask).numpy(), **tol, err_msg="dsd: d sparse")
    np.testing.assert_allclose(rhs.grad.numpy(), rhs_ref.grad.numpy(), **tol, err_msg="dsd: d rhs")

    # dds
    sp = stk.Matrix(s.size(), s.data.clone(), s.row_indices, s.column_indices, s.offsets, s.column_indices_t, s.offsets_t, s.block_offsets_t)
    sp.requires_grad_(True)
    lhs, lhs_ref, d_ref = a.clone().requires_grad_(True), a.clone().requires_grad_(True), dense.clone().requires_grad_(True)
    out = stk.ops.dds(lhs.t() if ta else lhs, sp.t() if tb else sp)
    ref = (lhs_ref.t() if ta else lhs_ref) @ (d_ref.t() if tb else d_ref)
    dy = torch.randn(out.shape, generator=g)
    out.backward(dy)
    ref.backward(dy)
    np.testing.assert_allclose(stk.ops.to_dense(sp.grad).numpy(), (d_ref.grad * mask).numpy(), **tol, err_msg="dds: d sparse")
    np.testing.assert_allclose(lhs.grad.numpy(), lhs_ref.grad.numpy(), **tol, err_msg="dds: d lhs")

    # sdd
    lhs, lhs_ref = a.clone().requires_grad_(True), a.clone().requires_grad_(True)
    rhs, rhs_ref = b.clone().requires_grad_(True), b.clone().requires_grad_(True)
    out = stk.ops.sdd(lhs.t() if ta else lhs, rhs.t() if tb else rhs, s)
    ref = ((lhs_ref.t() if ta else lhs_ref) @ (rhs_ref.t() if tb else rhs_ref)) * mask
    dvalues = torch.randn(out.data.shape, generator=g)
    dy = stk.ops.to_dense(stk.Matrix(s.size(), dvalues, s.row_indices, s.column_indices, s.offsets, s.column_indices_t, s.offsets_t, s.block_offsets_t))
    out.data.backward(dvalues)
    ref.backward(dy)
    np.testing.assert_allclose(lhs.grad.numpy(), lhs_ref.grad.numpy(), **tol, err_msg="sdd: d lhs")
    np.testing.assert_allclose(rhs.grad.numpy(), rhs_ref.grad.numpy(), **tol, err_msg="sdd: d rhs")


def _random_case(seed, rows, cols, blocking, sparsity, dtype, index_dtype):
    np.random.seed(seed)
    g = torch.Generator().manual_seed(seed)
    mask = stk.random.dense_mask(rows, cols, sparsity, blocking)
    dense = (torch.randn(rows, cols, generator=g) * mask).to(dtype)
    s = stk.ops.to_sparse(dense, blocking)
    if index_dtype == torch.int32:
        s = stk.Matrix(s.size(), s.data, s.row_indices.int(), s.column_indices.int(), s.offsets)
    return dense, s, g


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,cols,n,blocking,sparsity,index_dtype", [
    (64, 96, 40, 8, 0.5, torch.int16), (64, 96, 40, 16, 0.75, torch.int32), (96, 64, 33, 32, 0.5, torch.int16),
    (256, 384, 264, 128, 0.5, torch.int16), (128, 128, 128, 128, 0.0, torch.int16), (128, 256, 8, 64, 1.0, torch.int16),
    (24, 40, 17, 1, 0.6, torch.int32), (320, 64, 300, 64, 0.4, torch.int16)])
def test_host_products_match_the_oracle(rows, cols, n, blocking, sparsity, index_dtype, dtype):
    # blockings from 1 to 128, patterns with empty rows and columns (sparsity 1.0: no block at all), ragged dense
    # extents, both index widths; operands as row-major tensors, .t() views and strided slices
    dense, s, g = _random_case(rows * 31 + cols + blocking, rows, cols, blocking, sparsity, dtype, index_dtype)
    topo = U.topo_of(s)
    data32 = U.np32(s.data)
    tol = _F32 if dtype == torch.float32 else U.TOL[dtype]
    operands = {
        "row-major": lambda r, c: torch.randn(r, c, generator=g).to(dtype),
        "transposed view": lambda r, c: torch.randn(c, r, generator=g).to(dtype).t(),
        "strided slice": lambda r, c: torch.randn(r, 2 * c + 3, generator=g).to(dtype)[:, 1:2 * c + 1:2],
    }
    for layout, make in operands.items():
        for trans in (False, True):
            k = rows if trans else cols
            rhs = make(k, n)
            got = torch.empty((cols if trans else rows, n), dtype=dtype)
            host_kernels.dsd((cols, rows) if trans else (rows, cols), s.data, s.offsets, s.row_indices, s.column_indices, s.offsets_t,
                             s.column_indices_t, s.block_offsets_t, trans, rhs, got)
            want = O.dsd((cols, rows) if trans else (rows, cols), data32, topo, trans, U.np32(rhs))
            np.testing.assert_allclose(U.np32(got), want, **tol, err_msg=f"dsd {layout} trans={trans}")
            k = cols if trans else rows
            lhs = make(n, k)
            got = torch.empty((n, rows if trans else cols), dtype=dtype)
            host_kernels.dds(lhs, (cols, rows) if trans else (rows, cols), s.data, s.offsets, s.row_indices, s.column_indices, s.offsets_t,
                             s.column_indices_t, s.block_offsets_t, trans, got)
            want = O.dds(U.np32(lhs), (cols, rows) if trans else (rows, cols), data32, topo, trans)
            np.testing.assert_allclose(U.np32(got), want, **tol, err_msg=f"dds {layout} trans={trans}")
        lhs, rhs = make(rows, 48), make(48, cols)
        got = torch.empty_like(s.data)
        host_kernels.sdd(lhs, rhs, (rows, cols), got, s.offsets, s.row_indices, s.column_indices)
        np.testing.assert_allclose(U.np32(got), O.sdd(U.np32(lhs), U.np32(rhs), topo), **tol, err_msg=f"sdd {layout}")


def test_host_products_against_brute_force_loops():
    # an independent statement of the three products: scalar loops over the dense matrix of the pattern
    dense, s, g = _random_case(5, 12, 20, 4, 0.5, torch.float32, torch.int16)
    d = dense.numpy().astype(np.float64)
    b = torch.randn(20, 7, generator=g)
    a = torch.randn(5, 12, generator=g)
    want = np.zeros((12, 7))
    for i in range(12):
        for j in range(7):
            for k in range(20):
                want[i, j] += d[i, k] * float(b[k, j])
    meta = (s.offsets, s.row_indices, s.column_indices, s.offsets_t, s.column_indices_t, s.block_offsets_t)
    got = torch.empty(12, 7)
    host_kernels.dsd((12, 20), s.data, *meta, False, b, got)      # (stk.ops would apply the reference's divisibility rules)
    np.testing.assert_allclose(got.numpy(), want, rtol=1e-5, atol=1e-5)
    want = np.zeros((5, 20))
    for i in range(5):
        for j in range(20):
            for k in range(12):
                want[i, j] += float(a[i, k]) * d[k, j]
    got = torch.empty(5, 20)
    host_kernels.dds(a, (12, 20), s.data, *meta, False, got)
    np.testing.assert_allclose(got.numpy(), want, rtol=1e-5, atol=1e-5)
    x, w = torch.randn(12, 32, generator=g), torch.randn(32, 20, generator=g)
    want = np.zeros((12, 20))
    nonzero = stk.ops.to_dense(stk.ops.ones_like(s)).numpy()
    for i in range(12):
        for j in range(20):
            if nonzero[i, j]:
                want[i, j] = sum(float(x[i, k]) * float(w[k, j]) for k in range(32))
    got = torch.empty_like(s.data)
    host_kernels.sdd(x, w, (12, 20), got, s.offsets, s.row_indices, s.column_indices)
    got = stk.Matrix(s.size(), got, s.row_indices, s.column_indices, s.offsets)
    np.testing.assert_allclose(stk.ops.to_dense(got).numpy(), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_sixteen_bit_conversions_of_the_host_library_are_torchs(dtype):
    # blocking 1, one block: out[i, j] = round(load(s) * load(rhs[j])) - every 16-bit pattern through the load, and the
    # fp32 products of two 16-bit numbers (up to 22 significant bits: ties, subnormal results, overflow) through the store
    every = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
    one = torch.ones(1, 1, 1, dtype=dtype)
    idx, off = torch.zeros(1, dtype=torch.int16), torch.tensor([0, 1], dtype=torch.int32)
    got = torch.empty(1, 65536, dtype=dtype)
    host_kernels.dsd((1, 1), one, off, idx, idx, off, idx, torch.zeros(1, dtype=torch.int32), False, every.view(1, -1), got)
    finite = ~torch.isnan(every.float())
    assert torch.equal(got[0][finite].float(), every[finite].float())       # (values: 0 + 1 * -0 is +0)
    nonzero = finite & (every.float() != 0)
    assert torch.equal(got.view(torch.int16)[0][nonzero], every.view(torch.int16)[nonzero])
    assert bool(torch.isnan(got[0][~finite].float()).all())
    g = torch.Generator().manual_seed(3)
    for scale in (1.0, 1e-3, 250.0, 6e-5):
        a = (torch.randn(4096, generator=g) * scale).to(dtype)
        b = (torch.randn(4096, generator=g) * scale).to(dtype)
        for k in range(0, 4096, 512):
            s = a[k].reshape(1, 1, 1)
            host_kernels.dsd((1, 1), s, off, idx, idx, off, idx, torch.zeros(1, dtype=torch.int32), False, b.view(1, -1), got[:, :4096])
            want = (a[k].float() * b.float()).to(dtype)
            assert torch.equal(got[0, :4096].float(), want.float()), (dtype, scale, k)


def test_host_products_keep_the_error_contract():
    s = stk.ops.to_sparse(torch.ones(128, 256), 128)
    with pytest.raises(AssertionError):
        stk.ops.dsd(s, torch.ones(128, 128))                     # inner dimensions differ (triton_kernels.py:243)
    with pytest.raises(AssertionError):
        stk.ops.dds(torch.ones(128, 256), s)                     # (triton_kernels.py:299)
    with pytest.raises(AssertionError):
        stk.ops.sdd(torch.ones(128, 100), torch.ones(100, 256), s)   # k not divisible by 32 (triton_kernels.py:15-19)
    with pytest.raises(NotImplementedError):
        stk.ops.dsd(stk.ops.to_sparse(torch.ones(128, 128, dtype=torch.float64), 128), torch.ones(128, 128, dtype=torch.float64))
    with pytest.raises(NotImplementedError, match="GPU"):
        stk.ops.sdd_fused(torch.ones(128, 128), torch.ones(128, 256), s, "relu")
    lib = host_kernels.load()
    # metadata that points outside the matrix is refused before anything is read through it
    bad = torch.tensor([0, 7], dtype=torch.int16)
    rc = lib.stk_cpu_dsd(128, 256, 8, s.data.data_ptr(), s.offsets.data_ptr(), bad.data_ptr(), s.offsets_t.data_ptr(),
                         s.column_indices_t.data_ptr(), s.block_offsets_t.data_ptr(), 0, torch.ones(256, 8).data_ptr(), 8, 1,
                         torch.empty(128, 8).data_ptr(), 8, 2, 128, host_kernels.STK_F32, 0)
    assert rc == 1 and b"outside the matrix" in lib.stk_cpu_last_error()


def test_products_never_mix_host_and_device_tensors():
    # the dispatch is by where the output lives; a device tensor among host operands is an error, not a copy
    class Fake:
        is_cuda = True
    with pytest.raises(RuntimeError, match="host memory"):
        host_kernels._host_only(torch.ones(1), Fake())


def test_index_walks_under_the_address_and_undefined_behaviour_sanitizers(tmp_path):
    """tests/host_check.cc drives every stk_cpu_* entry point over seeded random patterns (empty rows and columns,
    both index widths, transposes, ragged dense extents, refused metadata) and checks the results against dense loops
    of its own.  Built together with the library's source under -fsanitize=address,undefined, any read or write outside
    an operand, an output or a metadata array ends the run."""
    exe = str(tmp_path / "host_check")
    build = subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-static-libasan",
                            os.path.join(ROOT, "tests", "host_check.cc"), os.path.join(ROOT, "stk_amd", "csrc", "host.cc"), "-o", exe],
                           capture_output=True, text=True, timeout=600)
    assert build.returncode == 0, build.stderr
    run = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-4000:]
    assert "host_check ok" in run.stdout
