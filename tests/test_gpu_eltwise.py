"""GPU parity of stk.ops.mul: the reference's element-wise grid (stk/ops/eltwise_ops_test.py:9-36, 53-83).

14 sizes x {float16, bfloat16}, blocking 128: the product of two matrices with one topology against torch.mul on
their dense copies, forward and both gradients.  The reference drives the backward pass with a gradient of ones
(`stk.ops.sum(out).backward()`); here it is run once that way and once with a seeded N(0, 1) gradient on the values,
so that a gradient that mixed up blocks cannot pass.  The product of two 16-bit numbers rounded once is what both
sides compute, so the comparison is exact.
"""
import itertools

import numpy as np
import pytest
import torch

import stk_amd as stk
from tests import _util as U

pytestmark = pytest.mark.gpu
DEV = "cuda"

_SIZES = (
    (128, 128, 0.0), (256, 256, 0.5), (2048, 1024, 0.8), (512, 128, 0.0), (128, 512, 0.0),
    (1024, 512, 0.0), (1024, 512, 0.5), (1024, 512, 0.75), (512, 1024, 0.0), (512, 1024, 0.5), (512, 1024, 0.75),
    (1024, 1024, 0.0), (1024, 1024, 0.5), (1024, 1024, 0.75),
)
_DTYPES = (torch.float16, torch.bfloat16)


def _dense_and_sparse(rows, cols, sparsity, blocking, dtype, std=0.1):
    # stk/ops/linear_ops_test.py:57-63: built on the host, then moved
    mask = stk.random.dense_mask(rows, cols, sparsity, blocking)
    dense = (torch.randn(rows, cols) * std * mask).to(dtype)
    sparse = stk.ops.to_sparse(dense, blocking)
    return dense.to(DEV).requires_grad_(True), sparse.to(DEV).requires_grad_(True)


def _dense_and_sparse_like(x, std=0.1):
    # stk/ops/eltwise_ops_test.py:40-50: new values on x's pattern; the transpose metadata is rebuilt on the device
    values = (torch.randn(x.data.shape) * std).to(x.dtype).to(x.device)
    sparse = stk.Matrix(x.size(), values, x.row_indices, x.column_indices, x.offsets)
    return stk.ops.to_dense(sparse).requires_grad_(True), sparse.requires_grad_(True)


@pytest.mark.parametrize("m,n,sparsity,dtype", [(*s, d) for s, d in itertools.product(_SIZES, _DTYPES)])
def test_eltwise_mul(m, n, sparsity, dtype):
    seed = U.stable_seed("mul", m, n, sparsity, dtype)
    np.random.seed(seed)
    torch.manual_seed(seed)
    a_dense, a = _dense_and_sparse(m, n, sparsity, 128, dtype)
    b_dense, b = _dense_and_sparse_like(a)
    assert torch.equal(b.column_indices_t, a.column_indices_t) and torch.equal(b.block_offsets_t, a.block_offsets_t)

    out = stk.ops.mul(a, b)
    expected = torch.mul(a_dense, b_dense)
    assert isinstance(out, stk.Matrix) and out.dtype == dtype and out.data.shape == a.data.shape
    dense_out = stk.ops.to_dense(out)
    assert dense_out.dim() == 2 and dense_out.shape == expected.shape
    assert torch.equal(dense_out, expected)

    # the reference's procedure: sum of the values, gradient of ones
    expected.sum().backward()
    stk.ops.sum(out).backward()
    for sparse, dense, what in ((a, a_dense, "lhs"), (b, b_dense, "rhs")):
        grad = stk.ops.to_dense(sparse.grad)
        assert grad.dim() == 2 and grad.shape == dense.grad.shape
        # the dense side also has gradients outside the pattern (zeros times ones): compare on the pattern
        mask = stk.ops.to_dense(stk.ops.ones_like(sparse)).bool()
        assert torch.equal(grad[mask], dense.grad[mask]), what
        assert not bool(grad[~mask].any()), what

    # and with a seeded gradient on the values
    for t in (a.data, b.data, a_dense, b_dense):
        t.grad = None
    g = torch.randn(out.data.shape).to(dtype).to(DEV)
    g_dense = stk.ops.to_dense(stk.Matrix(a.size(), g, a.row_indices, a.column_indices, a.offsets, a.column_indices_t, a.offsets_t, a.block_offsets_t))
    stk.ops.mul(a, b).data.backward(g)
    torch.mul(a_dense, b_dense).backward(g_dense)
    assert torch.equal(stk.ops.to_dense(a.grad), a_dense.grad) and torch.equal(stk.ops.to_dense(b.grad), b_dense.grad)
