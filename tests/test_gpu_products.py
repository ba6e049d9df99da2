"""GPU parity, floating-point side: sdd / dsd / dds forward and both gradients.

Every product runs through the C ABI on the GPU and is compared with the CPU
oracle (fp32 block walk restating the reference kernels) on the same seeded,
dtype-rounded inputs.  Tolerances (tests/_util.py): rtol 1e-2 with atol 1e-2
for bfloat16 and atol 5e-3 for float16.  The size / transpose / dtype grid is
the reference's (stk/ops/linear_ops_test.py:21-47), extended by blocking 64,
32-bit indices, ragged and empty patterns.
"""
import itertools

import numpy as np
import pytest
import torch

import stk_amd as stk
from oracle import stk_oracle as O
from tests import _util as U

pytestmark = pytest.mark.gpu
DEV = "cuda"

_SIZES = (
    (128, 128, 128, 0.0), (256, 256, 256, 0.5), (2048, 1024, 512, 0.8), (512, 128, 128, 0.0),
    (128, 128, 512, 0.0), (1024, 512, 512, 0.0), (1024, 512, 512, 0.5), (1024, 512, 512, 0.75),
    (512, 512, 1024, 0.0), (512, 512, 1024, 0.5), (512, 512, 1024, 0.75),
    (1024, 1024, 1024, 0.0), (1024, 1024, 1024, 0.5), (1024, 1024, 1024, 0.75),
)
_TRANSPOSE = ((False, False), (False, True), (True, False), (True, True))
_DTYPES = (torch.float16, torch.bfloat16)
_SMALL = ((128, 64, 192, 0.0), (256, 192, 320, 0.5), (512, 256, 128, 0.8), (64, 64, 64, 0.0))

_GRID = [(*s, *t, 128, d) for s, t, d in itertools.product(_SIZES, _TRANSPOSE, _DTYPES)]
_GRID += [(*s, *t, 64, d) for s, t, d in itertools.product(_SMALL, _TRANSPOSE, _DTYPES)]
# float32 values, which the reference's launchers pass on like any other dtype (stk/backend/triton_kernels.py:250, 306, 358)
_GRID += [(*s, *t, 128, torch.float32) for s, t in itertools.product(_SIZES, _TRANSPOSE)]
_GRID += [(*s, *t, 64, torch.float32) for s, t in itertools.product(_SMALL, _TRANSPOSE)]


def _seed(*args):
    """Seeds numpy and torch from the test's arguments; the same inputs in every process, so that a failure
    seen once can be reproduced from its test id."""
    s = U.stable_seed(*args)
    np.random.seed(s)
    torch.manual_seed(s)
    return s


def _incoming_gradient(shape, dtype):
    """A seeded N(0, 1) gradient in the output's dtype: every block row and column of it is different, so a
    backward pass that picked the wrong block of it, or its transpose inside a block, cannot pass."""
    return torch.randn(*shape).to(dtype).to(DEV)


def _dense(rows, cols, dtype, std=0.1):
    return (torch.randn(rows, cols) * std).to(dtype).to(DEV).requires_grad_(True)


def _dense_and_sparse(rows, cols, sparsity, blocking, dtype, std=0.1):
    mask = stk.random.dense_mask(rows, cols, sparsity, blocking)
    dense = (torch.randn(rows, cols) * std * mask).to(dtype)
    sparse = stk.ops.to_sparse(dense, blocking)        # built on the host, like the reference's tests
    return dense, sparse.to(DEV).requires_grad_(True)


@pytest.mark.parametrize("m,k,n,sparsity,trans_a,trans_b,blocking,dtype", _GRID)
def test_dsd(m, k, n, sparsity, trans_a, trans_b, blocking, dtype):
    _seed("dsd", m, k, n, sparsity, trans_a, trans_b, blocking, dtype)
    a_dense, a = _dense_and_sparse(*((k, m) if trans_a else (m, k)), sparsity, blocking, dtype)
    b = _dense(*((n, k) if trans_b else (k, n)), dtype)
    lhs = a.t() if trans_a else a
    rhs = b.t() if trans_b else b
    out = stk.ops.dsd(lhs, rhs)
    assert out.shape == (m, n) and out.dtype == dtype and out.is_contiguous()
    topo = U.topo_of(a)
    want = O.dsd((m, k), U.np32(a.data), topo, trans_a, U.np32(rhs))
    U.assert_close(out, want, dtype, "dsd forward")

    g = _incoming_gradient((m, n), dtype)
    out.backward(g)
    g32 = U.np32(g)
    # d data: (dy rhs^T) sampled on the stored pattern (transposed when the operand is)
    rhs32 = U.np32(rhs)
    want_data = O.sdd(rhs32, g32.T, topo) if trans_a else O.sdd(g32, rhs32.T, topo)
    assert a.grad.data.shape == a.data.shape
    U.assert_close(a.grad.data, want_data, dtype, "dsd grad wrt sparse")
    # d rhs = op(S)^T dy, in the layout of b
    want_rhs = O.dsd((k, m), U.np32(a.data), topo, not trans_a, g32)
    assert b.grad.shape == b.shape
    U.assert_close(b.grad, want_rhs.T if trans_b else want_rhs, dtype, "dsd grad wrt dense")


@pytest.mark.parametrize("m,k,n,sparsity,trans_a,trans_b,blocking,dtype", _GRID)
def test_dds(m, k, n, sparsity, trans_a, trans_b, blocking, dtype):
    _seed("dds", m, k, n, sparsity, trans_a, trans_b, blocking, dtype)
    a = _dense(*((k, m) if trans_a else (m, k)), dtype)
    b_dense, b = _dense_and_sparse(*((n, k) if trans_b else (k, n)), sparsity, blocking, dtype)
    lhs = a.t() if trans_a else a
    rhs = b.t() if trans_b else b
    out = stk.ops.dds(lhs, rhs)
    assert out.shape == (m, n) and out.dtype == dtype and out.is_contiguous()
    topo = U.topo_of(b)
    want = O.dds(U.np32(lhs), (k, n), U.np32(b.data), topo, trans_b)
    U.assert_close(out, want, dtype, "dds forward")

    g = _incoming_gradient((m, n), dtype)
    out.backward(g)
    g32 = U.np32(g)
    want_lhs = O.dds(g32, (n, k), U.np32(b.data), topo, not trans_b)
    assert a.grad.shape == a.shape
    U.assert_close(a.grad, want_lhs.T if trans_a else want_lhs, dtype, "dds grad wrt dense")
    lhs32 = U.np32(lhs)
    want_data = O.sdd(g32.T, lhs32, topo) if trans_b else O.sdd(lhs32.T, g32, topo)
    U.assert_close(b.grad.data, want_data, dtype, "dds grad wrt sparse")


@pytest.mark.parametrize("m,k,n,sparsity,trans_a,trans_b,blocking,dtype", _GRID)
def test_sdd(m, k, n, sparsity, trans_a, trans_b, blocking, dtype):
    _seed("sdd", m, k, n, sparsity, trans_a, trans_b, blocking, dtype)
    a = _dense(*((k, m) if trans_a else (m, k)), dtype)
    b = _dense(*((n, k) if trans_b else (k, n)), dtype)
    _, topo_m = _dense_and_sparse(m, n, sparsity, blocking, dtype)
    lhs = a.t() if trans_a else a
    rhs = b.t() if trans_b else b
    out = stk.ops.sdd(lhs, rhs, topo_m)
    assert isinstance(out, stk.Matrix) and out.data.shape == topo_m.data.shape and out.dtype == dtype
    topo = U.topo_of(topo_m)
    want = O.sdd(U.np32(lhs), U.np32(rhs), topo)
    U.assert_close(out.data, want, dtype, "sdd forward")
    # the reference's own comparator: dense product masked to the topology
    U.assert_close(out.data, O.dense_masked_sdd(U.np32(lhs), U.np32(rhs), topo), dtype, "sdd vs dense-masked")

    g = _incoming_gradient(want.shape, dtype)
    out.data.backward(g)
    g32 = U.np32(g)
    want_lhs = O.dsd((m, n), g32, topo, False, U.np32(rhs).T)
    want_rhs = O.dds(U.np32(lhs).T, (m, n), g32, topo, False)
    U.assert_close(a.grad, want_lhs.T if trans_a else want_lhs, dtype, "sdd grad wrt lhs")
    U.assert_close(b.grad, want_rhs.T if trans_b else want_rhs, dtype, "sdd grad wrt rhs")


_ACTIVATIONS = (None, "relu", "gelu_tanh", "gelu", "silu")
_TORCH_ACTIVATIONS = {None: lambda v: v, "relu": torch.relu, "gelu": torch.nn.functional.gelu, "silu": torch.nn.functional.silu,
                      "gelu_tanh": lambda v: torch.nn.functional.gelu(v, approximate="tanh")}


def _fused_case(m, k, n, sparsity, blocking, dtype, trans_a=False, trans_b=False):
    # operands scaled so that the sums reach the saturating parts of the activations
    a = (torch.randn(*((k, m) if trans_a else (m, k))) * 0.5).to(dtype).to(DEV)
    b = (torch.randn(*((n, k) if trans_b else (k, n))) * 0.5).to(dtype).to(DEV)
    _, topo_m = _dense_and_sparse(m, n, sparsity, blocking, dtype)
    mult = stk.Matrix(topo_m.size(), torch.randn(topo_m.data.shape).to(dtype).to(DEV), topo_m.row_indices, topo_m.column_indices,
                      topo_m.offsets, topo_m.column_indices_t, topo_m.offsets_t, topo_m.block_offsets_t)
    return (a.t() if trans_a else a), (b.t() if trans_b else b), topo_m, mult


@pytest.mark.parametrize("with_multiplier", [False, True])
@pytest.mark.parametrize("activation", _ACTIVATIONS)
@pytest.mark.parametrize("m,k,n,sparsity,blocking,dtype,trans_a,trans_b", [
    (1024, 256, 2048, 0.5, 128, torch.bfloat16, False, False),   # more blocks than compute units: 2 x 2 and 1 x 2 tiles
    (512, 128, 512, 0.5, 128, torch.float16, True, True),        # few blocks: one block per workgroup
    (512, 96, 512, 0.6, 128, torch.bfloat16, False, True),       # k not a multiple of the K-tile: register staging
    (2048, 128, 2048, 0.7, 64, torch.float16, False, False),     # 64-blocks, tiles of up to 4 x 4 blocks
    (256, 96, 256, 0.5, 64, torch.bfloat16, True, False),        # 64-blocks, k split over the wavefronts
])
def test_sdd_fused_against_oracle(m, k, n, sparsity, blocking, dtype, trans_a, trans_b, activation, with_multiplier):
    _seed("sdd_fused", m, k, n, blocking, dtype, activation, with_multiplier)
    lhs, rhs, topo_m, mult = _fused_case(m, k, n, sparsity, blocking, dtype, trans_a, trans_b)
    out = stk.ops.sdd_fused(lhs, rhs, topo_m, activation=activation, multiplier=mult if with_multiplier else None)
    assert isinstance(out, stk.Matrix) and out.data.shape == topo_m.data.shape and out.dtype == dtype
    want = O.sdd_fused(U.np32(lhs), U.np32(rhs), U.topo_of(topo_m), activation, U.np32(mult.data) if with_multiplier else None)
    # the oracle's fp32 values against the kernel's, which are rounded to 16 bits once or (with a multiplier) twice
    U.assert_close(out.data, want, dtype, f"sdd_fused {activation} mul={with_multiplier}")
    # ... and the passes the fused store replaces, run one after the other on the rounded values
    plain = stk.ops.sdd(lhs, rhs, topo_m)
    unfused = _TORCH_ACTIVATIONS[activation](plain.data.float()).to(dtype)
    if with_multiplier:
        unfused = stk.ops.mul(stk.Matrix(topo_m.size(), unfused, *[getattr(topo_m, f) for f in (
            "row_indices", "column_indices", "offsets", "column_indices_t", "offsets_t", "block_offsets_t")]), mult).data
    if activation in (None, "relu"):
        assert torch.equal(out.data, unfused)     # these commute with the rounding: bit-identical
    else:
        # the separate passes round three times (sum, activation, product), the fused store twice, each up to
        # half an ulp (2^-9 for bfloat16): they may differ by 2.5 such steps, more than either does from the oracle
        assert np.allclose(U.np32(out.data), U.np32(unfused), rtol=2e-2, atol=2e-2)


def test_sdd_fused_dmoe_gated_layer():
    # gate(x W1) * (x V1) of a gated MoE layer on a ragged dMoE topology: 2 x 2-block tiles, odd rows
    tokens = np.array([300, 0, 129, 1, 640, 128, 77, 256])
    topo, tm, x, w1, _ = _dmoe_case(tokens, 256, 512, 128, torch.bfloat16, 5)
    v1 = (torch.randn(w1.shape, generator=torch.Generator().manual_seed(6)) * 0.02).to(w1.dtype).to(DEV)
    x = x * 20
    up = stk.ops.sdd(x, v1, tm)
    out = stk.ops.sdd_fused(x, w1, tm, activation="silu", multiplier=up)
    want = O.sdd_fused(U.np32(x), U.np32(w1), topo, "silu", U.np32(up.data))
    U.assert_close(out.data, want, torch.bfloat16, "gated dmoe layer")


@pytest.mark.parametrize("activation,with_multiplier", [("gelu_tanh", False), ("silu", True), (None, True), ("relu", False), ("gelu", True)])
@pytest.mark.parametrize("trans_a,trans_b", [(False, False), (True, True)])
@pytest.mark.parametrize("save_sums", (False, True))
def test_sdd_fused_gradients(activation, with_multiplier, trans_a, trans_b, save_sums):
    # backward recomputes the sums, or reads the kept ones; checked against torch autograd on the dense fp32 product
    # gathered to blocks, under the north-star tolerance and the two scale-free bounds
    _seed("sdd_fused_grad", activation, with_multiplier, trans_a, trans_b)
    m, k, n, b, dtype = 512, 128, 768, 128, torch.bfloat16
    a = _dense(*((k, m) if trans_a else (m, k)), dtype, std=0.3)
    bb = _dense(*((n, k) if trans_b else (k, n)), dtype, std=0.3)
    lhs, rhs = (a.t() if trans_a else a), (bb.t() if trans_b else bb)
    _, topo_m = _dense_and_sparse(m, n, 0.5, b, dtype)
    mult = None
    if with_multiplier:
        values = torch.randn(topo_m.data.shape).to(dtype).to(DEV).requires_grad_(True)
        mult = stk.Matrix(topo_m.size(), values, topo_m.row_indices, topo_m.column_indices, topo_m.offsets,
                          topo_m.column_indices_t, topo_m.offsets_t, topo_m.block_offsets_t)
    weight = (torch.randn(topo_m.data.shape) * 0.1).to(dtype).to(DEV)
    out = stk.ops.sdd_fused(lhs, rhs, topo_m, activation=activation, multiplier=mult, save_sums=save_sums)
    (out.data.float() * weight.float()).sum().backward()

    lf, rf = lhs.detach().float().requires_grad_(True), rhs.detach().float().requires_grad_(True)
    blocks = (lf @ rf).view(m // b, b, n // b, b).permute(0, 2, 1, 3)[topo_m.row_indices.long(), topo_m.column_indices.long()]
    ref = _TORCH_ACTIVATIONS[activation](blocks)
    mf = None
    if with_multiplier:
        mf = mult.data.detach().float().requires_grad_(True)
        ref = ref * mf
    (ref * weight.float()).sum().backward()
    U.assert_close(out.data, U.np32(ref), dtype, "fused forward")
    U.assert_close(a.grad, U.np32(lf.grad.t() if trans_a else lf.grad), dtype, "fused grad wrt lhs")
    U.assert_close(bb.grad, U.np32(rf.grad.t() if trans_b else rf.grad), dtype, "fused grad wrt rhs")
    if with_multiplier:
        U.assert_close(mult.data.grad, U.np32(mf.grad), dtype, "fused grad wrt multiplier")
        assert mult.data.grad.dtype == dtype
        U.assert_close_scaled(mult.data.grad, mf.grad, dtype, "fused grad wrt multiplier")
    U.assert_close_scaled(a.grad, lf.grad.t() if trans_a else lf.grad, dtype, "fused grad wrt lhs")
    U.assert_close_scaled(bb.grad, rf.grad.t() if trans_b else rf.grad, dtype, "fused grad wrt rhs")


@pytest.mark.parametrize("blocking,dtype", [(128, torch.bfloat16), (128, torch.float16), (64, torch.float16), (64, torch.bfloat16)])
@pytest.mark.parametrize("m,k,n,sparsity", [(384, 128, 512, 0.5), (2048, 256, 2048, 0.7), (256, 96, 256, 0.0)])
def test_sdd_fused_keeps_the_sums(m, k, n, sparsity, blocking, dtype):
    # the second output of stk_sdd_fused_sums is the plain sdd, bit for bit, and the first is unchanged by it; the
    # element-wise pass over the kept sums is within the tolerance of the product that applies the derivative itself
    _seed("sdd_fused_sums", m, k, n, blocking, dtype)
    lhs, rhs, topo_m, g = _fused_case(m, k, n, sparsity, blocking, dtype)
    from stk_amd.backend import hip_kernels
    meta = (topo_m.offsets, topo_m.row_indices, topo_m.column_indices)
    plain, fused = torch.empty_like(topo_m.data), torch.empty_like(topo_m.data)
    hip_kernels.sdd(lhs, rhs, tuple(topo_m.size()), plain, *meta)
    hip_kernels.sdd_fused(lhs, rhs, tuple(topo_m.size()), fused, *meta, "gelu_tanh", g.data)
    out, sums = torch.full_like(plain, float("nan")), torch.full_like(plain, float("nan"))
    hip_kernels.sdd_fused(lhs, rhs, tuple(topo_m.size()), out, *meta, "gelu_tanh", g.data, sums=sums)
    assert torch.equal(sums.view(torch.int16), plain.view(torch.int16))
    assert torch.equal(out.view(torch.int16), fused.view(torch.int16))
    for kind in ("gelu_tanh_grad", "silu_grad", "relu_grad", "gelu_grad", "relu", "gelu"):
        # (on the kept, rounded sums: where an activation bends, its derivative at a rounded sum is not within the
        # tolerance of its derivative at the fp32 sum, which is what the product that recomputes the sums uses)
        want = O.activation(U.np32(sums).astype(np.float64), kind) * U.np32(g.data).astype(np.float64)
        U.assert_close(hip_kernels.activation_product(sums, g.data, kind), want, dtype, kind)
    assert torch.equal(hip_kernels.activation_product(sums, None, None), sums)


@pytest.mark.parametrize("blocking,dtype", [(128, torch.bfloat16), (64, torch.float16)])
@pytest.mark.parametrize("activation", ["relu", "gelu_tanh", "gelu", "silu"])
def test_sdd_store_applies_the_derivative_of_an_activation(activation, blocking, dtype):
    # the backward pass of sdd_fused in one launch: act'(lhs x rhs) * incoming gradient
    _seed("sdd_fused_derivative", activation, blocking, dtype)
    lhs, rhs, topo_m, g = _fused_case(384, 128, 512, 0.5, blocking, dtype)
    from stk_amd.backend import hip_kernels
    out = torch.empty_like(topo_m.data)
    hip_kernels.sdd_fused(lhs, rhs, tuple(topo_m.size()), out, topo_m.offsets, topo_m.row_indices, topo_m.column_indices,
                          activation + "_grad", g.data)
    want = O.sdd_fused(U.np32(lhs), U.np32(rhs), U.topo_of(topo_m), activation + "_grad", U.np32(g.data))
    U.assert_close(out, want, dtype, f"sdd with {activation}' and a multiplier")


def test_sdd_fused_argument_contract():
    lhs, rhs, topo_m, mult = _fused_case(256, 64, 256, 0.5, 128, torch.bfloat16)
    with pytest.raises(ValueError):
        stk.ops.sdd_fused(lhs, rhs, topo_m, activation="swish")
    with pytest.raises(AssertionError):
        stk.ops.sdd_fused(lhs, rhs, topo_m, multiplier=mult.data)           # a Matrix is expected
    other = stk.ops.to_sparse(torch.ones(128, 256, dtype=torch.bfloat16), 128).to(DEV)
    with pytest.raises(AssertionError):
        stk.ops.sdd_fused(lhs, rhs, topo_m, multiplier=other)               # another shape
    with pytest.raises(Exception):
        stk.ops.sdd_fused(lhs.cpu(), rhs.cpu(), topo_m)                     # no host implementation: fails loudly


@pytest.mark.parametrize("blocking", [64, 128])
@pytest.mark.parametrize("k", [32, 96, 160])
def test_sdd_inner_dimension_not_a_multiple_of_the_k_tile(k, blocking):
    # k only has to be divisible by 32 (stk/backend/triton_kernels.py:18); the kernels step by 64
    _seed("ktail", k, blocking)
    dtype = torch.bfloat16
    a, b = _dense(2 * blocking, k, dtype).detach(), _dense(3 * blocking, k, dtype).detach()
    _, topo_m = _dense_and_sparse(2 * blocking, 3 * blocking, 0.34, blocking, dtype)
    topo = U.topo_of(topo_m)
    U.assert_close(stk.ops.sdd(a, b.t(), topo_m).data, O.sdd(U.np32(a), U.np32(b).T, topo), dtype, "sdd nt")
    U.assert_close(stk.ops.sdd(a.t().contiguous().t(), b.t().contiguous(), topo_m).data, O.sdd(U.np32(a), U.np32(b).T, topo), dtype, "sdd tn")


@pytest.mark.parametrize("blocking", [64, 128])
def test_int32_indices_and_ragged_pattern(blocking):
    _seed("i32", blocking)
    dtype = torch.bfloat16
    b = blocking
    rows, cols = 6 * b, 5 * b
    mask = torch.zeros(6, 5)
    mask[0, :] = 1          # full row
    mask[2, 3] = 1          # single block; rows 1, 3, 5 and column 1.. partly empty
    mask[4, 0] = mask[4, 4] = 1
    mask[:, 1] = 0
    dense = (torch.randn(rows, cols) * 0.1 * mask.repeat_interleave(b, 0).repeat_interleave(b, 1)).to(dtype)
    s16 = stk.ops.to_sparse(dense, b).to(DEV)
    s32 = stk.Matrix(s16.size(), s16.data, s16.row_indices.int(), s16.column_indices.int(), s16.offsets)
    assert s32.column_indices_t.dtype == torch.int32
    topo = U.topo_of(s16)
    x = _dense(cols, 2 * b, dtype).detach()
    y = _dense(2 * b, rows, dtype).detach()
    for s in (s16, s32):
        U.assert_close(stk.ops.dsd(s, x), O.dsd((rows, cols), U.np32(s.data), topo, False, U.np32(x)), dtype, "dsd")
        U.assert_close(stk.ops.dsd(s.t(), y.t()), O.dsd((cols, rows), U.np32(s.data), topo, True, U.np32(y).T), dtype, "dsd t")
        U.assert_close(stk.ops.dds(y, s), O.dds(U.np32(y), (rows, cols), U.np32(s.data), topo, False), dtype, "dds")
        U.assert_close(stk.ops.dds(x.t(), s.t()), O.dds(U.np32(x).T, (cols, rows), U.np32(s.data), topo, True), dtype, "dds t")
        U.assert_close(stk.ops.sdd(y.t(), x.t(), s).data, O.sdd(U.np32(y).T, U.np32(x).T, topo), dtype, "sdd")
    # rows of the output that meet no block are exact zeros
    out = stk.ops.dsd(s16, x)
    for r in (1, 3, 5):
        assert bool((out[r * b:(r + 1) * b] == 0).all())


@pytest.mark.parametrize("blocking", [64, 128])
def test_empty_sparse_operand(blocking):
    dtype = torch.float16
    b = blocking
    s = stk.ops.to_sparse(torch.zeros(2 * b, 3 * b, dtype=dtype), b).to(DEV)
    x = _dense(3 * b, 128, dtype).detach()
    y = _dense(b, 2 * b, dtype).detach()
    assert bool((stk.ops.dsd(s, x) == 0).all())
    assert bool((stk.ops.dds(y, s) == 0).all())
    assert stk.ops.sdd(x.new_zeros(2 * b, 64), x.new_zeros(64, 3 * b), s).data.shape == (0, b, b)


def test_dimension_contract():
    # same triggers as stk/backend/triton_kernels.py:15-19, 243, 299, 351
    dtype = torch.float16
    s = stk.ops.to_sparse(torch.ones(256, 256, dtype=dtype), 128).to(DEV)
    with pytest.raises(AssertionError):
        stk.ops.dsd(s, torch.zeros(128, 128, dtype=dtype, device=DEV))        # inner dimension
    with pytest.raises(AssertionError):
        stk.ops.dsd(s, torch.zeros(256, 64, dtype=dtype, device=DEV))         # n not divisible by the blocking
    with pytest.raises(AssertionError):
        stk.ops.dds(torch.zeros(128, 128, dtype=dtype, device=DEV), s)
    with pytest.raises(AssertionError):
        stk.ops.sdd(torch.zeros(256, 48, dtype=dtype, device=DEV), torch.zeros(48, 256, dtype=dtype, device=DEV), s)  # k % 32
    with pytest.raises(AssertionError):
        stk.ops.sdd(torch.zeros(256, 64, dtype=dtype, device=DEV), torch.zeros(32, 256, dtype=dtype, device=DEV), s)


def test_unaligned_views_are_accepted():
    # a row-offset view keeps 16-byte alignment only by luck; odd element offsets force the copy path
    dtype = torch.bfloat16
    _seed("views")
    s_dense, s = _dense_and_sparse(256, 256, 0.5, 128, dtype)
    big = (torch.randn(256, 300) * 0.1).to(dtype).to(DEV)
    rhs = big[:, 3:259]                    # stride 300, offset 3 elements: not 16-byte aligned
    want = O.dsd((256, 256), U.np32(s.data), U.topo_of(s), False, U.np32(rhs))
    U.assert_close(stk.ops.dsd(s, rhs), want, dtype, "dsd with an unaligned view")


def test_config2_uniform_random_all_variants():
    # 4096 x 4096, blocking 128, 25 % of the blocks, bf16 ~ N(0, 0.02)
    dtype = torch.bfloat16
    np.random.seed(2)
    torch.manual_seed(2)
    n = 4096
    mask = stk.random.dense_mask(n, n, 0.75, 128)
    s_dense = (torch.randn(n, n) * 0.02 * mask).to(dtype)
    s = stk.ops.to_sparse(s_dense, 128).to(DEV)
    assert s.data.shape[0] == 256
    topo = U.topo_of(s)
    x = (torch.randn(n, n) * 0.02).to(dtype).to(DEV)
    data32, x32 = U.np32(s.data), U.np32(x)
    for ta, tb in _TRANSPOSE:
        lhs_s = s.t() if ta else s
        rhs = x.t() if tb else x
        rhs32 = x32.T if tb else x32
        U.assert_close(stk.ops.dsd(lhs_s, rhs), O.dsd((n, n), data32, topo, ta, rhs32), dtype, f"dsd {ta} {tb}")
        U.assert_close(stk.ops.dds(rhs, lhs_s), O.dds(rhs32, (n, n), data32, topo, ta), dtype, f"dds {tb} {ta}")
        lhs = x.t() if ta else x
        lhs32 = x32.T if ta else x32
        U.assert_close(stk.ops.sdd(lhs, rhs, s).data, O.sdd(lhs32, rhs32, topo), dtype, f"sdd {ta} {tb}")


@pytest.mark.parametrize("slice_last_round", [True, False])
def test_random_pattern_dealt_by_stripes_of_the_dense_operand(slice_last_round, monkeypatch):
    # a random pattern with enough work for the eight-wave kernels and a dense operand of 2048 columns: the plan tells
    # the launches to deal the lone lines to the compute dies by stripes of the dense operand (in the dsd with a sliced
    # last round: the lines of its whole rounds).  A few repeated rows make pairs, whose tiles lie in front of the lone
    # lines' in the grid.  Against the oracle, bit for bit against the launches without a plan (no slicing), and through
    # the joint launch of an sdd and a dsd, where the list of lone lines starts anywhere in the grid.
    from stk_amd.backend import hip_kernels
    monkeypatch.setattr(hip_kernels, "SLICE_LAST_ROUND", slice_last_round)
    dtype = torch.bfloat16
    rng = np.random.RandomState(5)
    mask = rng.rand(48, 40) < 0.5
    mask[7] = mask[6]
    mask[21] = mask[20]
    mask[22] = mask[20]
    dense = torch.from_numpy(np.kron(mask, np.ones((128, 128), dtype=np.float32)))
    values = (torch.randn(dense.shape, generator=torch.Generator().manual_seed(5)) * 0.05).to(dtype) * dense.to(dtype)
    s = stk.ops.to_sparse(torch.where((dense > 0) & (values == 0), torch.ones_like(values), values).to(DEV), 128)
    topo = U.topo_of(s)
    rows, cols = s.size()
    g = torch.Generator().manual_seed(6)
    b = (torch.randn(cols, 2048, generator=g) * 0.05).to(dtype).to(DEV)
    bt = (torch.randn(rows, 2048, generator=g) * 0.05).to(dtype).to(DEV)
    a = (torch.randn(2048, rows, generator=g) * 0.05).to(dtype).to(DEV)
    plan = hip_kernels.fusion_plan(s.offsets, s.column_indices, s.offsets_t, s.column_indices_t).cpu().numpy()
    br, bc, nnz = rows // 128, cols // 128, s.data.shape[0]
    hints = plan[8 + 8 * ((nnz + br + 1) // 2) + (3 * (br + bc) + 3) // 4 * 4 + 4 * 5 * (2 + br + bc):]
    assert 0 < hints[22] <= 16 and 0 < hints[32 + 23] <= 16, "the plan asks for stripes at this width"
    data32 = U.np32(s.data)
    got = {"dsd": stk.ops.dsd(s, b), "dsd t": stk.ops.dsd(s.t(), bt), "dds": stk.ops.dds(a, s), "dds t": stk.ops.dds(b.t(), s.t())}
    U.assert_close(got["dsd"], O.dsd((rows, cols), data32, topo, False, U.np32(b)), dtype, "dsd")
    U.assert_close(got["dsd t"], O.dsd((cols, rows), data32, topo, True, U.np32(bt)), dtype, "dsd t")
    U.assert_close(got["dds"], O.dds(U.np32(a), (rows, cols), data32, topo, False), dtype, "dds")
    U.assert_close(got["dds t"], O.dds(U.np32(b).T, (cols, rows), data32, topo, True), dtype, "dds t")
    if not slice_last_round:
        monkeypatch.setattr(hip_kernels, "FUSION", False)
        plain = {"dsd": stk.ops.dsd(s, b), "dsd t": stk.ops.dsd(s.t(), bt), "dds": stk.ops.dds(a, s), "dds t": stk.ops.dds(b.t(), s.t())}
        monkeypatch.setattr(hip_kernels, "FUSION", True)
        for what in got:
            assert torch.equal(got[what], plain[what]), what
        dy = bt
        ds = torch.empty_like(s.data)
        drhs = torch.empty(cols, 2048, dtype=dtype, device=DEV)
        meta = (s.offsets, s.row_indices, s.column_indices, s.offsets_t, s.column_indices_t, s.block_offsets_t)
        w = (torch.randn(cols, 2048, generator=g) * 0.05).to(dtype).to(DEV)
        hip_kernels.sdd_dsd(s.size(), dy, w.t(), ds, s.data, *meta, True, dy, drhs)
        assert torch.equal(ds, stk.ops.sdd(dy, w.t(), s).data) and torch.equal(drhs, got["dsd t"])


def _dmoe_case(tokens, hidden, ffn, blocking, dtype, seed):
    topo = O.dmoe_topology(tokens, ffn, blocking)
    g = torch.Generator().manual_seed(seed)
    rows, cols = topo.shape
    x = (torch.randn(rows, hidden, generator=g) * 0.02).to(dtype).to(DEV)
    w1 = (torch.randn(hidden, cols, generator=g) * 0.02).to(dtype).to(DEV)
    w2 = (torch.randn(cols, hidden, generator=g) * 0.02).to(dtype).to(DEV)
    nnz = len(topo.row_indices)
    data = torch.empty(nnz, blocking, blocking, dtype=dtype, device=DEV)
    return topo, U.matrix_from_topology(stk, topo, data, DEV), x, w1, w2


@pytest.mark.parametrize("blocking,dtype", [(128, torch.bfloat16), (64, torch.float16)])
def test_dmoe_small_against_oracle(blocking, dtype):
    # scaled-down dMoE FFN (ragged experts, one empty, one large) checked in full against the oracle
    tokens = np.array([300, 0, 129, 1, 640, 128, 77, 256])
    topo, tm, x, w1, w2 = _dmoe_case(tokens, 256, 512, blocking, dtype, 3)
    h = stk.ops.sdd(x, w1, tm)
    want_h = O.sdd(U.np32(x), U.np32(w1), topo)
    U.assert_close(h.data, want_h, dtype, "dmoe sdd")
    y = stk.ops.dsd(h, w2)
    U.assert_close(y, O.dsd(topo.shape, U.np32(h.data), topo, False, U.np32(w2)), dtype, "dmoe dsd")
    dw1 = stk.ops.dds(x.t(), h)          # weight gradient shape of layer 0: walks the CSC metadata
    U.assert_close(dw1, O.dds(U.np32(x).T, topo.shape, U.np32(h.data), topo, False), dtype, "dmoe dds")
    dw2 = stk.ops.dsd(h.t(), x)          # transposed sparse lhs: block_offsets_t gather
    U.assert_close(dw2, O.dsd((topo.shape[1], topo.shape[0]), U.np32(h.data), topo, True, U.np32(x)), dtype, "dmoe dsd t")


@pytest.mark.parametrize("b", [128, 64])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hidden", [256, 2048])
def test_dsd_runs_of_identical_rows(hidden, dtype, b):
    # block rows in runs of 1..7 identical rows (and an expert without tokens): pairs become 256-row
    # tiles, the last three rows of an odd run one 384-row tile; the dense operand also as a .t() view.
    # (hidden 256: little work per compute unit, which runs on four-wave 128x128 tiles instead)
    # With 64-blocks the same token counts give runs of 2..14 rows (and one of 1): fours, threes, pairs, a lone row.
    tokens = np.array([128, 256, 0, 384, 512, 640, 768, 896, 100, 60])
    topo, tm, x, w1, w2 = _dmoe_case(tokens, hidden, 4096, b, dtype, 5)
    g = torch.Generator().manual_seed(11)
    h = stk.Matrix(tm.size(), (torch.randn(tm.data.shape, generator=g) * 0.05).to(dtype).to(DEV), tm.row_indices, tm.column_indices, tm.offsets)
    want = O.dsd(topo.shape, U.np32(h.data), topo, False, U.np32(w2))
    U.assert_close(stk.ops.dsd(h, w2), want, dtype, "dsd runs")
    w2t = w2.t().contiguous()
    U.assert_close(stk.ops.dsd(h, w2t.t()), want, dtype, "dsd runs, transposed view")
    # identical columns walked through the transpose metadata: three block columns per expert
    tokens = np.array([300, 128, 650]) if hidden == 256 else np.array([3000, 1280, 6500, 2000, 4000])
    topo, tm, x, w1, w2 = _dmoe_case(tokens, hidden if hidden == 256 else 4096, 384, b, dtype, 6)
    h = stk.Matrix(tm.size(), (torch.randn(tm.data.shape, generator=g) * 0.05).to(dtype).to(DEV), tm.row_indices, tm.column_indices, tm.offsets)
    U.assert_close(stk.ops.dsd(h.t(), x), O.dsd((topo.shape[1], topo.shape[0]), U.np32(h.data), topo, True, U.np32(x)), dtype, "dsd t, runs of three columns")
    # dds over the same runs: identical block columns (three or six per expert) and, transposed, identical block rows
    U.assert_close(stk.ops.dds(x.t(), h), O.dds(U.np32(x).T, topo.shape, U.np32(h.data), topo, False), dtype, "dds, runs of columns")
    v = _dense(256, topo.shape[1], dtype, 0.05).detach()
    U.assert_close(stk.ops.dds(v, h.t()), O.dds(U.np32(v), (topo.shape[1], topo.shape[0]), U.np32(h.data), topo, True), dtype, "dds t, runs of rows")


@pytest.mark.parametrize("b", [128, 64])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_sdd_runs_of_identical_rows_with_odd_and_even_lengths(dtype, b):
    # sdd takes its tiles from the plan: rows in runs of 1..5 identical rows (2x2-block tiles over row pairs,
    # 1x2 over the odd row out), rows of odd and even lengths (a row of odd length ends with a tile of one
    # block, also in the 2x2 case), empty rows in between, rows starting at odd block ids.  With 64-blocks the
    # tiles are up to 4x4 blocks: fours of rows, then a pair, then a single row; up to four blocks wide.
    rng = np.random.RandomState(4)
    rows = []
    width = 48
    # (more blocks than compute units, so that sdd takes the fused tiles and not one block per workgroup)
    for n, blocks in [(1, 11), (2, 21), (3, 5), (4, 8), (5, 13), (2, 32), (1, 1), (3, 19), (2, 6), (7, 9), (6, 2), (9, 7)]:
        pattern = np.zeros(width, bool)
        pattern[rng.choice(width, blocks, replace=False)] = True
        rows += [pattern] * n + ([np.zeros(width, bool)] if n % 2 else [])
    mask = torch.from_numpy(np.array(rows))
    _seed("sdd runs", str(dtype), b)
    dense = (torch.randn(mask.shape[0] * b, width * b) * 0.05 * mask.float().repeat_interleave(b, 0).repeat_interleave(b, 1)).to(dtype)
    topo_m = stk.ops.to_sparse(dense, b).to(DEV)
    assert topo_m.data.shape[0] > torch.cuda.get_device_properties(0).multi_processor_count
    topo = U.topo_of(topo_m)
    for k in (64, 160, 256):
        x = _dense(mask.shape[0] * b, k, dtype, 0.05).detach()
        w = _dense(k, width * b, dtype, 0.05).detach()
        U.assert_close(stk.ops.sdd(x, w, topo_m).data, O.sdd(U.np32(x), U.np32(w), topo), dtype, f"sdd runs, k={k}")
        wt = w.t().contiguous()
        U.assert_close(stk.ops.sdd(x, wt.t(), topo_m).data, O.sdd(U.np32(x), U.np32(w), topo), dtype, f"sdd runs, k={k}, rhs as a .t() view")


@pytest.mark.parametrize("blocks", [65, 130])
def test_lines_longer_than_the_lane_resident_walk_table(blocks):
    # dsd / dds hold 64 walk entries of a line at a time (one per lane); longer lines run the K loop in chunks
    dtype = torch.bfloat16
    b = 128
    _seed("long", blocks)
    rows, cols = 3 * b, blocks * b
    mask = torch.ones(3, blocks)
    mask[2, 1::2] = 0            # rows 0 and 1 identical (a fused pair), row 2 a lone row with half of the blocks
    dense = (torch.randn(rows, cols) * 0.05 * mask.repeat_interleave(b, 0).repeat_interleave(b, 1)).to(dtype)
    s = stk.ops.to_sparse(dense, b).to(DEV)
    topo = U.topo_of(s)
    x = _dense(cols, 256, dtype, 0.05).detach()
    y = _dense(256, rows, dtype, 0.05).detach()
    U.assert_close(stk.ops.dsd(s, x), O.dsd((rows, cols), U.np32(s.data), topo, False, U.np32(x)), dtype, "dsd long rows")
    U.assert_close(stk.ops.dds(x.t(), s.t()), O.dds(U.np32(x).T, (cols, rows), U.np32(s.data), topo, True), dtype, "dds t long rows")
    U.assert_close(stk.ops.dsd(s.t(), y.t()), O.dsd((cols, rows), U.np32(s.data), topo, True, U.np32(y).T), dtype, "dsd t short columns")
    # and long columns: the transposed pattern stored as its own matrix
    st = stk.ops.to_sparse(dense.t().contiguous(), b).to(DEV)
    topo_t = U.topo_of(st)
    U.assert_close(stk.ops.dds(y, st.t()), O.dds(U.np32(y), (rows, cols), U.np32(st.data), topo_t, True), dtype, "dds t short rows")
    U.assert_close(stk.ops.dds(x.t(), st), O.dds(U.np32(x).T, (cols, rows), U.np32(st.data), topo_t, False), dtype, "dds long columns")
    U.assert_close(stk.ops.dsd(st.t(), x), O.dsd((rows, cols), U.np32(st.data), topo_t, True, U.np32(x)), dtype, "dsd t long columns")


@pytest.mark.parametrize("b", [128, 64])
def test_results_do_not_depend_on_the_fusion_plan(monkeypatch, b):
    # identical rows / columns computed as fused tiles (pairs, threes; fours with 64-blocks) or one line at a time:
    # every output element accumulates its k-steps in the same order, so the results are equal bit for bit (as long
    # as dsd does not cut tiles along k, which needs its workspace)
    from stk_amd.backend import hip_kernels
    monkeypatch.setattr(hip_kernels, "SLICE_LAST_ROUND", False)
    dtype = torch.bfloat16
    tokens = np.array([300, 0, 129, 384, 640, 128, 77, 256, 40])
    topo, tm, x, w1, w2 = _dmoe_case(tokens, 4096, 4096, b, dtype, 9)    # enough work for the fused tiles of all three

    h0 = stk.ops.sdd(x, w1, tm)

    def run():
        h = stk.ops.sdd(x, w1, tm)
        return h.data.clone(), stk.ops.dsd(h0, w2), stk.ops.dds(x.t(), h0), stk.ops.dsd(h0.t(), x), stk.ops.dds(w1, h0.t())

    fused = run()
    monkeypatch.setattr(hip_kernels, "FUSION", False)
    plain = run()
    for a, c, what in zip(fused, plain, ("sdd", "dsd", "dds", "dsd t", "dds t")):
        if what == "sdd" and b == 64:
            # without a plan a 64-block is computed with k split over the four wavefronts of its workgroup and the
            # partial sums added at the end: the same sums in another order
            U.assert_close_scaled(a, c.float(), dtype, "sdd, 64-blocks with and without a plan")
        else:
            assert torch.equal(a, c), what
    U.assert_close(plain[1], O.dsd(topo.shape, U.np32(h0.data), topo, False, U.np32(w2)), dtype, "dsd without plan")


_JOINT_TOKENS = [300, 0, 129, 384, 640, 128, 77, 256, 512, 1000, 40, 896]
# (dtype, blocking, hidden, ffn, tokens per expert); the first two have the work per compute unit that the joint launches
# ask for (nonzero blocks x hidden / 128 >= 40 x 256 compute units), the others run the two products one after the other
_JOINT_CASES = [(torch.bfloat16, 128, 1024, 4096, _JOINT_TOKENS + [512, 384, 640, 512]),
                (torch.float16, 128, 1024, 4096, _JOINT_TOKENS + [256] * 8),
                (torch.float16, 128, 512, 2048, _JOINT_TOKENS), (torch.bfloat16, 128, 256, 2048, _JOINT_TOKENS),
                (torch.bfloat16, 128, 384, 4096, _JOINT_TOKENS + [512] * 6), (torch.float16, 64, 1024, 2048, _JOINT_TOKENS)]


@pytest.mark.parametrize("dtype,blocking,hidden,ffn,tokens", _JOINT_CASES)
def test_both_gradients_of_sdd_in_one_call(dtype, blocking, hidden, ffn, tokens, monkeypatch):
    # stk_dsd_dds: dS rhs^T and lhs^T dS from one call (one launch for 128-blocks with enough work; otherwise the two
    # products one after the other) against the oracle's dsd and dds, and bit for bit against the separate launches
    from stk_amd.backend import autograd, hip_kernels
    monkeypatch.setattr(hip_kernels, "SLICE_LAST_ROUND", False)
    topo, tm, x, w1, w2 = _dmoe_case(np.array(tokens), hidden, ffn, blocking, dtype, 31)
    g = torch.Generator().manual_seed(32)
    ds = (torch.randn(tm.data.shape, generator=g) * 0.05).to(dtype).to(DEV)
    dsm = stk.Matrix(tm.size(), ds, tm.row_indices, tm.column_indices, tm.offsets, tm.column_indices_t, tm.offsets_t, tm.block_offsets_t)
    rows, cols = tm.size()
    dx = torch.full((rows, hidden), float("nan"), dtype=dtype, device=DEV)
    dw1 = torch.full((hidden, cols), float("nan"), dtype=dtype, device=DEV)
    hip_kernels.dsd_dds(tm.size(), ds, tm.offsets, tm.row_indices, tm.column_indices, tm.offsets_t, tm.column_indices_t, tm.block_offsets_t,
                        w1.t(), dx, x.t(), dw1)
    U.assert_close(dx, O.dsd(topo.shape, U.np32(ds), topo, False, U.np32(w1).T), dtype, "dS W1^T")
    U.assert_close(dw1, O.dds(U.np32(x).T, topo.shape, U.np32(ds), topo, False), dtype, "x^T dS")
    assert torch.equal(dx, stk.ops.dsd(dsm, w1.t())) and torch.equal(dw1, stk.ops.dds(x.t(), dsm))
    # through autograd: the gradients of sdd with the joint call and with two launches
    grads = {}
    for joint in (True, False):
        monkeypatch.setattr(autograd, "JOINT_GRADIENTS", joint)
        xs, ws = x.detach().clone().requires_grad_(True), w1.detach().clone().requires_grad_(True)
        stk.ops.sdd(xs, ws, tm).data.backward(ds)
        grads[joint] = (xs.grad, ws.grad)
    assert torch.equal(grads[True][0], grads[False][0]) and torch.equal(grads[True][1], grads[False][1])
    assert torch.equal(grads[True][0], dx) and torch.equal(grads[True][1], dw1)


@pytest.mark.parametrize("dtype,blocking,hidden,ffn,tokens", _JOINT_CASES)
def test_both_gradients_of_sdd_with_a_transposed_rhs_in_one_call(dtype, blocking, hidden, ffn, tokens, monkeypatch):
    # stk_dsd_dsd: for S = x W^T with W stored [columns of S, hidden], dS W and dS^T x from one call (one launch for
    # 128-blocks with enough work; otherwise the two products one after the other) against the oracle's dsd, and bit for
    # bit against the separate launches
    from stk_amd.backend import autograd, hip_kernels
    monkeypatch.setattr(hip_kernels, "SLICE_LAST_ROUND", False)
    topo, tm, x, w1, w2 = _dmoe_case(np.array(tokens), hidden, ffn, blocking, dtype, 35)
    w = w2                                                   # [columns of S, hidden], row-major
    g = torch.Generator().manual_seed(36)
    ds = (torch.randn(tm.data.shape, generator=g) * 0.05).to(dtype).to(DEV)
    dsm = stk.Matrix(tm.size(), ds, tm.row_indices, tm.column_indices, tm.offsets, tm.column_indices_t, tm.offsets_t, tm.block_offsets_t)
    rows, cols = tm.size()
    dx = torch.full((rows, hidden), float("nan"), dtype=dtype, device=DEV)
    dw = torch.full((cols, hidden), float("nan"), dtype=dtype, device=DEV)
    hip_kernels.dsd_dsd(tm.size(), ds, tm.offsets, tm.row_indices, tm.column_indices, tm.offsets_t, tm.column_indices_t, tm.block_offsets_t,
                        w, dx, x, dw)
    U.assert_close(dx, O.dsd(topo.shape, U.np32(ds), topo, False, U.np32(w)), dtype, "dS W")
    U.assert_close(dw, O.dsd((cols, rows), U.np32(ds), topo, True, U.np32(x)), dtype, "dS^T x")
    assert torch.equal(dx, stk.ops.dsd(dsm, w)) and torch.equal(dw, stk.ops.dsd(dsm.t(), x))
    # through autograd: the gradients of sdd(x, W^T) with the joint call and with two launches
    grads = {}
    for joint in (True, False):
        monkeypatch.setattr(autograd, "JOINT_GRADIENTS", joint)
        xs, ws = x.detach().clone().requires_grad_(True), w.detach().clone().requires_grad_(True)
        stk.ops.sdd(xs, ws.t(), tm).data.backward(ds)
        grads[joint] = (xs.grad, ws.grad)
    assert torch.equal(grads[True][0], grads[False][0]) and torch.equal(grads[True][1], grads[False][1])
    assert torch.equal(grads[True][0], dx) and torch.equal(grads[True][1], dw)


@pytest.mark.parametrize("transpose_a", [False, True])
@pytest.mark.parametrize("dtype,blocking,hidden,ffn,tokens", _JOINT_CASES)
def test_both_gradients_of_dsd_in_one_call(dtype, blocking, hidden, ffn, tokens, transpose_a, monkeypatch):
    # stk_sdd_dsd: dy rhs^T on the pattern and op(S)^T dy from one call (one launch for 128-blocks with enough work;
    # otherwise the two products one after the other) against the oracle's sdd and dsd, and bit for bit against the
    # separate launches
    from stk_amd.backend import autograd, hip_kernels
    monkeypatch.setattr(hip_kernels, "SLICE_LAST_ROUND", False)
    topo, tm, x, w1, w2 = _dmoe_case(np.array(tokens), hidden, ffn, blocking, dtype, 33)
    g = torch.Generator().manual_seed(34)
    s = (torch.randn(tm.data.shape, generator=g) * 0.05).to(dtype).to(DEV)
    sm = stk.Matrix(tm.size(), s, tm.row_indices, tm.column_indices, tm.offsets, tm.column_indices_t, tm.offsets_t, tm.block_offsets_t)
    rows, cols = tm.size()
    meta = (tm.offsets, tm.row_indices, tm.column_indices, tm.offsets_t, tm.column_indices_t, tm.block_offsets_t)
    # y = S w2 [rows, hidden] or y = S^T x [cols, hidden]
    rhs = x if transpose_a else w2
    dy = (torch.randn(cols if transpose_a else rows, hidden, generator=g) * 0.05).to(dtype).to(DEV)
    ds = torch.full(tuple(s.shape), float("nan"), dtype=dtype, device=DEV)
    drhs = torch.full(tuple(rhs.shape), float("nan"), dtype=dtype, device=DEV)
    lhs, rhs_sdd = (rhs, dy.t()) if transpose_a else (dy, rhs.t())
    hip_kernels.sdd_dsd(tm.size(), lhs, rhs_sdd, ds, s, *meta, not transpose_a, dy, drhs)
    U.assert_close(ds, O.sdd(U.np32(lhs), U.np32(rhs_sdd), topo), dtype, "dy rhs^T on the pattern")
    logical = topo.shape if transpose_a else (cols, rows)
    U.assert_close(drhs, O.dsd(logical, U.np32(s), topo, not transpose_a, U.np32(dy)), dtype, "op(S)^T dy")
    assert torch.equal(ds, stk.ops.sdd(lhs, rhs_sdd, tm).data)
    assert torch.equal(drhs, stk.ops.dsd(sm if transpose_a else sm.t(), dy))
    # through autograd: the gradients of dsd with the joint call and with two launches
    grads = {}
    for joint in (True, False):
        monkeypatch.setattr(autograd, "JOINT_DSD_GRADIENTS", joint)
        ss, rs = s.detach().clone().requires_grad_(True), rhs.detach().clone().requires_grad_(True)
        m = stk.Matrix(tm.size(), ss, tm.row_indices, tm.column_indices, tm.offsets, tm.column_indices_t, tm.offsets_t, tm.block_offsets_t)
        stk.ops.dsd(m.t() if transpose_a else m, rs).backward(dy)
        grads[joint] = (ss.grad, rs.grad)
    assert torch.equal(grads[True][0], grads[False][0]) and torch.equal(grads[True][1], grads[False][1])
    assert torch.equal(grads[True][0], ds) and torch.equal(grads[True][1], drhs)


def test_gradients_side_by_side_equal_gradients_one_after_the_other(monkeypatch):
    # backward launches the two gradients of a product on two streams; same kernels, so the same bits
    from stk_amd.backend import autograd
    tokens = np.array([256, 384, 128, 512, 256, 384, 640, 128])
    topo, tm, x, w1, w2 = _dmoe_case(tokens, 256, 512, 128, torch.bfloat16, 21)
    grads = {}
    for overlap in (True, False, True):
        monkeypatch.setattr(autograd, "OVERLAP_GRADIENTS", overlap)
        xs, w1s, w2s = (t.detach().clone().requires_grad_(True) for t in (x, w1, w2))
        h = stk.ops.sdd(xs, w1s, tm)
        y = stk.ops.dsd(h, w2s)
        z = stk.ops.dds(y.t()[:256].contiguous(), h)          # a third product on the same sparse values
        (y.float().square().sum() + z.float().sum()).backward()
        torch.cuda.synchronize()
        got = [xs.grad.clone(), w1s.grad.clone(), w2s.grad.clone()]
        if overlap in grads:
            assert all(torch.equal(a, b) for a, b in zip(got, grads[overlap]))     # and repeatable
        grads[overlap] = got
    assert all(torch.equal(a, b) for a, b in zip(grads[True], grads[False]))
    assert all(torch.isfinite(g.float()).all() and g.float().abs().sum() > 0 for g in grads[True])


def test_products_on_a_second_stream_match_the_default_stream():
    # the launches follow torch's current stream; the fusion plan built on one stream is used from another
    tokens = np.array([256, 384, 128, 512, 256, 384])
    topo, tm, x, w1, w2 = _dmoe_case(tokens, 256, 512, 128, torch.bfloat16, 9)
    h0 = stk.ops.sdd(x, w1, tm)
    y0 = stk.ops.dsd(h0, w2)
    d0 = stk.ops.dds(x.t(), h0)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        h1 = stk.ops.sdd(x, w1, tm)
        y1 = stk.ops.dsd(h1, w2)
        d1 = stk.ops.dds(x.t(), h1)
    side.synchronize()
    assert torch.equal(h0.data, h1.data) and torch.equal(y0, y1) and torch.equal(d0, d1)
    # a topology first seen on the side stream, then used on the default stream
    topo2, tm2, x2, w12, w22 = _dmoe_case(tokens[::-1].copy(), 256, 512, 128, torch.bfloat16, 10)
    with torch.cuda.stream(side):
        ha = stk.ops.sdd(x2, w12, tm2)
    hb = stk.ops.sdd(x2, w12, tm2)
    torch.cuda.synchronize()
    assert torch.equal(ha.data, hb.data)
    U.assert_close(hb.data, O.sdd(U.np32(x2), U.np32(w12), topo2), torch.bfloat16, "sdd after a plan built on another stream")


def _sliced_ran(fn):
    """Runs fn() with the dsd workspace cleared and reports whether the launch cut tiles into slices along k
    (it then wrote partial tiles into the workspace)."""
    from stk_amd.backend import hip_kernels
    for ws, _ in hip_kernels._dsd_workspaces.values():
        ws.zero_()
    out = fn()
    torch.cuda.synchronize()
    touched = False
    for ws, _ in hip_kernels._dsd_workspaces.values():
        touched = touched or bool(ws.count_nonzero().item() > 0)
    return out, touched


def _assert_counters_zero(m, n):
    from stk_amd.backend import hip_kernels
    counters = 4 * torch.cuda.get_device_properties(0).multi_processor_count
    for ws, _ in hip_kernels._dsd_workspaces.values():
        assert ws[:counters].count_nonzero().item() == 0, "counters of the sliced launch are not back at zero"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_dsd_sliced_last_round_dmoe_rows(dtype, monkeypatch):
    # fewer tiles than compute units: dsd cuts them into slices along k, whose partial tiles are added up by the
    # workgroup that finishes last; experts with 1..8 block rows (pairs, threes, lone rows), one without tokens;
    # both rhs layouts; without the fusion plan nothing is cut
    from stk_amd.backend import hip_kernels
    tokens = np.array([128, 256, 0, 384, 512, 640, 768, 896, 100, 300, 1000, 129, 5, 640, 384, 200])
    topo, tm, x, w1, w2 = _dmoe_case(tokens, 1024, 4096, 128, dtype, 21)
    g = torch.Generator().manual_seed(22)
    h = stk.Matrix(tm.size(), (torch.randn(tm.data.shape, generator=g) * 0.02).to(dtype).to(DEV), tm.row_indices, tm.column_indices, tm.offsets)
    y, ran = _sliced_ran(lambda: stk.ops.dsd(h, w2))
    assert ran, "expected tiles cut along k for this shape"
    _assert_counters_zero(*y.shape)
    assert torch.equal(y, stk.ops.dsd(h, w2)), "results must repeat bit for bit whichever workgroup adds the slices up"
    w2t = w2.t().contiguous()
    y_t = stk.ops.dsd(h, w2t.t())
    monkeypatch.setattr(hip_kernels, "FUSION", False)
    y_noplan, ran = _sliced_ran(lambda: stk.ops.dsd(h, w2))
    assert not ran
    monkeypatch.setattr(hip_kernels, "FUSION", True)
    monkeypatch.setattr(hip_kernels, "SLICE_LAST_ROUND", False)
    want, ran = _sliced_ran(lambda: stk.ops.dsd(h, w2))
    assert not ran
    # the unsplit result is the one the other tests pin against the oracle; per expert it is a dense product
    pad = O.padded_tokens_per_expert(tokens, 128)
    hd = stk.ops.to_dense(h)
    r0 = 0
    for e, p in enumerate(pad):
        if p:
            he = hd[r0:r0 + p, e * 4096:(e + 1) * 4096].float()
            U.assert_close(want[r0:r0 + p], U.np32(he @ w2[e * 4096:(e + 1) * 4096].float()), dtype, f"dsd expert {e}")
        r0 += p
    del hd
    assert torch.equal(y_noplan, want)
    for got, what in ((y, "sliced"), (y_t, "sliced, transposed view")):
        U.assert_close(got, U.np32(want), dtype, what)
    _assert_counters_zero(*y.shape)


def test_dsd_sliced_last_round_transposed_and_long_lines():
    from stk_amd.backend import hip_kernels
    dtype = torch.bfloat16
    # transposed operand: the lines are the block columns (4 identical ones per expert, 15..32 blocks each)
    tokens = np.array([2048, 4096, 3000, 1800, 4096, 2200, 2600, 3600])
    topo, tm, x, w1, w2 = _dmoe_case(tokens, 2048, 512, 128, dtype, 23)
    g = torch.Generator().manual_seed(24)
    h = stk.Matrix(tm.size(), (torch.randn(tm.data.shape, generator=g) * 0.02).to(dtype).to(DEV), tm.row_indices, tm.column_indices, tm.offsets)
    dw2, ran = _sliced_ran(lambda: stk.ops.dsd(h.t(), x))
    assert ran
    _assert_counters_zero(*dw2.shape)
    pad = O.padded_tokens_per_expert(tokens, 128)
    hd = stk.ops.to_dense(h)
    r0 = 0
    for e, p in enumerate(pad):
        want = hd[r0:r0 + p, e * 512:(e + 1) * 512].float().t() @ x[r0:r0 + p].float()
        U.assert_close(dw2[e * 512:(e + 1) * 512], U.np32(want), dtype, f"dsd t expert {e}")
        r0 += p
    # eight block rows of 256 blocks: few tiles, cut into more than two slices each, whose partial tiles are
    # added in the order of the slices
    _seed("sliced long")
    rows, cols = 8 * 128, 256 * 128
    s = stk.ops.to_sparse((torch.randn(rows, cols) * 0.02).to(dtype), 128).to(DEV)
    v = _dense(cols, 2048, dtype, 0.02).detach()
    y, ran = _sliced_ran(lambda: stk.ops.dsd(s, v))
    assert ran
    _assert_counters_zero(*y.shape)
    U.assert_close(y, U.np32(stk.ops.to_dense(s).float() @ v.float()), dtype, "dsd long rows, several slices per tile")
    assert torch.equal(y, stk.ops.dsd(s, v))


def test_dsd_sliced_last_round_random_pattern():
    # no repeated rows, 60..90 blocks per row, two rows empty: lone-row tiles cut into slices (an empty row has one)
    dtype = torch.float16
    _seed("sliced random")
    b, rb, cb = 128, 26, 256
    mask = (torch.rand(rb, cb) < 0.3).float()
    mask[3] = 0
    mask[25] = 0
    dense = (torch.randn(rb * b, cb * b) * 0.02 * mask.repeat_interleave(b, 0).repeat_interleave(b, 1)).to(dtype)
    s = stk.ops.to_sparse(dense, b).to(DEV)
    v = _dense(cb * b, 1024, dtype, 0.02).detach()
    y, ran = _sliced_ran(lambda: stk.ops.dsd(s, v))
    assert ran
    _assert_counters_zero(*y.shape)
    U.assert_close(y, U.np32(dense.to(DEV).float() @ v.float()), dtype, "dsd random pattern")
    assert y[3 * b:4 * b].count_nonzero().item() == 0 and y[25 * b:].count_nonzero().item() == 0


def _routed_topology(choices, blocking, ffn, dtype):
    """Expert choices [tokens, top_k] -> (route result, topology Matrix with uninitialised values), both from the
    library's own kernels (stk_route, stk_dmoe_topology), plus the padded rows per expert on the host."""
    r = stk.ops.route(choices.to(DEV), 64, blocking)
    rows = r.row_slots.numel()
    tm = stk.ops.dmoe_topology(r.padded_bins, blocking, rows // blocking, ffn // blocking, dtype=dtype)
    pad = np.diff(np.concatenate([[0], r.padded_bins.cpu().numpy()]))
    return r, tm, pad


def _expert_blocks(values, r0, p, ffn, b):
    """The rows [r0, r0 + p) of a block-diagonal dMoE matrix (one expert) as a dense [p, ffn] tensor, gathered
    from the blocked values [nnz, b, b] (ffn / b blocks per block row, block rows in order)."""
    w, rb0, nb = ffn // b, r0 // b, p // b
    return values[rb0 * w:(rb0 + nb) * w].reshape(nb, w, b, b).permute(0, 2, 1, 3).reshape(p, ffn)


def _check_dmoe_products_full_size(choices, hidden, ffn, blocking, dtype, seed):
    """The six products of a dMoE FFN, forward and backward, at full size on a routed topology.  Too big for the
    CPU oracle inside a test; the block-diagonal structure makes every expert an ordinary dense product, so
    each product is checked expert by expert against fp32 torch.matmul on the GPU on the same 16-bit inputs:
    within the north-star tolerance and within the scale-free bounds of tests/_util.py.  The topology is
    checked bit for bit against the oracle's closed form."""
    r, tm, pad = _routed_topology(choices, blocking, ffn, dtype)
    counts = np.bincount(choices.reshape(-1).numpy(), minlength=64)
    assert np.array_equal(pad, O.padded_tokens_per_expert(counts, blocking))
    U.assert_topology_equal(tm, O.dmoe_topology(counts, ffn, blocking), "routed topology")
    rows, cols = tm.size()
    g = torch.Generator(device=DEV).manual_seed(seed)
    rnd = lambda *shape: (torch.randn(*shape, generator=g, device=DEV) * 0.02).to(dtype)
    x, w1, w2 = rnd(rows, hidden), rnd(hidden, cols), rnd(cols, hidden)
    dy = rnd(rows, hidden)
    h = stk.ops.sdd(x, w1, tm)                 # forward, layer 0
    y = stk.ops.dsd(h, w2)                     # forward, layer 1
    dw1 = stk.ops.dds(x.t(), h)                # weight gradient of layer 0 (h stands in for dh: same topology)
    dw2 = stk.ops.dsd(h.t(), dy)               # weight gradient of layer 1
    dx = stk.ops.dsd(h, w1.t())                # input gradient of layer 0
    dh = stk.ops.sdd(dy, w2.t(), tm)           # gradient of the hidden activations
    assert y.shape == (rows, hidden) and dw1.shape == (hidden, cols) and dw2.shape == (cols, hidden) and dx.shape == (rows, hidden)
    r0 = 0
    for e, p in enumerate(int(v) for v in pad):
        c0, c1 = e * ffn, (e + 1) * ffn
        if p == 0:
            # an expert without tokens owns empty block columns: its weight gradients are exact zeros
            assert dw1[:, c0:c1].count_nonzero().item() == 0 and dw2[c0:c1].count_nonzero().item() == 0, f"expert {e}"
            continue
        xe, dye = x[r0:r0 + p].float(), dy[r0:r0 + p].float()
        w1e, w2e = w1[:, c0:c1].float(), w2[c0:c1].float()
        he = _expert_blocks(h.data, r0, p, ffn, blocking)
        U.assert_close_scaled(he, xe @ w1e, dtype, f"expert {e} sdd(x, W1)")
        hf = he.float()
        U.assert_close_scaled(y[r0:r0 + p], hf @ w2e, dtype, f"expert {e} dsd(h, W2)")
        U.assert_close_scaled(dw1[:, c0:c1], xe.t() @ hf, dtype, f"expert {e} dds(x^T, h)")
        U.assert_close_scaled(dw2[c0:c1], hf.t() @ dye, dtype, f"expert {e} dsd(h^T, dy)")
        U.assert_close_scaled(dx[r0:r0 + p], hf @ w1e.t(), dtype, f"expert {e} dsd(h, W1^T)")
        U.assert_close_scaled(_expert_blocks(dh.data, r0, p, ffn, blocking), dye @ w2e.t(), dtype, f"expert {e} sdd(dy, W2^T)")
        r0 += p
    assert r0 == rows
    # linearity in the dense operand: dsd(h, 2 w2) == 2 dsd(h, w2) exactly (power-of-two scaling), wherever the
    # sum is a normal number of the 16-bit type (float16 rounds sums below 2^-14 on a fixed grid; a rounded value of
    # at least 2^-13 cannot come from such a sum)
    y2 = stk.ops.dsd(h, w2 * 2)
    normal = y.float().abs() >= 2.0 ** -13
    assert torch.equal(y2[normal], (y * 2)[normal]) and float(normal.float().mean()) > 0.9


def _top1_choices(tokens, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(tokens, 64, generator=g).argmax(dim=1, keepdim=True).to(torch.int32)


def test_dmoe_config3_full_size():
    # 16384 tokens, top-1 over 64 experts from N(0, 1) logits, hidden 1024, ffn 4096, blocking 128, bf16
    _check_dmoe_products_full_size(_top1_choices(16384, 0), 1024, 4096, 128, torch.bfloat16, 3)


def test_dmoe_config4_full_size():
    # 32768 tokens, top-2 from Zipf(1.2)-skewed popularity (Gumbel trick), hidden 2048, ffn 8192, blocking 128, bf16
    g = torch.Generator().manual_seed(0)
    logp = -1.2 * torch.log(torch.arange(1, 65, dtype=torch.float64))
    u = torch.rand(32768, 64, generator=g, dtype=torch.float64).clamp_min(1e-300)
    choices = (logp[None, :] - torch.log(-torch.log(u))).topk(2, dim=1).indices.to(torch.int32)
    _check_dmoe_products_full_size(choices, 2048, 8192, 128, torch.bfloat16, 4)


def test_dmoe_config5_full_size():
    # config 3's routing with blocking 64 and fp16
    _check_dmoe_products_full_size(_top1_choices(16384, 0), 1024, 4096, 64, torch.float16, 5)


def test_dmoe_config5_extreme_skew_full_size():
    # one expert takes half of the 16384 tokens, the others share the rest; blocking 64, fp16
    g = torch.Generator().manual_seed(0)
    top = torch.randint(1, 64, (16384,), generator=g, dtype=torch.int32)
    top[torch.randperm(16384, generator=g)[:8192]] = 0
    _check_dmoe_products_full_size(top[:, None], 1024, 4096, 64, torch.float16, 6)


@pytest.mark.parametrize("dtype", _DTYPES + (torch.float32,))
def test_config1_seed0_mask_all_products(dtype):
    """BASELINE configuration 1 on the HIP path: stk.random.mask(1024, 1024, 0.5, 128) from numpy seed 0 (the
    known-answer topology of tests/golden/config1_topology.json), dense operands 1024 x 1024 ~ N(0, 1) from torch
    seed 0 - in fp32 as the configuration states, and rounded to the two 16-bit types - sdd / dsd / dds in all four
    transpose variants against the oracle.  (The configuration on host tensors: tests/test_host_products.py.)  With
    N(0, 1) operands the sums are ~32, far above the absolute tolerance, so the comparison is a relative one."""
    import json
    import os
    np.random.seed(0)
    torch.manual_seed(0)
    s = stk.random.mask(1024, 1024, 0.5, 128)
    with open(os.path.join(os.path.dirname(__file__), "golden", "config1_topology.json")) as f:
        golden = json.load(f)
    for name in ("row_indices", "column_indices", "offsets", "offsets_t", "column_indices_t", "block_offsets_t"):
        assert getattr(s, name).tolist() == golden[name], name
    values = torch.randn(s.data.shape).to(dtype)
    s = stk.Matrix(s.size(), values, s.row_indices, s.column_indices, s.offsets, s.column_indices_t, s.offsets_t, s.block_offsets_t).to(DEV)
    a = torch.randn(1024, 1024).to(dtype).to(DEV)
    b = torch.randn(1024, 1024).to(dtype).to(DEV)
    topo = U.topo_of(s)
    # fp32: sums of 1024 products of N(0, 1) values in two orders differ by some 1e-5 whatever their own size
    tol = dict(rtol=1e-4, atol=2e-3) if dtype == torch.float32 else None
    data32, a32, b32 = U.np32(s.data), U.np32(a), U.np32(b)
    for ta, tb in _TRANSPOSE:
        lhs, lhs32 = (a.t(), a32.T) if ta else (a, a32)
        rhs, rhs32 = (b.t(), b32.T) if tb else (b, b32)
        U.assert_close_scaled(stk.ops.sdd(lhs, rhs, s).data, O.sdd(lhs32, rhs32, topo), dtype, f"sdd {ta} {tb}", tol)
        U.assert_close_scaled(stk.ops.dsd(s.t() if ta else s, rhs), O.dsd((1024, 1024), data32, topo, ta, rhs32), dtype, f"dsd {ta} {tb}", tol)
        U.assert_close_scaled(stk.ops.dds(lhs, s.t() if tb else s), O.dds(lhs32, (1024, 1024), data32, topo, tb), dtype, f"dds {ta} {tb}", tol)
    # the reference's own comparator for this configuration: to_dense + matmul, masked to the topology
    dense = stk.ops.to_dense(s).float()
    U.assert_close_scaled(stk.ops.dsd(s, b), dense @ b.float(), dtype, "dsd vs to_dense + matmul", tol)
    U.assert_close_scaled(stk.ops.dds(a, s), a.float() @ dense, dtype, "dds vs to_dense + matmul", tol)
    U.assert_close_scaled(stk.ops.sdd(a, b, s).data, O.dense_masked_sdd(a32, b32, topo), dtype, "sdd vs matmul masked to the topology", tol)


def test_products_on_a_topology_built_in_inference_mode():
    # tensors made under inference mode keep no version counter; the fusion plan must not need one
    dtype = torch.bfloat16
    _seed("inference")
    with torch.inference_mode():
        choices = torch.randint(0, 64, (4096, 1), dtype=torch.int32)
        r = stk.ops.route(choices.to(DEV), 64, 128)
        tm = stk.ops.dmoe_topology(r.padded_bins, 128, r.row_slots.numel() // 128, 4, dtype=dtype)
        assert tm.offsets.is_inference()
        rows, cols = tm.size()
        x, w1, w2 = ((torch.randn(*shape) * 0.05).to(dtype).to(DEV) for shape in ((rows, 256), (256, cols), (cols, 256)))
        h = stk.ops.sdd(x, w1, tm)
        y = stk.ops.dsd(h, w2)
        dw1 = stk.ops.dds(x.t(), h)
        s = stk.ops.to_sparse(stk.ops.to_dense(h), 128)
        assert torch.equal(s.data, h.data)
    topo = U.topo_of(tm)
    U.assert_close(h.data, O.sdd(U.np32(x), U.np32(w1), topo), dtype, "sdd in inference mode")
    U.assert_close(y, O.dsd(topo.shape, U.np32(h.data), topo, False, U.np32(w2)), dtype, "dsd in inference mode")
    U.assert_close(dw1, O.dds(U.np32(x).T, topo.shape, U.np32(h.data), topo, False), dtype, "dds in inference mode")


def test_fusion_plan_follows_replaced_column_indices():
    # one offsets tensor (a fixed number of blocks per row) used with column indices that are replaced by a new
    # tensor of the same size: the caching allocator hands the new one the old address, and a plan kept for the
    # old pattern (rows marked identical) would compute the wrong blocks
    from stk_amd.backend import hip_kernels
    dtype = torch.bfloat16
    _seed("replaced indices")
    b, rb, cb, per_row = 128, 24, 16, 4
    offsets = (torch.arange(rb + 1, dtype=torch.int32) * per_row).to(DEV)
    x = _dense(rb * b, 256, dtype, 0.05).detach()
    w = _dense(256, cb * b, dtype, 0.05).detach()
    v = _dense(cb * b, 256, dtype, 0.05).detach()
    for trial, identical_rows in enumerate((True, False, True, False)):
        if identical_rows:
            cols = np.tile(np.arange(per_row) * 3, (rb, 1))
        else:
            cols = np.stack([np.sort(np.random.choice(cb, per_row, replace=False)) for _ in range(rb)])
        ci = torch.from_numpy(cols.reshape(-1).astype(np.int16)).to(DEV)
        ri = torch.arange(rb, dtype=torch.int16).repeat_interleave(per_row).to(DEV)
        data = torch.empty(rb * per_row, b, b, dtype=dtype, device=DEV)
        m = stk.Matrix(torch.Size((rb * b, cb * b)), data, ri, ci, offsets)
        topo = U.topo_of(m)
        out = stk.ops.sdd(x, w, m)
        U.assert_close(out.data, O.sdd(U.np32(x), U.np32(w), topo), dtype, f"sdd, trial {trial}")
        U.assert_close(stk.ops.dsd(out, v), O.dsd(topo.shape, U.np32(out.data), topo, False, U.np32(v)), dtype, f"dsd, trial {trial}")
        U.assert_close(stk.ops.dds(x.t(), out), O.dds(U.np32(x).T, topo.shape, U.np32(out.data), topo, False), dtype, f"dds, trial {trial}")
        cached = offsets._stk_plan
        assert cached[0][0] is ci          # the entry holds the tensors it describes
        del m, ci, out, topo               # only the cache keeps the old column indices alive now
    assert hip_kernels.fusion_plan(offsets, cached[0][0], blocking=128) is cached[1]
