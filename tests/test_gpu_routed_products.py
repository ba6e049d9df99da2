"""GPU parity of the products that read and write the token rows in place: stk_sdd_gather (padded_gather + sdd_fused
in one launch) and stk_dsd_scatter (dsd + padded_scatter for top-1 in one launch), through the C ABI.

Both are defined as "what the two launches give", and the two launches are pinned elsewhere (the products against
the oracle, the copies bit for bit), so the comparison here is bit for bit against them, on the sizes that reach
each kernel (one block per workgroup, the fused tiles with a plan, the sliced last round with its workspace and the
plain grid without), plus one comparison of the whole routed layer against fp32 torch.
"""
import pytest
import torch

import stk_amd as stk
from stk_amd.backend import hip_kernels
from tests import _util as U

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = (torch.bfloat16, torch.float16)


def _choices(tokens, experts, top_k, seed, skew=False, empty=()):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(tokens, experts, generator=g)
    if skew:
        logits[:, 0] += 2.0          # about half of the tokens choose expert 0
    for e in empty:
        logits[:, e] = -1e9          # experts without a token
    return logits.topk(top_k, dim=1).indices.to(torch.int32)


def _layer(tokens, hidden, experts, ffn, top_k, dtype, seed, skew=False, empty=(), capacity=False):
    """Tokens, routing, topology and both weight matrices of a dropless mixture-of-experts layer on the GPU."""
    torch.manual_seed(seed)
    x = torch.randn(tokens, hidden).to(dtype).to(DEV)
    top = _choices(tokens, experts, top_k, seed, skew, empty).to(DEV)
    rows = stk.ops.route_capacity(tokens * top_k, experts, 128) if capacity else None
    r = stk.ops.route(top, experts, 128, padded_rows=rows)
    padded = r.row_slots.numel()
    topo = stk.ops.dmoe_topology(r.padded_bins, 128, padded // 128, ffn // 128, dtype=dtype)
    w1 = (torch.randn(hidden, experts * ffn) * 0.05).to(dtype).to(DEV)
    w2 = (torch.randn(experts * ffn, hidden) * 0.05).to(dtype).to(DEV)
    return x, r, topo, w1, w2


def _same_bits(a, b):
    return torch.equal(a.view(torch.int16), b.view(torch.int16))


# (tokens, hidden, experts, ffn per expert, top_k): the first reaches the kernel with one block per workgroup (few
# blocks), the others the fused tiles of a plan (pairs, threes and lone rows among the experts' rows)
GATHER_SIZES = (
    (700, 256, 4, 256, 1),
    (700, 96, 4, 256, 2),
    (4096, 512, 8, 1024, 1),
    (3000, 320, 8, 768, 2),
)


@pytest.mark.parametrize("dtype", DTYPES, ids=("bf16", "f16"))
@pytest.mark.parametrize("tokens,hidden,experts,ffn,top_k", GATHER_SIZES)
@pytest.mark.parametrize("transposed_weight", (False, True))
def test_sdd_gather_is_gather_then_sdd(tokens, hidden, experts, ffn, top_k, dtype, transposed_weight):
    seed = U.stable_seed("sdd_gather", tokens, hidden, experts, ffn, top_k, dtype, transposed_weight)
    x, r, topo, w1, _ = _layer(tokens, hidden, experts, ffn, top_k, dtype, seed, skew=top_k == 1, empty=(1,))
    if transposed_weight:
        w1 = w1.t().contiguous().t()     # the .t() view of a row-major [n, k]
    padded = stk.ops.padded_gather(x, r)
    for activation in (None, "gelu_tanh"):
        want = stk.ops.sdd_fused(padded, w1, topo, activation)
        out = torch.full_like(topo.data, float("nan"))
        assert hip_kernels.sdd_gather(x, r.row_slots, r.top_k, w1, topo.size(), out, topo.offsets, topo.row_indices, topo.column_indices,
                                      activation), "the library has this kernel"
        assert _same_bits(out, want.data), activation
        got = stk.ops.gather_sdd(x, r, w1, topo, activation)
        assert isinstance(got, stk.Matrix) and _same_bits(got.data, want.data)


def test_sdd_gather_rows_beyond_the_last_expert_and_strided_tokens():
    # a padded layout sized by its upper bound: the rows behind the last expert's are padding too; the token rows
    # are a slice of a wider array
    tokens, hidden, experts, ffn = 2000, 256, 8, 512
    x, r, topo, w1, _ = _layer(tokens, hidden, experts, ffn, 1, torch.bfloat16, 5, capacity=True)
    wide = torch.randn(tokens, hidden + 64, device=DEV).to(torch.bfloat16)
    xs = wide[:, 64:]
    want = stk.ops.sdd(stk.ops.padded_gather(xs, r), w1, topo)
    got = stk.ops.gather_sdd(xs, r, w1, topo)
    assert _same_bits(got.data, want.data)
    assert int((r.row_slots < 0).sum()) >= 128


def test_sdd_gather_refuses_what_it_has_no_kernel_for():
    x, r, topo, w1, _ = _layer(700, 256, 4, 256, 1, torch.bfloat16, 1)
    out = torch.empty_like(topo.data)
    lib = hip_kernels._lib.load()
    args = lambda blocking, activation: (
        x.data_ptr(), 700, 256, r.row_slots.data_ptr(), 1, w1.data_ptr(), w1.stride(0), w1.stride(1), topo.size()[0], 256, topo.size()[1],
        out.data_ptr(), None, topo.row_indices.data_ptr(), topo.column_indices.data_ptr(), topo.row_indices.numel(), blocking, hip_kernels._lib.STK_BF16,
        hip_kernels._lib.STK_I16, None, activation, None)
    assert lib.stk_sdd_gather(*args(64, 0)) == hip_kernels._lib.STK_ERR_UNSUPPORTED
    assert lib.stk_sdd_gather(*args(128, hip_kernels.ACTIVATIONS["gelu_grad"])) == hip_kernels._lib.STK_ERR_UNSUPPORTED
    assert b"derivative" in lib.stk_last_error()
    # with gradients wanted the two steps run, and the gradients are theirs
    x.requires_grad_(True)
    w1.requires_grad_(True)
    got = stk.ops.gather_sdd(x, r, w1, topo)
    got.data.float().square().sum().backward()
    gx, gw = x.grad.clone(), w1.grad.clone()
    x.grad = w1.grad = None
    stk.ops.sdd(stk.ops.padded_gather(x, r), w1, topo).data.float().square().sum().backward()
    assert _same_bits(gx, x.grad) and _same_bits(gw, w1.grad)


# (tokens, hidden, experts, ffn per expert): enough blocks x columns for the eight-wavefront tiles
SCATTER_SIZES = (
    (8192, 1024, 8, 2560),
    (6000, 768, 16, 5120),
)


@pytest.mark.parametrize("dtype", DTYPES, ids=("bf16", "f16"))
@pytest.mark.parametrize("tokens,hidden,experts,ffn", SCATTER_SIZES)
@pytest.mark.parametrize("weighted", (False, True))
@pytest.mark.parametrize("sliced", (True, False))
def test_dsd_scatter_is_dsd_then_scatter(tokens, hidden, experts, ffn, dtype, weighted, sliced, monkeypatch):
    seed = U.stable_seed("dsd_scatter", tokens, hidden, experts, ffn, dtype, weighted)
    x, r, topo, w1, w2 = _layer(tokens, hidden, experts, ffn, 1, dtype, seed, skew=True, empty=(2,))
    monkeypatch.setattr(hip_kernels, "SLICE_LAST_ROUND", sliced)
    hip_kernels.release_workspaces()
    h = stk.ops.sdd_fused(stk.ops.padded_gather(x, r), w1, topo, "gelu_tanh")
    weights = torch.rand(tokens, 1, device=DEV) + 0.5 if weighted else None
    for rhs in (w2, w2.t().contiguous().t()):
        want = stk.ops.padded_scatter(stk.ops.dsd(h, rhs), r, weights)
        out = torch.full((tokens, hidden), float("nan"), dtype=dtype, device=DEV)
        assert hip_kernels.dsd_scatter(h.size(), h.data, h.offsets, h.column_indices, h.offsets_t, h.column_indices_t, rhs, r.row_slots,
                                       weights, out), "the library has this kernel"
        assert _same_bits(out, want)
        assert _same_bits(stk.ops.dsd_scatter(h, rhs, r, weights), want)
        # once more: the workspace's counters are back at zero
        out.fill_(float("nan"))
        assert hip_kernels.dsd_scatter(h.size(), h.data, h.offsets, h.column_indices, h.offsets_t, h.column_indices_t, rhs, r.row_slots,
                                       weights, out)
        assert _same_bits(out, want)
    hip_kernels.release_workspaces()


def test_dsd_scatter_falls_back_where_it_has_no_kernel():
    # little work (four-wavefront tiles in stk_dsd), top-2, a transposed operand, gradients: the two steps run
    x, r, topo, w1, w2 = _layer(700, 256, 4, 256, 1, torch.bfloat16, 2)
    h = stk.ops.sdd(stk.ops.padded_gather(x, r), w1, topo)
    out = torch.empty(700, 256, dtype=torch.bfloat16, device=DEV)
    assert not hip_kernels.dsd_scatter(h.size(), h.data, h.offsets, h.column_indices, h.offsets_t, h.column_indices_t, w2, r.row_slots, None, out)
    assert _same_bits(stk.ops.dsd_scatter(h, w2, r), stk.ops.padded_scatter(stk.ops.dsd(h, w2), r))
    x2, r2, topo2, w12, w22 = _layer(700, 256, 4, 256, 2, torch.bfloat16, 3)
    h2 = stk.ops.sdd(stk.ops.padded_gather(x2, r2), w12, topo2)
    weights = torch.rand(700, 2, device=DEV)
    assert _same_bits(stk.ops.dsd_scatter(h2, w22, r2, weights), stk.ops.padded_scatter(stk.ops.dsd(h2, w22), r2, weights))
    w2.requires_grad_(True)
    y = stk.ops.dsd_scatter(h, w2, r)
    y.float().sum().backward()
    assert w2.grad is not None and w2.grad.shape == w2.shape


@pytest.mark.parametrize("dtype", DTYPES, ids=("bf16", "f16"))
def test_routed_layer_with_both_against_fp32(dtype):
    """The whole forward pass of a top-1 layer, x -> gather_sdd(gelu) -> dsd_scatter(weights), against the same
    arithmetic in fp32 torch on every token's own expert (16-bit hidden activations, as the kernels round them)."""
    tokens, hidden, experts, ffn = 8192, 1024, 8, 2560
    x, r, topo, w1, w2 = _layer(tokens, hidden, experts, ffn, 1, dtype, 11)
    weights = torch.rand(tokens, 1, device=DEV) + 0.5
    h = stk.ops.gather_sdd(x, r, w1, topo, "gelu_tanh")
    y = stk.ops.dsd_scatter(h, w2, r, weights)
    expert = torch.bucketize(r.slot_rows.long(), r.padded_bins.long(), right=True)   # the expert that owns each token's row
    want = torch.empty(tokens, hidden, device=DEV)
    for e in range(experts):
        mine = (expert == e).nonzero().flatten()
        he = torch.nn.functional.gelu(x[mine].float() @ w1[:, e * ffn:(e + 1) * ffn].float(), approximate="tanh").to(dtype).float()
        want[mine] = ((he @ w2[e * ffn:(e + 1) * ffn].float()).to(dtype).float() * weights[mine]).to(dtype).float()
    # the result is rounded twice (the product, then the weighted row), and both sides' first roundings may fall on
    # different sides of a tie for sums that differ in the last fp32 bits: two units of the 16-bit format
    U.assert_close_scaled(y.float(), want, dtype, tol=dict(rtol=2.0 ** -6 if dtype == torch.bfloat16 else 1e-2, atol=1e-2))
