"""Token routing around the block-sparse products of a dropless mixture-of-experts layer.

The reference has no code for this step: its callers sort the expert choices, pad every
expert's rows to the block size and copy the token rows into that layout before they build
stk.Matrix (stk/matrix.py:134-157), and copy the results back afterwards.  Here the sort
and the two copies are HIP kernels; `Route.padded_bins` feeds stk.ops.dmoe_topology."""
from collections import namedtuple

import torch

from stk_amd.backend import hip_kernels
from stk_amd.matrix import Matrix

Route = namedtuple("Route", "indices bin_ids bins padded_bins slot_rows row_slots top_k blocking")


@torch.no_grad()
def route(top_experts, num_experts, blocking, padded_rows=None):
    """Routing of the (token, choice) slots given top_experts [tokens, top_k] (or [tokens]) on the GPU.

    indices / bin_ids    slot numbers in a stable sort by expert, and their experts
    bins / padded_bins   inclusive prefix sums of the slots per expert, plain and with every
                         expert rounded up to a multiple of `blocking`
    slot_rows            row of slot token * top_k + choice in the padded layout
    row_slots            slot held by each row of the padded layout, -1 for padding

    padded_rows: rows of the padded layout.  None reads padded_bins[-1] back (one device
    synchronisation, exact size); an int that is at least padded_bins[-1] avoids that -
    `route_capacity` gives one that is always enough."""
    top_k = top_experts.size(1) if top_experts.dim() == 2 else 1
    slots = top_experts.numel()
    exact = padded_rows is None
    capacity = route_capacity(slots, num_experts, blocking) if exact else padded_rows
    r = hip_kernels.route(top_experts, num_experts, blocking, capacity)
    indices, bin_ids, bins, padded_bins, slot_rows, row_slots = r
    if exact:
        row_slots = row_slots[:int(padded_bins[-1].item())]
    return Route(indices, bin_ids, bins, padded_bins, slot_rows, row_slots, top_k, blocking)


def route_capacity(slots, num_experts, blocking):
    """Largest padded layout `slots` slots over `num_experts` experts can need (a multiple of blocking)."""
    return (slots + num_experts * (blocking - 1)) // blocking * blocking


class _PaddedGather(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, route):
        ctx.route = route
        return hip_kernels.padded_gather(x, route.row_slots, route.top_k)

    @staticmethod
    def backward(ctx, grad):
        r = ctx.route
        return hip_kernels.padded_scatter(grad, r.slot_rows, r.top_k), None


class _PaddedScatter(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, route, weights):
        ctx.route = route
        ctx.save_for_backward(x if weights is not None and weights.requires_grad else None, weights)
        return hip_kernels.padded_scatter(x, route.slot_rows, route.top_k, weights)

    @staticmethod
    def backward(ctx, grad):
        r = ctx.route
        x, weights = ctx.saved_tensors
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = hip_kernels.padded_gather(grad, r.row_slots, r.top_k, weights)
        if weights is not None and ctx.needs_input_grad[2]:
            dw = hip_kernels.padded_scatter_weight_gradient(x, grad, r.slot_rows, r.top_k).to(weights.dtype).view_as(weights)
        return dx, None, dw


def padded_gather(x, route):
    """x [tokens, hidden] -> [padded_rows, hidden]: every slot's token row at its place in the padded
    layout, zeros in the padding rows."""
    return _PaddedGather.apply(x, route)


def padded_scatter(x, route, weights=None):
    """x [padded_rows, hidden] -> [tokens, hidden]: each token's top_k rows, multiplied by
    weights [tokens, top_k] (or [tokens * top_k]) when given, added up in fp32 in the order of the choices."""
    return _PaddedScatter.apply(x, route, weights)


def _wants_grad(*tensors):
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def gather_sdd(x, route, rhs, topo, activation=None):
    """stk.ops.sdd_fused(padded_gather(x, route), rhs, topo, activation) in one launch: the sampled product reads the
    token rows where they lie, and the padded copy of x is never made.  The result is bit-identical to the two steps.
    Used when nothing needs a gradient (the backward pass of the product needs the padded copy anyway) and the library
    has the kernel (128-blocks); otherwise the two steps run."""
    from stk_amd.ops import linear_ops
    assert isinstance(topo, Matrix) and topo.is_contiguous()
    if x.is_cuda and not _wants_grad(x, rhs):
        out = torch.empty_like(topo.data)
        if hip_kernels.sdd_gather(x, route.row_slots, route.top_k, rhs, topo.size(), out, topo.offsets, topo.row_indices, topo.column_indices,
                                  activation):
            return Matrix(topo.size(), out, topo.row_indices, topo.column_indices, topo.offsets,
                          topo.column_indices_t, topo.offsets_t, topo.block_offsets_t)
    return linear_ops.sdd_fused(padded_gather(x, route), rhs, topo, activation)


def dsd_scatter(a, rhs, route, weights=None):
    """padded_scatter(stk.ops.dsd(a, rhs), route, weights) in one launch for top_k = 1: the product's store writes
    every row to its token's place (times its weight), and the padded result is never made.  The result is
    bit-identical to the two steps.  Used when nothing needs a gradient, the routing is top-1 and the library has the
    kernel (128-blocks, a multiple of 256 columns, enough work for the eight-wavefront tiles); otherwise the two steps
    run."""
    from stk_amd.ops import linear_ops
    assert isinstance(a, Matrix)
    if route.top_k == 1 and a.is_contiguous() and a.data.is_cuda and not _wants_grad(a.data, rhs, weights):
        tokens = route.slot_rows.numel()
        out = torch.empty((tokens, rhs.shape[1]), dtype=a.dtype, device=a.data.device)
        if hip_kernels.dsd_scatter(a.size(), a.data, a.offsets, a.column_indices, a.offsets_t, a.column_indices_t, rhs,
                                   route.row_slots, weights, out):
            return out
    return padded_scatter(linear_ops.dsd(a, rhs), route, weights)
