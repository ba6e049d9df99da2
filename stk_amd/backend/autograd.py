"""Autograd functions for the three products.

Forward argument order and output allocation follow stk/backend/sputnik.py
(DSD :85-127, DDS :161-200, SDD :234-270, RowIndices :304-313); the module is
also importable as `stk_amd.backend.sputnik`.

Backward restates the gradient algebra of sputnik.py:65-82 / :131-155 /
:204-228 / :274-299 as explicit formulas.  With C = A B:
    dA = dC B^T,   dB = A^T dC,
and a gradient with respect to an operand that reached the op as a .t() view
is produced in the layout of the underlying storage and returned as .t(), so
that it accumulates into the base tensor without a copy.  Sparse operands carry
a transpose flag instead of a view; the kernels then walk the CSC metadata.
"""
import torch

from stk_amd.backend import hip_kernels as backend
from stk_amd.backend.autocast import custom_bwd, custom_fwd


def _is_transposed_view(x):
    return (not x.is_contiguous()) and x.stride(0) == 1 and x.stride(1) == x.size(0)


def _plain(dy):
    """Incoming gradients may be expanded scalars or other odd views (sputnik.py:50-55)."""
    if dy.is_contiguous() or _is_transposed_view(dy):
        return dy
    return dy.contiguous()


class _Sparse:
    """The tensors of a sparse operand plus the shape of its storage."""

    def __init__(self, shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t):
        self.shape = tuple(shape)
        self.data = data
        self.meta = (offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t)

    def logical_shape(self, transposed):
        return (self.shape[1], self.shape[0]) if transposed else self.shape


def _run_dsd(sp, data, transposed, rhs):
    shape = sp.logical_shape(transposed)
    out = torch.empty((shape[0], rhs.size(1)), dtype=rhs.dtype, device=rhs.device)
    backend.dsd(shape, data, *sp.meta, transposed, rhs, out)
    return out


def _run_dds(lhs, sp, data, transposed):
    shape = sp.logical_shape(transposed)
    out = torch.empty((lhs.size(0), shape[1]), dtype=lhs.dtype, device=lhs.device)
    backend.dds(lhs, shape, data, *sp.meta, transposed, out)
    return out


def _run_sdd(lhs, rhs, sp):
    out = torch.empty(sp.data.shape, dtype=lhs.dtype, device=lhs.device)
    offsets, row_indices, column_indices, _, _, block_offsets_t = sp.meta
    # visiting blocks column by column keeps the rhs panel of a block column in cache
    backend.sdd(lhs, rhs, sp.shape, out, offsets, row_indices, column_indices, block_order=block_offsets_t)
    return out


# The two gradients of a product are independent launches that read the same incoming gradient.  With this
# switch on, the second one runs on a side stream (default priority) next to the first: the workgroups of one
# fill the compute units that the other leaves idle in its last round.
OVERLAP_GRADIENTS = True
_side_streams = {}
# Both gradients of sdd (stk_dsd_dds, stk_dsd_dsd) in one launch where the operands' layouts allow it, instead of two
# launches side by side; the same results.
JOINT_GRADIENTS = True
# The same for both gradients of dsd (stk_sdd_dsd).  What a joint launch gains is its tail: the short tiles of the second
# product fill the compute units that the last round of the first leaves idle.  An sdd that runs as one workgroup per
# compute unit walking its tile list has no such round left, and the two launches are then the shorter way (benchmark
# topology, sdd(dy, W2^T) + dsd(h^T, dy) back to back: 462 us as two launches, 473 us as one).
JOINT_DSD_GRADIENTS = False


def _side_stream(device):
    stream = _side_streams.get(device.index)
    if stream is None:
        stream = _side_streams[device.index] = torch.cuda.Stream(device=device)
        backend.CONCURRENT_STREAMS.add(stream.cuda_stream)   # its dsd launches get a workspace of their own
    return stream


def _both(first, second, device):
    """first() and second() -> their results (None for a callable that is None), launched side by side when
    both are wanted.  Each callable launches one product and returns its freshly allocated output."""
    if first is None or second is None or not OVERLAP_GRADIENTS or device.type != "cuda":
        return (first() if first is not None else None), (second() if second is not None else None)
    main = torch.cuda.current_stream(device)
    side = _side_stream(device)
    side.wait_stream(main)          # the operands are ready on the main stream
    with torch.cuda.stream(side):
        b = second()
    a = first()
    main.wait_stream(side)          # whatever follows on the main stream sees both results
    b.record_stream(main)           # allocated under the side stream, used and freed under the main one
    return a, b


class DSD(torch.autograd.Function):

    @staticmethod
    @custom_fwd
    def forward(ctx, shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t,
                block_offsets_t, transpose_a, rhs):
        ctx.save_for_backward(data, offsets, row_indices, column_indices, offsets_t, column_indices_t,
                              block_offsets_t, rhs)
        ctx.storage_shape = (shape[1], shape[0]) if transpose_a else tuple(shape)
        ctx.transpose_a = transpose_a
        out = torch.empty((shape[0], rhs.size(1)), dtype=rhs.dtype, device=rhs.device)
        backend.dsd(shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t,
                    block_offsets_t, transpose_a, rhs, out)
        return out

    @staticmethod
    @custom_bwd
    def backward(ctx, dy):
        data, *meta, rhs = ctx.saved_tensors
        sp = _Sparse(ctx.storage_shape, data, *meta)
        ta = ctx.transpose_a
        dy = _plain(dy)
        want_data = want_rhs = None
        rhs_is_view = _is_transposed_view(rhs)
        if JOINT_DSD_GRADIENTS and dy.is_cuda and ctx.needs_input_grad[1] and ctx.needs_input_grad[9] and not rhs_is_view:
            # dy rhs^T on the pattern and op(S)^T dy read the same dy: one call (sputnik.py:131-155 makes two)
            ddata = torch.empty_like(data)
            drhs = torch.empty_like(rhs, memory_format=torch.contiguous_format)
            backend.prepare_plan(data, meta[0], meta[2], meta[3], meta[4])
            if ta:
                backend.sdd_dsd(sp.shape, rhs, dy.t(), ddata, data, *meta, False, dy, drhs)
            else:
                backend.sdd_dsd(sp.shape, dy, rhs.t(), ddata, data, *meta, True, dy, drhs)
            return None, ddata, None, None, None, None, None, None, None, drhs
        if ctx.needs_input_grad[1]:
            # d op(S) = dy rhs^T on the pattern; for a transposed S the stored blocks hold (rhs dy^T)
            want_data = (lambda: _run_sdd(rhs, dy.t(), sp)) if ta else (lambda: _run_sdd(dy, rhs.t(), sp))
        if ctx.needs_input_grad[9]:
            if rhs_is_view:
                want_rhs = lambda: _run_dds(dy.t(), sp, data, ta)       # dy^T op(S), returned transposed
            else:
                want_rhs = lambda: _run_dsd(sp, data, not ta, dy)       # op(S)^T dy
        ddata, drhs = _both(want_data, want_rhs, dy.device)
        if drhs is not None and rhs_is_view:
            drhs = drhs.t()
        return None, ddata, None, None, None, None, None, None, None, drhs


class DDS(torch.autograd.Function):

    @staticmethod
    @custom_fwd
    def forward(ctx, lhs, shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t,
                block_offsets_t, transpose_b):
        ctx.save_for_backward(lhs, data, offsets, row_indices, column_indices, offsets_t, column_indices_t,
                              block_offsets_t)
        ctx.storage_shape = (shape[1], shape[0]) if transpose_b else tuple(shape)
        ctx.transpose_b = transpose_b
        out = torch.empty((lhs.size(0), shape[1]), dtype=lhs.dtype, device=lhs.device)
        backend.dds(lhs, shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t,
                    block_offsets_t, transpose_b, out)
        return out

    @staticmethod
    @custom_bwd
    def backward(ctx, dy):
        lhs, data, *meta = ctx.saved_tensors
        sp = _Sparse(ctx.storage_shape, data, *meta)
        tb = ctx.transpose_b
        dy = _plain(dy)
        want_lhs = want_data = None
        lhs_is_view = _is_transposed_view(lhs)
        if ctx.needs_input_grad[0]:
            if lhs_is_view:
                want_lhs = lambda: _run_dsd(sp, data, tb, dy.t())       # op(S) dy^T, returned transposed
            else:
                want_lhs = lambda: _run_dds(dy, sp, data, not tb)       # dy op(S)^T
        if ctx.needs_input_grad[2]:
            # d op(S) = lhs^T dy on the pattern; for a transposed S the stored blocks hold (dy^T lhs)
            want_data = (lambda: _run_sdd(dy.t(), lhs, sp)) if tb else (lambda: _run_sdd(lhs.t(), dy, sp))
        dlhs, ddata = _both(want_lhs, want_data, dy.device)
        if dlhs is not None and lhs_is_view:
            dlhs = dlhs.t()
        return dlhs, None, ddata, None, None, None, None, None, None, None


def _sdd_operand_gradients(ctx, lhs, rhs, sp, ds):
    """Gradients of S = lhs rhs (on the pattern) with respect to lhs and rhs, given dS as the values `ds`."""
    want_lhs = want_rhs = None
    lhs_is_view, rhs_is_view = _is_transposed_view(lhs), _is_transposed_view(rhs)
    if JOINT_GRADIENTS and ds.is_cuda and ctx.needs_input_grad[0] and ctx.needs_input_grad[1] and not lhs_is_view and not rhs_is_view:
        # dS rhs^T and lhs^T dS read the same dS: one call (sputnik.py:274-299 makes two)
        dlhs = torch.empty((sp.shape[0], rhs.size(0)), dtype=lhs.dtype, device=lhs.device)
        drhs = torch.empty((lhs.size(1), sp.shape[1]), dtype=rhs.dtype, device=rhs.device)
        backend.dsd_dds(sp.shape, ds, *sp.meta, rhs.t(), dlhs, lhs.t(), drhs)
        return dlhs, drhs
    if JOINT_GRADIENTS and ds.is_cuda and ctx.needs_input_grad[0] and ctx.needs_input_grad[1] and not lhs_is_view and rhs_is_view:
        # rhs is a .t() view of a row-major tensor, whose gradient is dS^T lhs: two dsd on the same dS, one call
        base = rhs.t()
        dlhs = torch.empty((sp.shape[0], rhs.size(0)), dtype=lhs.dtype, device=lhs.device)
        dbase = torch.empty((sp.shape[1], lhs.size(1)), dtype=rhs.dtype, device=rhs.device)
        backend.dsd_dsd(sp.shape, ds, *sp.meta, base, dlhs, lhs, dbase)
        return dlhs, dbase.t()
    if ctx.needs_input_grad[0]:
        if lhs_is_view:
            want_lhs = lambda: _run_dds(rhs, sp, ds, True)              # rhs dS^T, returned transposed
        else:
            want_lhs = lambda: _run_dsd(sp, ds, False, rhs.t())         # dS rhs^T
    if ctx.needs_input_grad[1]:
        if rhs_is_view:
            want_rhs = lambda: _run_dsd(sp, ds, True, lhs)              # dS^T lhs, returned transposed
        else:
            want_rhs = lambda: _run_dds(lhs.t(), sp, ds, False)         # lhs^T dS
    dlhs, drhs = _both(want_lhs, want_rhs, ds.device)
    if dlhs is not None and lhs_is_view:
        dlhs = dlhs.t()
    if drhs is not None and rhs_is_view:
        drhs = drhs.t()
    return dlhs, drhs


class SDD(torch.autograd.Function):

    @staticmethod
    @custom_fwd
    def forward(ctx, lhs, rhs, shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t,
                block_offsets_t):
        ctx.save_for_backward(lhs, rhs, offsets, row_indices, column_indices, offsets_t, column_indices_t,
                              block_offsets_t)
        ctx.shape = tuple(shape)
        out = torch.empty(data.shape, dtype=lhs.dtype, device=lhs.device)
        backend.prepare_plan(data, offsets, column_indices, offsets_t, column_indices_t)
        backend.sdd(lhs, rhs, shape, out, offsets, row_indices, column_indices, block_order=block_offsets_t)
        return out

    @staticmethod
    @custom_bwd
    def backward(ctx, dy):
        lhs, rhs, *meta = ctx.saved_tensors
        if not dy.is_contiguous():
            dy = dy.contiguous()
        dlhs, drhs = _sdd_operand_gradients(ctx, lhs, rhs, _Sparse(ctx.shape, dy, *meta), dy)
        return dlhs, drhs, None, None, None, None, None, None, None, None


_FUSED_ACTIVATIONS = (None, "none", "relu", "silu", "gelu", "gelu_tanh")   # (their derivatives are the backward pass's business)


class SDDFused(torch.autograd.Function):
    """activation(sdd(lhs, rhs)) * multiplier in one pass (no counterpart in the reference, whose callers run
    the activation and stk.ops.mul, stk/ops/eltwise_ops.py:3-28, as passes of their own).  Without save_sums only the
    result is stored; backward recomputes the sums in an sdd whose store applies the activation's derivative and
    multiplies by the incoming gradient.  With save_sums the forward product also stores the rounded sums (what the
    reference's callers keep: the result of sdd() in front of their activation), and backward gets the same gradient
    from one element-wise pass over them - less time, one more array of values.  Either way it then follows
    SDD.backward."""

    @staticmethod
    @custom_fwd
    def forward(ctx, lhs, rhs, shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t,
                block_offsets_t, activation, multiplier, save_sums=False):
        if activation not in _FUSED_ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}")
        out = torch.empty(data.shape, dtype=lhs.dtype, device=lhs.device)
        values = None if multiplier is None else multiplier.detach().contiguous()
        keep = bool(save_sums) and activation not in (None, "none") and lhs.is_cuda and any(ctx.needs_input_grad)
        sums = torch.empty_like(out) if keep else None
        backend.prepare_plan(data, offsets, column_indices, offsets_t, column_indices_t)
        backend.sdd_fused(lhs, rhs, shape, out, offsets, row_indices, column_indices, activation, values,
                          block_order=block_offsets_t, sums=sums)
        ctx.save_for_backward(lhs, rhs, offsets, row_indices, column_indices, offsets_t, column_indices_t,
                              block_offsets_t, *(() if values is None else (values,)), *(() if sums is None else (sums,)))
        ctx.shape = tuple(shape)
        ctx.activation = activation
        ctx.has_multiplier = values is not None
        ctx.has_sums = sums is not None
        return out

    @staticmethod
    @custom_bwd
    def backward(ctx, dy):
        lhs, rhs, *meta = ctx.saved_tensors
        sums = meta.pop() if ctx.has_sums else None
        values = meta.pop() if ctx.has_multiplier else None
        offsets, row_indices, column_indices, _, _, block_offsets_t = meta
        plain = ctx.activation in (None, "none")
        if not dy.is_contiguous():
            dy = dy.contiguous()

        def recompute(activation, multiplier):
            if sums is not None:
                return backend.activation_product(sums, multiplier, activation)
            out = torch.empty(dy.shape, dtype=lhs.dtype, device=lhs.device)
            backend.sdd_fused(lhs, rhs, ctx.shape, out, offsets, row_indices, column_indices, activation, multiplier,
                              block_order=block_offsets_t)
            return out

        # out = round(round(act(s)) * m): the gradient that reaches the sums is act'(s) * (dy * m), the one that reaches
        # the multiplier dy * round(act(s)).  Both come out of sdd launches that compute the sums again and apply the
        # derivative (or the activation) while they store - no element-wise passes over fp32 copies of the values.
        dmul = None
        if values is not None and ctx.needs_input_grad[11]:
            dmul = dy * recompute(ctx.activation, None)
        g = dy if values is None else dy * values
        dsums = g if plain else recompute(ctx.activation + "_grad", g)
        dlhs, drhs = _sdd_operand_gradients(ctx, lhs, rhs, _Sparse(ctx.shape, dsums, *meta), dsums)
        return dlhs, drhs, None, None, None, None, None, None, None, None, None, dmul, None


class RowIndices(torch.autograd.Function):

    @staticmethod
    def forward(ctx, shape, data, offsets, column_indices):
        out = torch.empty(column_indices.shape, dtype=column_indices.dtype, device=column_indices.device)
        backend.row_indices(shape, data, offsets, column_indices, out)
        return out


dsd = DSD.apply
dds = DDS.apply
sdd = SDD.apply
sdd_fused = SDDFused.apply
row_indices = RowIndices.apply
