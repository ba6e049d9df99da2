"""Format helpers for host (CPU) tensors.

The reference builds its matrices on the host and moves them to the device
afterwards (stk/ops/linear_ops_test.py:57-63, stk/random/random_ops.py:26-28),
so `to_sparse`, `to_dense` and the transpose metadata must accept CPU tensors.
Values of 2 or 4 bytes with 16- or 32-bit indices - everything the reference's
tests and the products use - go to the host library (host_kernels); what is left
(other element widths, 64-bit indices) is handled by the torch statements below.
Device tensors never come here: they go to the HIP kernels
(stk_amd/backend/hip_kernels.py).
"""
import torch

from stk_amd.backend import host_kernels

_NARROW = (torch.int16, torch.int32)


def transpose_meta(size, data, row_indices, column_indices, offsets):
    """stk/matrix.py:105-123 with a stable sort (ascending block id inside a column)."""
    if row_indices.dtype in _NARROW and row_indices.dtype == column_indices.dtype:
        return host_kernels.transpose_meta(size, data, row_indices, column_indices, offsets)
    block_cols = size[1] // data.shape[1]
    order = torch.argsort(column_indices.to(torch.int64), stable=True)
    column_indices_t = row_indices[order]
    block_offsets_t = order.to(torch.int32)
    per_column = torch.bincount(column_indices.to(torch.int64), minlength=block_cols)
    offsets_t = torch.zeros(block_cols + 1, dtype=torch.int32)
    offsets_t[1:] = torch.cumsum(per_column, 0)
    return column_indices_t, offsets_t, block_offsets_t


def _blocked_view(x, blocking):
    rows, cols = x.shape
    return x.reshape(rows // blocking, blocking, cols // blocking, blocking).permute(0, 2, 1, 3)


def to_sparse(x, blocking, index_dtype=torch.int16):
    """stk/ops/matrix_ops.py:64-85: nonzero blocks in row-major order."""
    if host_kernels.handles(x) and index_dtype in _NARROW:
        return host_kernels.to_sparse(x, blocking, index_dtype)
    blocks = _blocked_view(x, blocking)
    nonzero = (blocks != 0).flatten(2).any(dim=2)
    nonzero |= torch.isnan(blocks).flatten(2).any(dim=2) if x.is_floating_point() else False
    offsets = torch.zeros(nonzero.shape[0] + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(nonzero.sum(dim=1), 0)
    coords = torch.nonzero(nonzero)
    data = blocks[coords[:, 0], coords[:, 1]].contiguous().reshape(-1, blocking, blocking)
    return data, coords[:, 0].to(index_dtype), coords[:, 1].to(index_dtype), offsets


def to_dense(data, row_indices, column_indices, rows, cols):
    """stk/ops/matrix_ops.py:36-47: zeros, then every block copied to its place."""
    if host_kernels.handles(data) and row_indices.dtype in _NARROW and row_indices.dtype == column_indices.dtype:
        return host_kernels.to_dense(data, row_indices, column_indices, rows, cols)
    b = data.shape[-1]
    out = torch.zeros((rows, cols), dtype=data.dtype)
    _blocked_view(out, b)[row_indices.long(), column_indices.long()] = data
    return out
