"""stk.ops.dsd / dds / sdd (stk/ops/linear_ops.py:7-59): unpack a Matrix into
the positional arguments of the autograd functions; a transposed Matrix
becomes the transpose flag; sdd's result shares the topology's metadata."""
import torch

from stk_amd.backend import autograd as sputnik
from stk_amd.matrix import Matrix


def _unpack(m):
    return (m.size(), m.data, m.offsets, m.row_indices, m.column_indices,
            m.offsets_t, m.column_indices_t, m.block_offsets_t)


def dsd(a, b):
    assert isinstance(a, Matrix)
    assert isinstance(b, torch.Tensor)
    return sputnik.dsd(*_unpack(a), not a.is_contiguous(), b)


def dds(a, b):
    assert isinstance(a, torch.Tensor)
    assert isinstance(b, Matrix)
    return sputnik.dds(a, *_unpack(b), not b.is_contiguous())


def sdd(a, b, topo):
    assert isinstance(a, torch.Tensor)
    assert isinstance(b, torch.Tensor)
    assert isinstance(topo, Matrix)
    assert topo.is_contiguous()
    out = sputnik.sdd(a, b, *_unpack(topo))
    return Matrix(topo.size(), out, topo.row_indices, topo.column_indices, topo.offsets,
                  topo.column_indices_t, topo.offsets_t, topo.block_offsets_t)


def sdd_fused(a, b, topo, activation=None, multiplier=None, save_sums=False):
    """activation(sdd(a, b, topo)) * multiplier in one pass: the activation ("relu", "gelu_tanh",
    "gelu", "silu" or None) is applied to the fp32 sums before they are rounded, and the rounded
    values are multiplied by those of `multiplier` (a Matrix with topo's topology, or None) as
    stk.ops.mul would (stk/ops/eltwise_ops.py:3-28).  By default only the result is stored and the
    backward pass computes the sums again (one more sdd); with save_sums the product also stores the
    rounded sums (one more array of values, what a caller of the reference keeps anyway) and the
    backward pass is an element-wise pass over them."""
    assert isinstance(a, torch.Tensor)
    assert isinstance(b, torch.Tensor)
    assert isinstance(topo, Matrix)
    assert topo.is_contiguous()
    if multiplier is not None:
        assert isinstance(multiplier, Matrix)
        assert multiplier.size() == topo.size()
    out = sputnik.sdd_fused(a, b, *_unpack(topo), activation, None if multiplier is None else multiplier.data, save_sums)
    return Matrix(topo.size(), out, topo.row_indices, topo.column_indices, topo.offsets,
                  topo.column_indices_t, topo.offsets_t, topo.block_offsets_t)
