"""stk.Matrix: a block-sparse matrix in the hybrid blocked-CSR-COO layout.

Public surface and semantics follow stk/matrix.py:126-329.  The matrix owns
  data [nnz, b, b], row_indices / column_indices [nnz] (int16), offsets [Rb+1]
  (int32) and the transpose metadata column_indices_t, offsets_t,
  block_offsets_t (stk/matrix.py:150-157),
all plain attributes of an nn.Module.  t() flips a flag and swaps the logical
size without touching storage (:205-220).

When the transpose metadata is not supplied it is built on the device that
holds the indices: by the HIP stable sort for GPU tensors, by torch for host
tensors.  Ties inside a block column keep ascending block id (the reference's
argsort, stk/matrix.py:110, leaves that order unspecified).
"""
import numpy as np
import torch

_INT16_MAX = int(np.iinfo(np.int16).max)


def _build_transpose_meta(size, data, row_indices, column_indices, offsets):
    if column_indices.is_cuda:
        from stk_amd.backend import hip_kernels
        return hip_kernels.transpose_meta(size, data, row_indices, column_indices, offsets)
    from stk_amd.backend import host_format
    return host_format.transpose_meta(size, data, row_indices, column_indices, offsets)


_transpose = _build_transpose_meta   # the reference's name for it (stk/matrix.py:105-123): same arguments, same three results


def _validate_matrix(shape, data, row_indices, column_indices, offsets):
    """Shape / dtype / device checks of stk/matrix.py:14-102 (ValueError on failure)."""
    if data.dim() == 1:
        data = data.reshape(data.numel(), 1, 1)
    if data.shape[-2] != data.shape[-1]:
        raise ValueError(f"Expected square blocking in data. Got block shape {list(data.shape[-2:])}")
    b = data.shape[-1]
    data = data.view(-1, b, b)
    if shape[-2] % b != 0 or shape[-1] % b != 0:
        raise ValueError(f"Matrix shape must be dividible by blocking. Got shape {shape} with {[b, b]} blocking.")
    if np.prod(shape) < data.numel():
        raise ValueError(f"Invalid matrix. Number of nonzeros exceeds matrix capacity ({data.numel()} v. {np.prod(shape)})")
    for name, t in (("row_indices", row_indices), ("column_indices", column_indices), ("offsets", offsets)):
        if t.dim() != 1:
            raise ValueError(f"Expected 1D {name}. Got {t.dim()}D {name}.")
    for name, t in (("row_indices", row_indices), ("column_indices", column_indices)):
        if t.numel() != data.shape[0]:
            raise ValueError(f"Expected 1 index per nonzero block. Got {t.numel()} {name} for {data.shape[0]} blocks")
    block_rows = np.prod(shape[:-1]) / b
    if offsets.numel() != block_rows + 1:
        raise ValueError(f"Expected one offset per block row plus one. Got {offsets.numel()} offsets with {block_rows} block rows.")
    on_gpu = [t.is_cuda for t in (data, row_indices, column_indices, offsets)]
    if any(on_gpu) and not all(on_gpu):
        raise ValueError(
            f"Expected data & meta-data on common device. Got data on {data.device}, row_indices on {row_indices.device} "
            f"column_indices on {column_indices.device} and offsets on {offsets.device}.")
    if data.dtype != torch.float16:
        raise ValueError(f"Expected float16 data. Got {data.dtype} data.")
    for name, t in (("row_indices", row_indices), ("column_indices", column_indices)):
        if t.dtype != torch.int16:
            raise ValueError(f"Expected int16 {name}. Got {t.dtype} {name}.")
    if offsets.dtype != torch.int32:
        raise ValueError(f"Expected int32 offsets. Got {offsets.dtype} offsets.")
    return data


class Matrix(torch.nn.Module):
    """A matrix stored in block compressed sparse row format with COO row indices."""

    _TENSORS = ("_data", "_row_indices", "_column_indices", "_offsets",
                "_column_indices_t", "_offsets_t", "_block_offsets_t")

    def __init__(self, size, data, row_indices, column_indices, offsets,
                 column_indices_t=None, offsets_t=None, block_offsets_t=None):
        super().__init__()
        if column_indices_t is None or offsets_t is None or block_offsets_t is None:
            column_indices_t, offsets_t, block_offsets_t = _build_transpose_meta(
                size, data, row_indices, column_indices, offsets)
        # plain attributes, as in the reference (tensors assigned to a Module are neither parameters nor
        # buffers); set past Module.__setattr__, whose checks cost more than the rest of the constructor
        self.__dict__.update(_size=size, _data=data, _row_indices=row_indices, _column_indices=column_indices,
                             _offsets=offsets, _column_indices_t=column_indices_t, _offsets_t=offsets_t,
                             _block_offsets_t=block_offsets_t, _transposed=False)

        # 16-bit indices must be able to address every block (stk/matrix.py:161-167)
        if column_indices.dtype == torch.int16:
            limit = _INT16_MAX * self.blocking
            if size[0] > limit or size[1] > limit:
                raise ValueError(f"Sparse matrix with shape {size} exceeds representable size with 16-bit indices.")

    # ---- construction helpers -------------------------------------------------
    def _like(self, size, data):
        return Matrix(size, data, self._row_indices, self._column_indices, self._offsets,
                      self._column_indices_t, self._offsets_t, self._block_offsets_t)

    def validate(self):
        _validate_matrix(self._size, self._data, self._row_indices, self._column_indices, self._offsets)

    def to(self, device):
        for name in self._TENSORS:
            setattr(self, name, getattr(self, name).to(device))
        return self

    def cuda(self):
        return self.to(torch.cuda.current_device())

    def clone(self):
        return Matrix(self.size(), *(getattr(self, name).clone() for name in self._TENSORS))

    def t(self):
        if self.dim() != 2:
            raise ValueError(f"t() expects a tensor with <= 2 dimensions, but self is {self.dim()}D.")
        out = self._like(self.size(), self._data)
        out._transposed = not self._transposed
        out._size = torch.Size((self._size[1], self._size[0]))
        return out

    def contiguous(self):
        raise ValueError("Not yet implemented.")

    def is_contiguous(self):
        return not self._transposed

    def view(self, *shape):
        assert self.is_contiguous()
        if shape[-1] != self.size()[-1]:
            raise ValueError(f"Can't change view on compressed dimension. {self.size()[-1]} v. {shape[-1]}.")
        if np.prod(shape) != np.prod(self.size()):
            raise ValueError(f"Mismatch in numel of Matrix and new shape. {np.prod(self.size())} v. {np.prod(shape)}")
        return self._like(shape, self._data)

    # ---- tensor-like surface --------------------------------------------------
    def size(self):
        return self._size

    @property
    def shape(self):
        return self.size()

    def dim(self):
        return len(self._size)

    @property
    def is_cuda(self):
        return self._data.is_cuda

    @property
    def device(self):
        return self._data.device

    @property
    def dtype(self):
        return self._data.dtype

    @property
    def nnz(self):
        return self._data.numel()

    @property
    def blocking(self):
        return self._data.shape[1]

    @property
    def requires_grad(self):
        return self._data.requires_grad

    def requires_grad_(self, x):
        self._data.requires_grad_(x)
        return self

    @property
    def grad(self):
        size = self.size()
        if self._transposed:
            size = torch.Size((size[1], size[0]))
        g = self._like(size, self._data.grad)
        return g.t() if self._transposed else g

    data = property(lambda self: self._data)
    row_indices = property(lambda self: self._row_indices)
    column_indices = property(lambda self: self._column_indices)
    offsets = property(lambda self: self._offsets)
    column_indices_t = property(lambda self: self._column_indices_t)
    offsets_t = property(lambda self: self._offsets_t)
    block_offsets_t = property(lambda self: self._block_offsets_t)
