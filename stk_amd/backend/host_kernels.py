"""Host (CPU) tensors: the same backend functions as hip_kernels, backed by libstk_amd_host.so.

The reference has no CPU kernels for the products (Triton needs a GPU), but it builds every matrix on the host
(stk/ops/linear_ops_test.py:57-63, stk/random/random_ops.py:26-28) and its plumbing configuration checks the products
on host tensors against to_dense + torch.matmul (linear_ops_test.py:83-96, 110-111).  `sdd`, `dsd`, `dds` and
`row_indices` keep the positional signatures of stk/backend/triton_kernels.py (:332-339, :222-233, :278-289,
:389-391); hip_kernels hands them every call whose tensors live in host memory.  The library is plain C++ (float16,
bfloat16 and float32 values, fp32 accumulation) declared in include/stk_amd_host.h; nothing here touches a GPU, and no
device tensor ever comes here.
"""
import ctypes
import os
import threading

import torch

from stk_amd.backend import _lib

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "libstk_amd_host.so")

STK_F32 = 2
_VALUE_DTYPES = {torch.float16: _lib.STK_F16, torch.bfloat16: _lib.STK_BF16, torch.float32: STK_F32}
_INDEX_DTYPES = {torch.int16: _lib.STK_I16, torch.int32: _lib.STK_I32}

_p, _i64, _int = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int

# name -> (restype, argtypes); mirrors include/stk_amd_host.h one to one
SIGNATURES = {
    "stk_cpu_last_error": (ctypes.c_char_p, []),
    "stk_cpu_sdd": (_int, [_p, _i64, _i64, _p, _i64, _i64, _i64, _i64, _i64, _p, _p, _p, _i64, _int, _int, _int]),
    "stk_cpu_dsd": (_int, [_i64, _i64, _i64, _p, _p, _p, _p, _p, _p, _int, _p, _i64, _i64, _p, _i64, _i64, _int, _int, _int]),
    "stk_cpu_dds": (_int, [_i64, _i64, _i64, _p, _i64, _i64, _p, _p, _p, _p, _p, _p, _int, _p, _i64, _i64, _int, _int, _int]),
    "stk_cpu_row_indices": (_int, [_p, _i64, _i64, _p, _int]),
    "stk_cpu_transpose_meta": (_int, [_p, _p, _i64, _i64, _int, _p, _p, _p]),
    "stk_cpu_to_dense": (_int, [_p, _p, _p, _i64, _int, _i64, _i64, _int, _int, _p]),
    "stk_cpu_to_sparse_count": (_int, [_p, _i64, _i64, _i64, _int, _int, _p, _p]),
    "stk_cpu_to_sparse_fill": (_int, [_p, _i64, _i64, _i64, _int, _int, _p, _p, _i64, _p, _p, _p, _int]),
}

_lock = threading.Lock()
_host = None


def load():
    """Returns the loaded host library, loading it on first use."""
    global _host
    if _host is not None:
        return _host
    with _lock:
        if _host is None:
            if not os.path.exists(LIB_PATH):
                raise RuntimeError(f"stk_amd: {LIB_PATH} is missing. Build it with `make -C stk_amd/csrc` (g++); "
                                   "host tensors have no other implementation.")
            lib = ctypes.CDLL(LIB_PATH)
            for name, (res, args) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = res
                fn.argtypes = args
            _host = lib
    return _host


def check(status):
    """The exceptions of the device boundary for the same status codes."""
    if status == _lib.STK_OK:
        return
    msg = load().stk_cpu_last_error().decode("utf-8", "replace")
    if status == _lib.STK_ERR_DIMS:
        raise AssertionError(msg)
    if status == _lib.STK_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)


def _value_dtype(t):
    if t.dtype not in _VALUE_DTYPES:
        raise NotImplementedError(f"stk_amd: products on host tensors take float16, bfloat16 or float32 values, got {t.dtype}")
    return _VALUE_DTYPES[t.dtype]


def _index(t):
    if t.dtype not in _INDEX_DTYPES:
        raise NotImplementedError(f"stk_amd: indices must be int16 or int32, got {t.dtype}")
    return t if t.is_contiguous() else t.contiguous()


def _offsets(t):
    if t.dtype != torch.int32:
        raise NotImplementedError(f"stk_amd: offsets must be int32, got {t.dtype}")
    return t if t.is_contiguous() else t.contiguous()


def _host_only(*tensors):
    for t in tensors:
        if t is not None and t.is_cuda:
            raise RuntimeError("stk_amd: operands of one product must all live in host memory or all on one GPU")


def sdd(lhs, rhs, shape, out, offsets, row_indices, column_indices):
    _host_only(lhs, rhs, out, row_indices, column_indices)
    m, k = lhs.shape
    n = rhs.shape[1]
    assert out.is_contiguous() and lhs.dtype == rhs.dtype == out.dtype
    ri, ci = _index(row_indices), _index(column_indices)
    assert ri.dtype == ci.dtype
    check(load().stk_cpu_sdd(lhs.data_ptr(), lhs.stride(0), lhs.stride(1), rhs.data_ptr(), rhs.stride(0), rhs.stride(1), m, k, n,
                             out.data_ptr(), ri.data_ptr(), ci.data_ptr(), ri.numel(), out.shape[-1], _value_dtype(out), _INDEX_DTYPES[ri.dtype]))


def dsd(shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t, transpose_a, rhs, out):
    _host_only(data, rhs, out, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t)
    m, k = shape
    data = data.detach()
    assert data.is_contiguous() and out.stride(1) == 1 and data.dtype == rhs.dtype == out.dtype
    ci, cit = _index(column_indices), _index(column_indices_t)
    assert ci.dtype == cit.dtype
    check(load().stk_cpu_dsd(m, k, rhs.shape[1], data.data_ptr(), _offsets(offsets).data_ptr(), ci.data_ptr(),
                             _offsets(offsets_t).data_ptr(), cit.data_ptr(), _offsets(block_offsets_t).data_ptr(), 1 if transpose_a else 0,
                             rhs.data_ptr(), rhs.stride(0), rhs.stride(1), out.data_ptr(), out.stride(0), data.shape[0], data.shape[-1],
                             _value_dtype(out), _INDEX_DTYPES[ci.dtype]))


def dds(lhs, shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t, transpose_b, out):
    _host_only(data, lhs, out, offsets, column_indices, offsets_t, column_indices_t, block_offsets_t)
    m, k = lhs.shape
    data = data.detach()
    assert data.is_contiguous() and out.stride(1) == 1 and data.dtype == lhs.dtype == out.dtype
    ci, cit = _index(column_indices), _index(column_indices_t)
    assert ci.dtype == cit.dtype
    check(load().stk_cpu_dds(m, k, shape[1], lhs.data_ptr(), lhs.stride(0), lhs.stride(1), data.data_ptr(),
                             _offsets(offsets).data_ptr(), ci.data_ptr(), _offsets(offsets_t).data_ptr(), cit.data_ptr(),
                             _offsets(block_offsets_t).data_ptr(), 1 if transpose_b else 0, out.data_ptr(), out.stride(0),
                             data.shape[0], data.shape[-1], _value_dtype(out), _INDEX_DTYPES[ci.dtype]))


def row_indices(shape, data, offsets, column_indices, out):
    _host_only(offsets, out)
    assert out.is_contiguous()
    offsets = _offsets(offsets)
    check(load().stk_cpu_row_indices(offsets.data_ptr(), offsets.numel() - 1, out.numel(), out.data_ptr(), _INDEX_DTYPES[out.dtype]))


def transpose_meta(size, data, row_indices, column_indices, offsets):
    """(column_indices_t, offsets_t, block_offsets_t), stable tie order."""
    block_cols = size[1] // data.shape[-1]
    ri, ci = _index(row_indices), _index(column_indices)
    assert ri.dtype == ci.dtype
    nnz = ci.numel()
    column_indices_t = torch.empty(nnz, dtype=ri.dtype)
    offsets_t = torch.empty(block_cols + 1, dtype=torch.int32)
    block_offsets_t = torch.empty(nnz, dtype=torch.int32)
    check(load().stk_cpu_transpose_meta(ri.data_ptr(), ci.data_ptr(), nnz, block_cols, _INDEX_DTYPES[ci.dtype],
                                        column_indices_t.data_ptr(), offsets_t.data_ptr(), block_offsets_t.data_ptr()))
    return column_indices_t, offsets_t, block_offsets_t


def handles(t):
    """Element types the format twins copy: 2- and 4-byte floating point and integers."""
    return t.element_size() in (2, 4) and not t.is_complex()


def to_dense(data, row_indices, column_indices, rows, cols):
    data = data.detach().contiguous()
    ri, ci = _index(row_indices), _index(column_indices)
    out = torch.empty((rows, cols), dtype=data.dtype)
    check(load().stk_cpu_to_dense(data.data_ptr(), ri.data_ptr(), ci.data_ptr(), data.shape[0], data.shape[-1], rows, cols,
                                  data.element_size(), _INDEX_DTYPES[ci.dtype], out.data_ptr()))
    return out


def to_sparse(x, blocking, index_dtype=torch.int16):
    """(data, row_indices, column_indices, offsets) of the nonzero blocks of x, row-major order."""
    rows, cols = x.shape
    x = x.detach()
    if x.stride(1) != 1 and cols > 1:
        x = x.contiguous()
    br, bc = rows // blocking, cols // blocking
    mask = torch.empty(max(br * bc, 1), dtype=torch.uint8)
    offsets = torch.empty(br + 1, dtype=torch.int32)
    lib = load()
    stride = x.stride(0) if rows > 1 else max(cols, 1)
    check(lib.stk_cpu_to_sparse_count(x.data_ptr(), rows, cols, stride, blocking, x.element_size(), mask.data_ptr(), offsets.data_ptr()))
    nnz = int(offsets[-1])
    data = torch.empty((nnz, blocking, blocking), dtype=x.dtype)
    row_indices = torch.empty(nnz, dtype=index_dtype)
    column_indices = torch.empty(nnz, dtype=index_dtype)
    check(lib.stk_cpu_to_sparse_fill(x.data_ptr(), rows, cols, stride, blocking, x.element_size(), mask.data_ptr(), offsets.data_ptr(), nnz,
                                     data.data_ptr(), row_indices.data_ptr(), column_indices.data_ptr(), _INDEX_DTYPES[index_dtype]))
    return data, row_indices, column_indices, offsets
