"""Kernel boundary: the functions the autograd layer calls, backed by libstk_amd.so.

`sdd`, `dsd`, `dds` and `row_indices` keep the positional signatures of
stk/backend/triton_kernels.py (:332-339, :222-233, :278-289, :389-391), write
into a caller-allocated `out`, return None and raise AssertionError for the
same shape violations (:15-19, :243, :299, :351).  `transpose_meta`, `to_dense`
and `to_sparse` are the device versions of stk/matrix.py:105-123 and
stk/ops/matrix_ops.py:36-85.

Device tensors launch on torch's current stream without synchronising (to_sparse
reads one int back, as the reference's torch.nonzero does); for them nothing falls
back to another implementation.  Calls of the four reference functions whose tensors
all live in host memory are handed to the host library (host_kernels), which is how
the reference's plumbing configuration - products on CPU tensors - runs here.
"""
import ctypes
import threading
import time

import torch

from stk_amd.backend import _lib, host_kernels

_VALUE_DTYPES = {torch.float16: _lib.STK_F16, torch.bfloat16: _lib.STK_BF16, torch.float32: _lib.STK_F32}
_INDEX_DTYPES = {torch.int16: _lib.STK_I16, torch.int32: _lib.STK_I32}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream(device=None):
    """Handle of torch's current stream on `device` (default: the current device).  Read through torch's C entry
    points where they exist: torch.cuda.current_stream() builds a Stream object, which costs several microseconds
    on a path that every launch takes."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device() if device is None or device.index is None else device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _capture_id(device=None):
    """Identifier of the graph capture under way on the current stream of `device`, 0 outside captures.  A buffer
    allocated or filled while a capture is under way exists only in that graph's replays: the caches below keep
    such a buffer apart from launches outside that capture."""
    out = ctypes.c_uint64(0)
    _lib.check(_lib.load().stk_stream_capture_id(_stream(device), ctypes.byref(out)))
    return out.value


class _on_device:
    """`with _on_device(d):` makes d the current device like torch.cuda.device(d), but costs nothing when it
    already is (the usual case, and this sits on the launch path of every product)."""

    def __init__(self, device):
        current = _raw_device() if _raw_device is not None else torch.cuda.current_device()
        self._guard = None if device.index is None or device.index == current else torch.cuda.device(device)

    def __enter__(self):
        if self._guard is not None:
            self._guard.__enter__()

    def __exit__(self, *exc):
        if self._guard is not None:
            return self._guard.__exit__(*exc)
        return False


def _need_gpu(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("stk_amd: this operation runs on a ROCm GPU only; got a tensor on " + str(t.device))


def _value_dtype(t):
    if t.dtype not in _VALUE_DTYPES:
        raise NotImplementedError(f"stk_amd: products need float16, bfloat16 or float32 values, got {t.dtype}")
    return _VALUE_DTYPES[t.dtype]


def _index(t, like=None):
    """Index tensors may arrive as strided views (stk/ops/matrix_ops.py:73-75)."""
    if t.dtype not in _INDEX_DTYPES:
        raise NotImplementedError(f"stk_amd: indices must be int16 or int32, got {t.dtype}")
    return t if t.is_contiguous() else t.contiguous()


def _offsets(t):
    if t.dtype != torch.int32:
        raise NotImplementedError(f"stk_amd: offsets must be int32, got {t.dtype}")
    return t if t.is_contiguous() else t.contiguous()


def _dense_operand(x):
    """A 2-D operand the kernels can read in place: unit stride in one dimension,
    the other stride a multiple of 8 elements, 16-byte aligned base.  Anything
    else is copied to row-major first."""
    assert x.dim() == 2
    s0, s1 = x.stride()
    ok = ((s1 == 1 and s0 % 8 == 0) or (s0 == 1 and s1 % 8 == 0 and x.size(0) > 1)) and x.data_ptr() % 16 == 0
    if not ok:
        x = x.contiguous()
        if x.data_ptr() % 16 or x.stride(0) % 8:
            raise NotImplementedError("stk_amd: dense operands need a row length divisible by 8")
    return x


def _blocking(data):
    return data.shape[-1]


def _validate_matmul_dims(m, k, n, blocking):
    # stk/backend/triton_kernels.py:15-19 with BLOCK_M = BLOCK_N = blocking, BLOCK_K = 32
    msg = "incompatible dimensions: tensor has dim with length: {}, which must be divisible by {}"
    assert m % blocking == 0, msg.format(m, blocking)
    assert k % 32 == 0, msg.format(k, 32)
    assert n % blocking == 0, msg.format(n, blocking)


# Tile fusion across identical neighbouring block rows / columns (stk_build_plan).  Results do not
# depend on it; switching it off makes every product take the one-line-per-tile kernels.
FUSION = True


def _version_of(t):
    """In-place modification counter of a tensor, or None for a tensor that keeps none (inference mode)."""
    return None if t.is_inference() else t._version


def _plan_cache_get(tensors, blocking):
    """The cache entry on tensors[0] (`offsets`) if it describes exactly these index tensors in their
    present state, else None.  The entry keeps the other index tensors it was built from: their storage
    stays alive, so an address cannot come back with other contents, and identity plus the version
    counters say whether they still hold what the plan describes.  A plan built with the transpose
    metadata also serves a request without it."""
    cached = getattr(tensors[0], "_stk_plan", None)
    if cached is None or cached[2] != blocking or len(cached[0]) < len(tensors) - 1:
        return None
    versions = tuple(_version_of(t) for t in tensors)
    if None in versions or cached[5][:len(versions)] != versions or not all(a is b for a, b in zip(cached[0], tensors[1:])):
        return None
    return cached


def _plan_cache_put(tensors, blocking, plan, stream_handle, built, capture):
    """Remembers `plan` on tensors[0]; tensors without a version counter (made under inference mode)
    cannot be watched for in-place changes and are not cached.  `capture`: the graph capture the plan was built in
    (0: none)."""
    versions = tuple(_version_of(t) for t in tensors)
    if None in versions:
        return False
    try:
        tensors[0]._stk_plan = (tuple(tensors[1:]), plan, blocking, stream_handle, built, versions, capture)
    except AttributeError:
        return False
    return True


def fusion_plan(offsets, column_indices, offsets_t=None, column_indices_t=None, blocking=128):
    """Device tensor with the fusion roles of the block rows (and, when the
    transpose metadata is given, of the block columns): which neighbouring lines
    repeat each other and are computed as one 256-wide tile.  Depends on the
    topology only, so it is cached on the `offsets` tensor and rebuilt when one of
    the index tensors has been replaced or modified in place.

    Under a graph capture: a plan built before the capture is used as it is (on another stream than the one that
    built it without waiting for the build, which a capture cannot do: the build must be complete when the capture
    starts, as it is after the synchronisation with which torch.cuda.graph() begins); a plan built inside a capture
    serves that capture only, and launches outside it build their own."""
    _need_gpu(offsets, column_indices)
    want_cols = offsets_t is not None and column_indices_t is not None
    tensors = (offsets, column_indices) + ((offsets_t, column_indices_t) if want_cols else ())
    cached = _plan_cache_get(tensors, blocking)
    if cached is not None:
        handle, built_in = _stream(offsets.device), cached[6]
        if built_in == 0 and cached[3] == handle:
            return cached[1]
        capture = _capture_id(offsets.device)
        if built_in in (0, capture):
            if cached[3] != handle and (built_in != 0 or capture == 0):
                # built on another stream: what this one launches next comes after the build
                torch.cuda.current_stream(offsets.device).wait_event(cached[4])
            return cached[1]
    else:
        capture = _capture_id(offsets.device)
    block_rows = offsets.numel() - 1
    block_cols = offsets_t.numel() - 1 if want_cols else 0
    lib = _lib.load()
    nnz = column_indices.numel()
    nbytes = lib.stk_plan_bytes(block_rows, block_cols, nnz)
    plan = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=offsets.device)
    ci = _index(column_indices)
    cit = _index(column_indices_t) if want_cols else None
    with _on_device(offsets.device):
        _lib.check(lib.stk_build_plan(
            _offsets(offsets).data_ptr(), ci.data_ptr(), block_rows,
            _offsets(offsets_t).data_ptr() if want_cols else None, cit.data_ptr() if want_cols else None, block_cols,
            nnz, blocking, _INDEX_DTYPES[ci.dtype], plan.data_ptr(), nbytes, _stream()))
    stream = torch.cuda.current_stream(offsets.device)
    built = torch.cuda.Event()
    built.record(stream)
    _plan_cache_put(tensors, blocking, plan, stream.cuda_stream, built, capture)
    return plan


def prepare_plan(data, offsets, column_indices, offsets_t, column_indices_t):
    """Builds the fusion plan of a topology for both directions if there is none yet.  sdd itself needs the block rows
    only (its signature, the reference's, has no transpose metadata), so a plan built by its first call would be built
    again, with the columns, by the dsd or dds that follows on the same topology; callers that have the whole metadata
    at hand (the autograd functions) call this first and every product finds the one plan."""
    b = data.shape[-1] if data.dim() == 3 else 0
    if FUSION and b in (64, 128) and offsets.is_cuda and column_indices.numel() > 0:
        fusion_plan(offsets, column_indices, offsets_t, column_indices_t, blocking=b)


ACTIVATIONS = {None: 0, "none": 0, "relu": 1, "gelu_tanh": 2, "gelu": 3, "silu": 4,
               # the derivatives: with the incoming gradient as the multiplier, the gradient with respect to the sums
               "relu_grad": 5, "gelu_tanh_grad": 6, "gelu_grad": 7, "silu_grad": 8}


def sdd(lhs, rhs, shape, out, offsets, row_indices, column_indices, block_order=None):
    """out[p] = lhs[block row p] @ rhs[block column p]; out is [nnz, b, b].

    block_order (optional, not in the reference signature) is a permutation of
    the blocks that sets the visiting order of workgroups for 64x64 blocks.
    """
    sdd_fused(lhs, rhs, shape, out, offsets, row_indices, column_indices, None, None, block_order)


def sdd_fused(lhs, rhs, shape, out, offsets, row_indices, column_indices, activation=None, multiplier=None,
              block_order=None, sums=None):
    """sdd whose store applies `activation` (a key of ACTIVATIONS) to the fp32 sums and, after the
    rounding, multiplies by `multiplier` ([nnz, b, b] values of a matrix with the same topology).
    `sums` (like `out`, or None) also receives the rounded sums themselves (stk_sdd_fused_sums).
    No counterpart as one call in the reference, whose callers run the activation and
    stk.ops.mul (stk/ops/eltwise_ops.py:3-28) as passes of their own over the values."""
    assert lhs.shape[1] == rhs.shape[0], "incompatible dimensions"
    m, k = lhs.shape
    n = rhs.shape[1]
    b = _blocking(out)
    _validate_matmul_dims(m, k, n, b)
    if not out.is_cuda:
        if ACTIVATIONS.get(activation, 1) != 0 or multiplier is not None or sums is not None:
            raise NotImplementedError("stk_amd: the fused store of sdd runs on a GPU only")
        return host_kernels.sdd(lhs, rhs, shape, out, offsets, row_indices, column_indices)
    _need_gpu(lhs, rhs, out)
    assert out.is_contiguous()
    if activation not in ACTIVATIONS:
        raise ValueError(f"unknown activation {activation!r}; one of {sorted(k for k in ACTIVATIONS if k)}")
    nnz = row_indices.numel()
    if multiplier is not None:
        _need_gpu(multiplier)
        assert multiplier.shape == out.shape and multiplier.dtype == out.dtype and multiplier.is_contiguous()
    if sums is not None:
        _need_gpu(sums)
        assert sums.shape == out.shape and sums.dtype == out.dtype and sums.is_contiguous() and sums.data_ptr() != out.data_ptr()
    if nnz == 0:
        return
    lhs, rhs = _dense_operand(lhs), _dense_operand(rhs)
    assert lhs.dtype == rhs.dtype == out.dtype
    ri, ci = _index(row_indices), _index(column_indices)
    assert ri.dtype == ci.dtype
    order = None
    if block_order is not None:
        assert block_order.dtype == torch.int32 and block_order.numel() == nnz
        order = block_order.contiguous()
    plan = fusion_plan(offsets, column_indices, blocking=b) if FUSION and b in (64, 128) and offsets is not None else None
    with _on_device(out.device):
        _lib.check(_lib.load().stk_sdd_fused_sums(
            lhs.data_ptr(), lhs.stride(0), lhs.stride(1), rhs.data_ptr(), rhs.stride(0), rhs.stride(1),
            m, k, n, out.data_ptr(), _offsets(offsets).data_ptr() if plan is not None else None, ri.data_ptr(), ci.data_ptr(),
            order.data_ptr() if order is not None else None, nnz,
            b, _value_dtype(out), _INDEX_DTYPES[ri.dtype], plan.data_ptr() if plan is not None else None,
            ACTIVATIONS[activation], multiplier.data_ptr() if multiplier is not None else None,
            sums.data_ptr() if sums is not None else None, _stream()))


def activation_product(sums, factor, activation):
    """round(round(act(sums)) * factor) over the values of a sparse matrix (factor None: the first rounding only);
    `activation` a key of ACTIVATIONS, derivatives included (stk_activation_product)."""
    _need_gpu(sums)
    if activation not in ACTIVATIONS:
        raise ValueError(f"unknown activation {activation!r}")
    sums = sums.detach().contiguous()
    out = torch.empty_like(sums)
    if factor is not None:
        _need_gpu(factor)
        factor = factor.detach().contiguous()
        assert factor.shape == sums.shape and factor.dtype == sums.dtype
    if sums.numel() == 0:
        return out
    with _on_device(sums.device):
        _lib.check(_lib.load().stk_activation_product(sums.data_ptr(), factor.data_ptr() if factor is not None else None, out.data_ptr(),
                                                      sums.numel(), ACTIVATIONS[activation], _value_dtype(sums), _stream()))
    return out


# dsd launches that fill the GPU only a few times cut the tiles of their last round into slices
# along k, which takes a workspace.  Results then differ in the last bit from the uncut sums;
# switching it off restores those.
SLICE_LAST_ROUND = True
# Partial tiles (256 KiB each) the workspace of a device has room for: 256 of them (64 MiB) let a last round of
# 128 tiles be cut in two, or one of 64 tiles in four; a launch that would like more is cut less.  The buffer is
# allocated on the first dsd that can use it and kept; release_workspaces() frees it.
DSD_WORKSPACE_SLOTS = 256
# Streams whose dsd launches may run beside those of other streams (the autograd layer's side stream): they get
# a workspace of their own.  Everything else shares one per device, and a launch on another stream than the
# last one first waits for that stream.
CONCURRENT_STREAMS = set()
_dsd_workspaces = {}   # (device index, concurrent lane) -> [buffer, stream of the last launch]


def release_workspaces():
    """Frees the dsd workspaces (they are allocated again on demand)."""
    _dsd_workspaces.clear()


def _workspace_choice(capturing, entry_stream, handle):
    """Which workspace a dsd launch on the stream `handle` takes.  `capturing`: a graph capture is under way on that
    stream; `entry_stream`: handle of the stream that last used the device's shared workspace (None: there is none yet).
      "private"  a buffer of the launch's own.  Every captured launch: its buffer comes out of the graph's memory pool, so
                 replays - on whatever stream, next to whatever eager launches or other graphs - share counters and
                 partial-tile slots with nobody.
      "create"   no shared workspace yet: allocate it for this stream.
      "shared"   the shared workspace, last used on this very stream: launches on one stream cannot overlap.
      "wait"     the shared workspace after waiting for the stream that used it last."""
    if capturing:
        return "private"
    if entry_stream is None:
        return "create"
    return "shared" if entry_stream == handle else "wait"


def _new_workspace(device, nbytes, counters):
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    ws[:counters].zero_()   # (a fill kernel, also under capture; the slots behind the counters need no initial value)
    return ws


def _dsd_workspace(device, m, n, blocking):
    """Workspace of stk_dsd for this shape, or None: [counters | slots], the counters zero between launches."""
    if not SLICE_LAST_ROUND:
        return None
    lib = _lib.load()
    if lib.stk_dsd_workspace_bytes(m, n, blocking) <= 0:
        return None
    handle = _stream(device)
    key = (device.index, handle in CONCURRENT_STREAMS)
    entry = _dsd_workspaces.get(key)
    counters = lib.stk_dsd_workspace_counter_bytes()
    nbytes = counters + DSD_WORKSPACE_SLOTS * lib.stk_dsd_workspace_slot_bytes()
    if entry is not None and entry[0].numel() != nbytes:
        entry = None
    choice = _workspace_choice(_capture_id(device) != 0, None if entry is None else entry[1].cuda_stream, handle)
    if choice == "private":
        # zeroed by a fill kernel that is part of the graph; the memory goes back to the graph's pool when the
        # caller drops it, where only later allocations of the same capture, which run behind this launch, reuse it
        return _new_workspace(device, nbytes, counters)
    if choice == "create":
        entry = _dsd_workspaces[key] = [_new_workspace(device, nbytes, counters), torch.cuda.current_stream(device)]
    elif choice == "wait":
        stream = torch.cuda.current_stream(device)
        stream.wait_stream(entry[1])   # launches that share a workspace must not overlap
        entry[1] = stream
    return entry[0]


def dsd(shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t,
        block_offsets_t, transpose_a, rhs, out):
    """out = op(sparse) @ rhs; `shape` is the logical shape of the sparse operand."""
    assert shape[1] == rhs.shape[0], "incompatible dimensions"
    m, k = shape
    n = rhs.shape[1]
    b = _blocking(data)
    _validate_matmul_dims(m, k, n, b)
    if not out.is_cuda:
        return host_kernels.dsd(shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t,
                                transpose_a, rhs, out)
    _need_gpu(data, rhs, out)
    rhs = _dense_operand(rhs)
    data = data.detach()
    assert data.is_contiguous() and out.stride(1) == 1
    assert data.dtype == rhs.dtype == out.dtype
    ci, cit = _index(column_indices), _index(column_indices_t)
    plan = fusion_plan(offsets, column_indices, offsets_t, column_indices_t, blocking=b) if FUSION and b in (64, 128) and data.shape[0] > 0 else None
    with _on_device(out.device):
        ws = _dsd_workspace(out.device, m, n, b) if plan is not None else None
        status = _lib.load().stk_dsd(
            m, k, n, data.data_ptr(), _offsets(offsets).data_ptr(), ci.data_ptr(),
            _offsets(offsets_t).data_ptr(), cit.data_ptr(), _offsets(block_offsets_t).data_ptr(),
            1 if transpose_a else 0, rhs.data_ptr(), rhs.stride(0), rhs.stride(1),
            out.data_ptr(), out.stride(0), data.shape[0], b, _value_dtype(out), _INDEX_DTYPES[ci.dtype],
            plan.data_ptr() if plan is not None else None,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, _stream())
        if status != _lib.STK_OK and ws is not None:
            release_workspaces()   # whatever a failed launch left in the counters is not reused
        _lib.check(status)


def dds(lhs, shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t,
        block_offsets_t, transpose_b, out):
    """out = lhs @ op(sparse); `shape` is the logical shape of the sparse operand."""
    assert lhs.shape[1] == shape[0], "incompatible dimensions"
    m, k = lhs.shape
    n = shape[1]
    b = _blocking(data)
    _validate_matmul_dims(m, k, n, b)
    if not out.is_cuda:
        return host_kernels.dds(lhs, shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t,
                                transpose_b, out)
    _need_gpu(data, lhs, out)
    lhs = _dense_operand(lhs)
    data = data.detach()
    assert data.is_contiguous() and out.stride(1) == 1
    assert data.dtype == lhs.dtype == out.dtype
    ci, cit = _index(column_indices), _index(column_indices_t)
    plan = fusion_plan(offsets, column_indices, offsets_t, column_indices_t, blocking=b) if FUSION and b in (64, 128) and data.shape[0] > 0 else None
    with _on_device(out.device):
        _lib.check(_lib.load().stk_dds(
            m, k, n, lhs.data_ptr(), lhs.stride(0), lhs.stride(1), data.data_ptr(),
            _offsets(offsets).data_ptr(), ci.data_ptr(), _offsets(offsets_t).data_ptr(), cit.data_ptr(),
            _offsets(block_offsets_t).data_ptr(), 1 if transpose_b else 0,
            out.data_ptr(), out.stride(0), data.shape[0], b, _value_dtype(out), _INDEX_DTYPES[ci.dtype],
            plan.data_ptr() if plan is not None else None, _stream()))


def dsd_dds(shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t, rhs, out_dsd, lhs, out_dds):
    """out_dsd = sparse @ rhs and out_dds = lhs @ sparse for one sparse operand [m, k] = `shape`, in one launch where
    the layouts allow it (the two gradients of sdd, stk/backend/sputnik.py:274-299); otherwise the two products one
    after the other.  The results are those of dsd (without its workspace) and dds, bit for bit."""
    _need_gpu(data, rhs, lhs, out_dsd, out_dds)
    m, k = shape
    assert rhs.shape[0] == k and lhs.shape[1] == m, "incompatible dimensions"
    b = _blocking(data)
    _validate_matmul_dims(m, k, rhs.shape[1], b)
    _validate_matmul_dims(lhs.shape[0], m, k, b)
    rhs, lhs = _dense_operand(rhs), _dense_operand(lhs)
    data = data.detach()
    assert data.is_contiguous() and out_dsd.stride(1) == 1 and out_dds.stride(1) == 1
    assert data.dtype == rhs.dtype == lhs.dtype == out_dsd.dtype == out_dds.dtype
    ci, cit = _index(column_indices), _index(column_indices_t)
    plan = fusion_plan(offsets, column_indices, offsets_t, column_indices_t, blocking=b) if FUSION and b in (64, 128) and data.shape[0] > 0 else None
    with _on_device(out_dsd.device):
        _lib.check(_lib.load().stk_dsd_dds(
            m, k, data.data_ptr(), _offsets(offsets).data_ptr(), ci.data_ptr(),
            _offsets(offsets_t).data_ptr(), cit.data_ptr(), _offsets(block_offsets_t).data_ptr(),
            rhs.shape[1], rhs.data_ptr(), rhs.stride(0), rhs.stride(1), out_dsd.data_ptr(), out_dsd.stride(0),
            lhs.shape[0], lhs.data_ptr(), lhs.stride(0), lhs.stride(1), out_dds.data_ptr(), out_dds.stride(0),
            data.shape[0], b, _value_dtype(data), _INDEX_DTYPES[ci.dtype], plan.data_ptr() if plan is not None else None, _stream()))


def dsd_dsd(shape, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t, rhs, out, rhs_t, out_t):
    """out = sparse @ rhs and out_t = sparse^T @ rhs_t for one sparse operand [m, k] = `shape`, in one launch where the
    layouts allow it (the two gradients of an sdd whose rhs was a .t() view, stk/backend/sputnik.py:274-299); otherwise
    the two products one after the other.  The results are those of two dsd calls without the workspace, bit for bit."""
    _need_gpu(data, rhs, rhs_t, out, out_t)
    m, k = shape
    assert rhs.shape[0] == k and rhs_t.shape[0] == m, "incompatible dimensions"
    b = _blocking(data)
    _validate_matmul_dims(m, k, rhs.shape[1], b)
    _validate_matmul_dims(k, m, rhs_t.shape[1], b)
    rhs, rhs_t = _dense_operand(rhs), _dense_operand(rhs_t)
    data = data.detach()
    assert data.is_contiguous() and out.stride(1) == 1 and out_t.stride(1) == 1
    assert data.dtype == rhs.dtype == rhs_t.dtype == out.dtype == out_t.dtype
    ci, cit = _index(column_indices), _index(column_indices_t)
    plan = fusion_plan(offsets, column_indices, offsets_t, column_indices_t, blocking=b) if FUSION and b in (64, 128) and data.shape[0] > 0 else None
    with _on_device(out.device):
        _lib.check(_lib.load().stk_dsd_dsd(
            m, k, data.data_ptr(), _offsets(offsets).data_ptr(), ci.data_ptr(),
            _offsets(offsets_t).data_ptr(), cit.data_ptr(), _offsets(block_offsets_t).data_ptr(),
            rhs.shape[1], rhs.data_ptr(), rhs.stride(0), rhs.stride(1), out.data_ptr(), out.stride(0),
            rhs_t.shape[1], rhs_t.data_ptr(), rhs_t.stride(0), rhs_t.stride(1), out_t.data_ptr(), out_t.stride(0),
            data.shape[0], b, _value_dtype(data), _INDEX_DTYPES[ci.dtype], plan.data_ptr() if plan is not None else None, _stream()))


def sdd_dsd(shape, lhs, rhs_sdd, out_sdd, data, offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t,
            transpose_a, rhs_dsd, out_dsd):
    """out_sdd = lhs @ rhs_sdd on the topology [m, n] = `shape` and out_dsd = op(sparse) @ rhs_dsd for the values `data` on the
    same topology, in one launch where the layouts allow it (the two gradients of dsd, stk/backend/sputnik.py:131-155);
    otherwise the two products one after the other.  The results are those of sdd and dsd (without its workspace), bit
    for bit."""
    _need_gpu(data, lhs, rhs_sdd, rhs_dsd, out_sdd, out_dsd)
    m, n = shape
    b = _blocking(data)
    assert lhs.shape[0] == m and rhs_sdd.shape[1] == n and lhs.shape[1] == rhs_sdd.shape[0], "incompatible dimensions"
    assert rhs_dsd.shape[0] == (m if transpose_a else n), "incompatible dimensions"
    _validate_matmul_dims(m, lhs.shape[1], n, b)
    _validate_matmul_dims(n if transpose_a else m, rhs_dsd.shape[0], rhs_dsd.shape[1], b)
    lhs, rhs_sdd, rhs_dsd = _dense_operand(lhs), _dense_operand(rhs_sdd), _dense_operand(rhs_dsd)
    data = data.detach()
    assert data.is_contiguous() and out_sdd.is_contiguous() and out_sdd.shape == data.shape and out_dsd.stride(1) == 1
    assert data.dtype == lhs.dtype == rhs_sdd.dtype == rhs_dsd.dtype == out_sdd.dtype == out_dsd.dtype
    ri, ci, cit = _index(row_indices), _index(column_indices), _index(column_indices_t)
    assert ri.dtype == ci.dtype == cit.dtype
    plan = fusion_plan(offsets, column_indices, offsets_t, column_indices_t, blocking=b) if FUSION and b in (64, 128) and data.shape[0] > 0 else None
    with _on_device(out_dsd.device):
        _lib.check(_lib.load().stk_sdd_dsd(
            m, n, _offsets(offsets).data_ptr(), ri.data_ptr(), ci.data_ptr(),
            _offsets(offsets_t).data_ptr(), cit.data_ptr(), _offsets(block_offsets_t).data_ptr(),
            lhs.data_ptr(), lhs.stride(0), lhs.stride(1), rhs_sdd.data_ptr(), rhs_sdd.stride(0), rhs_sdd.stride(1), lhs.shape[1],
            out_sdd.data_ptr(), data.data_ptr(), 1 if transpose_a else 0, rhs_dsd.shape[1], rhs_dsd.data_ptr(), rhs_dsd.stride(0),
            rhs_dsd.stride(1), out_dsd.data_ptr(), out_dsd.stride(0),
            data.shape[0], b, _value_dtype(data), _INDEX_DTYPES[ci.dtype], plan.data_ptr() if plan is not None else None, _stream()))


def row_indices(shape, data, offsets, column_indices, out):
    """out[offsets[r]:offsets[r+1]] = r for every block row r."""
    if not out.is_cuda:
        return host_kernels.row_indices(shape, data, offsets, column_indices, out)
    _need_gpu(offsets, out)
    assert out.is_contiguous()
    offsets = _offsets(offsets)
    with _on_device(out.device):
        _lib.check(_lib.load().stk_row_indices(
            offsets.data_ptr(), offsets.numel() - 1, out.numel(), out.data_ptr(), _INDEX_DTYPES[out.dtype], _stream()))


def transpose_meta(size, data, row_indices, column_indices, offsets):
    """(column_indices_t, offsets_t, block_offsets_t), stable tie order."""
    _need_gpu(row_indices, column_indices)
    block_cols = size[1] // _blocking(data)
    ri, ci = _index(row_indices), _index(column_indices)
    assert ri.dtype == ci.dtype
    nnz = ci.numel()
    dev = ci.device
    column_indices_t = torch.empty(nnz, dtype=ri.dtype, device=dev)
    offsets_t = torch.empty(block_cols + 1, dtype=torch.int32, device=dev)
    block_offsets_t = torch.empty(nnz, dtype=torch.int32, device=dev)
    lib = _lib.load()
    ws_bytes = lib.stk_transpose_meta_workspace_bytes(nnz)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    with _on_device(dev):
        _lib.check(lib.stk_transpose_meta(
            ri.data_ptr(), ci.data_ptr(), nnz, block_cols, _INDEX_DTYPES[ci.dtype],
            column_indices_t.data_ptr(), offsets_t.data_ptr(), block_offsets_t.data_ptr(),
            ws.data_ptr(), ws_bytes, _stream()))
    return column_indices_t, offsets_t, block_offsets_t


def dmoe_topology(padded_bins, blocking, block_rows, blocks_per_row, index_dtype=torch.int16):
    """(offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t) of the
    block-diagonal dropless-MoE pattern, one launch, no sort.  padded_bins: int32 device tensor,
    inclusive prefix sum of the per-expert row counts (each a multiple of `blocking`)."""
    _need_gpu(padded_bins)
    assert padded_bins.dim() == 1 and padded_bins.numel() > 0
    bins = _offsets(padded_bins)
    dev = bins.device
    experts = bins.numel()
    nnz = block_rows * blocks_per_row
    offsets = torch.empty(block_rows + 1, dtype=torch.int32, device=dev)
    offsets_t = torch.empty(experts * blocks_per_row + 1, dtype=torch.int32, device=dev)
    row_indices = torch.empty(nnz, dtype=index_dtype, device=dev)
    column_indices = torch.empty(nnz, dtype=index_dtype, device=dev)
    column_indices_t = torch.empty(nnz, dtype=index_dtype, device=dev)
    block_offsets_t = torch.empty(nnz, dtype=torch.int32, device=dev)
    with _on_device(dev):
        _lib.check(_lib.load().stk_dmoe_topology(
            bins.data_ptr(), experts, blocking, block_rows, blocks_per_row, _INDEX_DTYPES[index_dtype],
            offsets.data_ptr(), row_indices.data_ptr(), column_indices.data_ptr(),
            offsets_t.data_ptr(), column_indices_t.data_ptr(), block_offsets_t.data_ptr(), _stream()))
    return offsets, row_indices, column_indices, offsets_t, column_indices_t, block_offsets_t


def _elem_bytes(t):
    if t.element_size() not in (2, 4):
        raise NotImplementedError(f"stk_amd: format conversion handles 2- and 4-byte elements, got {t.dtype}")
    return t.element_size()


def to_dense(data, row_indices, column_indices, rows, cols):
    _need_gpu(data)
    data = data.detach().contiguous()
    b = _blocking(data)
    ri, ci = _index(row_indices), _index(column_indices)
    out = torch.empty((rows, cols), dtype=data.dtype, device=data.device)
    with _on_device(data.device):
        _lib.check(_lib.load().stk_to_dense(
            data.data_ptr(), ri.data_ptr(), ci.data_ptr(), data.shape[0], b, rows, cols,
            _elem_bytes(data), _INDEX_DTYPES[ci.dtype], out.data_ptr(), _stream()))
    return out


NNZ_POLL_LIMIT = 20000   # polls of the pinned nnz word (some 2 ms) before to_sparse waits for the stream instead
_nnz_buffers = threading.local()   # per host thread: device index -> pinned int32[1] that stk_to_sparse_count_nnz writes nnz into


_TO_SPARSE_KEEP_BYTES = 1 << 16   # scratch allocations below this size stay alive behind the views returned


def to_sparse(x, blocking, index_dtype=torch.int16):
    """(data, row_indices, column_indices, offsets) of the nonzero blocks of x."""
    _need_gpu(x)
    assert x.dim() == 2
    rows, cols = x.shape
    assert rows % blocking == 0 and cols % blocking == 0
    if x.stride(1) != 1 and cols > 1:
        x = x.contiguous()
    x = x.detach()
    br, bc = rows // blocking, cols // blocking
    dev = x.device
    # one allocation for offsets (int32) and the block mask (bytes) behind it
    scratch = torch.empty(4 * (br + 1) + max(br * bc, 1), dtype=torch.uint8, device=dev)
    offsets, mask = scratch[:4 * (br + 1)].view(torch.int32), scratch[4 * (br + 1):]
    lib = _lib.load()
    with _on_device(dev):
        if _capture_id(dev):
            raise RuntimeError("to_sparse sizes its result by the number of nonzero blocks, which the host reads back: "
                               "it cannot be captured into a graph")
        # nnz arrives in pinned host memory, written by the counting kernel: one wait, no copy to launch
        buffers = _nnz_buffers.__dict__.setdefault("of_device", {})
        nnz_host = buffers.get(dev.index)
        if nnz_host is None:
            nnz_host = buffers[dev.index] = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        word = nnz_host.numpy()
        word[0] = -1
        _lib.check(lib.stk_to_sparse_count_nnz(
            x.data_ptr(), rows, cols, x.stride(0), blocking, _elem_bytes(x), mask.data_ptr(), offsets.data_ptr(), nnz_host.data_ptr(),
            _stream()))
        # the coordinates need no nnz: launched behind the count, into room for every block (the first nnz entries
        # are written; the index tensors returned are views of that room)
        half = (br * bc + 127) // 128 * 128   # (both index arrays start at a multiple of 256 bytes, like allocations of their own)
        room = torch.empty(2 * max(half, 128), dtype=index_dtype, device=dev)
        _lib.check(lib.stk_to_sparse_coordinates(rows, cols, blocking, mask.data_ptr(), offsets.data_ptr(), room.data_ptr(),
                                                 room.data_ptr() + half * room.element_size(), _INDEX_DTYPES[index_dtype], _stream()))
        # the counting kernel's last store is nnz: poll the pinned word instead of sleeping in a stream wait (whose
        # wake-up costs more than the kernels of a small matrix); after a while fall back to the wait, which also
        # reports a launch that failed
        spins = 0
        while word[0] < 0 and spins < NNZ_POLL_LIMIT:
            spins += 1
            if not spins & 1023:
                time.sleep(0)   # let other host threads have the interpreter
        if word[0] < 0:
            torch.cuda.current_stream(dev).synchronize()
            assert word[0] >= 0, "stk_to_sparse_count_nnz did not deliver nnz"
        nnz = int(word[0])
        row_indices, column_indices = room[:nnz], room[half:half + nnz]
        data = torch.empty((nnz, blocking, blocking), dtype=x.dtype, device=dev)
        _lib.check(lib.stk_to_sparse_gather(
            x.data_ptr(), rows, cols, x.stride(0), blocking, _elem_bytes(x), row_indices.data_ptr(), column_indices.data_ptr(), nnz,
            _INDEX_DTYPES[index_dtype], data.data_ptr(), _stream()))
        # A Matrix keeps these tensors for as long as it lives.  Where the room for every block is much more than the
        # nonzero blocks need (a large, very sparse matrix), they are copied out of it, and the offsets out of the
        # allocation they share with the block mask, so that the O(rows x columns / blocking^2) buffers can go.
        if room.numel() * room.element_size() >= _TO_SPARSE_KEEP_BYTES and 4 * nnz <= br * bc:
            row_indices, column_indices = row_indices.clone(), column_indices.clone()
        if scratch.numel() >= _TO_SPARSE_KEEP_BYTES and 4 * 4 * (br + 1) <= scratch.numel():
            offsets = offsets.clone()
    return data, row_indices, column_indices, offsets


# ---------------------------------------------------------------- token routing (no counterpart in the reference)
def _rows16(x):
    """2-D 16-bit tensor whose rows the copy kernels can read in place (unit column stride, rows at
    multiples of 16 bytes); anything else is copied to row-major first."""
    assert x.dim() == 2
    if x.numel() and not (x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.stride(0) >= x.size(1) and x.data_ptr() % 16 == 0):
        x = x.contiguous()
    return x


def _row_stride(x):
    return x.stride(0) if x.numel() and x.size(0) > 1 else max(x.size(1), 1)


def route(top_experts, num_experts, blocking, padded_rows):
    """(indices, bin_ids, bins, padded_bins, slot_rows, row_slots) of stk_route; all int32 on the
    device of top_experts.  padded_rows: rows of the padded layout (length of row_slots)."""
    _need_gpu(top_experts)
    e = top_experts.reshape(-1)
    if e.dtype != torch.int32:
        e = e.to(torch.int32)
    e = e.contiguous()
    dev, slots = e.device, e.numel()
    with _on_device(dev):
        lib = _lib.load()
        ws_bytes = lib.stk_route_workspace_bytes(slots, num_experts)
        # one allocation for the six outputs and the workspace
        parts = torch.empty(3 * slots + 2 * num_experts + padded_rows + (ws_bytes + 3) // 4, dtype=torch.int32, device=dev).split(
            [slots, slots, slots, num_experts, num_experts, padded_rows, (ws_bytes + 3) // 4])
        indices, bin_ids, slot_rows, bins, padded_bins, row_slots, ws = parts
        _lib.check(lib.stk_route(e.data_ptr(), slots, num_experts, blocking, padded_rows, indices.data_ptr(), bin_ids.data_ptr(),
                                 bins.data_ptr(), padded_bins.data_ptr(), slot_rows.data_ptr(), row_slots.data_ptr(),
                                 ws.data_ptr(), ws_bytes, _stream()))
    return indices, bin_ids, bins, padded_bins, slot_rows, row_slots


def _weights32(weights, slots):
    if weights is None:
        return None
    w = weights.detach().reshape(-1).to(torch.float32).contiguous()
    assert w.numel() == slots, f"one weight per slot: {w.numel()} weights for {slots} slots"
    return w


def padded_gather(x, row_slots, top_k, weights=None):
    """out[r] = (weights[s]) * x[s // top_k], s = row_slots[r]; zeros where s < 0."""
    _need_gpu(x, row_slots)
    x = _rows16(x.detach())
    tokens, cols = x.shape
    rows = row_slots.numel()
    w = _weights32(weights, tokens * top_k)
    out = torch.empty((rows, cols), dtype=x.dtype, device=x.device)
    with _on_device(x.device):
        _lib.check(_lib.load().stk_padded_gather(
            x.data_ptr(), tokens, cols, _row_stride(x), row_slots.data_ptr(), None if w is None else w.data_ptr(), top_k, rows,
            out.data_ptr(), max(cols, 1), _value_dtype(x), _stream()))
    return out


def padded_scatter(x, slot_rows, top_k, weights=None):
    """out[t] = sum_k (weights[s]) * x[slot_rows[s]], s = t * top_k + k."""
    _need_gpu(x, slot_rows)
    x = _rows16(x.detach())
    rows, cols = x.shape
    slots = slot_rows.numel()
    assert slots % top_k == 0, f"{slots} slots are not a multiple of top_k = {top_k}"
    tokens = slots // top_k
    w = _weights32(weights, slots)
    out = torch.empty((tokens, cols), dtype=x.dtype, device=x.device)
    with _on_device(x.device):
        _lib.check(_lib.load().stk_padded_scatter(
            x.data_ptr(), rows, cols, _row_stride(x), slot_rows.data_ptr(), None if w is None else w.data_ptr(), top_k, tokens,
            out.data_ptr(), max(cols, 1), _value_dtype(x), _stream()))
    return out


def padded_scatter_weight_gradient(x, grad, slot_rows, top_k):
    """fp32 [slots]: <x[slot_rows[s]], grad[s // top_k]>."""
    _need_gpu(x, grad, slot_rows)
    x, grad = _rows16(x.detach()), _rows16(grad.detach())
    assert x.dtype == grad.dtype and x.size(1) == grad.size(1)
    slots = slot_rows.numel()
    assert grad.size(0) * top_k == slots
    out = torch.empty(slots, dtype=torch.float32, device=x.device)
    with _on_device(x.device):
        _lib.check(_lib.load().stk_padded_scatter_weight_gradient(
            x.data_ptr(), x.size(0), x.size(1), _row_stride(x), grad.data_ptr(), _row_stride(grad), slot_rows.data_ptr(), top_k,
            grad.size(0), out.data_ptr(), _value_dtype(x), _stream()))
    return out


def sdd_gather(x, row_slots, top_k, rhs, shape, out, offsets, row_indices, column_indices, activation=None):
    """out = act(sdd(padded_gather(x, row_slots, top_k), rhs)) on the topology without the padded copy of x
    (stk_sdd_gather); bit-identical to padded_gather followed by sdd_fused.  False, with nothing launched, when
    the library has no such kernel for this case (the caller then makes the two calls); True otherwise."""
    _need_gpu(x, row_slots, rhs, out)
    m, n = shape
    b = _blocking(out)
    nnz = row_indices.numel()
    if b != 128 or activation not in ACTIVATIONS or ACTIVATIONS[activation] > ACTIVATIONS["silu"] or FUSION is False:
        return False
    x = _rows16(x.detach())
    tokens, k = x.shape
    assert k == rhs.shape[0] and n == rhs.shape[1], "incompatible dimensions"
    assert row_slots.dtype == torch.int32 and row_slots.is_contiguous() and row_slots.numel() >= m
    _validate_matmul_dims(m, k, n, b)
    if tokens == 0 or tokens * _row_stride(x) * 2 >= 1 << 32:
        return False
    if nnz == 0:
        return True
    rhs = _dense_operand(rhs)
    assert out.is_contiguous() and x.dtype == rhs.dtype == out.dtype
    ri, ci = _index(row_indices), _index(column_indices)
    plan = fusion_plan(offsets, column_indices, blocking=b) if offsets is not None else None
    with _on_device(out.device):
        status = _lib.load().stk_sdd_gather(
            x.data_ptr(), tokens, _row_stride(x), row_slots.data_ptr(), top_k, rhs.data_ptr(), rhs.stride(0), rhs.stride(1),
            m, k, n, out.data_ptr(), _offsets(offsets).data_ptr() if plan is not None else None, ri.data_ptr(), ci.data_ptr(), nnz,
            b, _value_dtype(out), _INDEX_DTYPES[ri.dtype], plan.data_ptr() if plan is not None else None, ACTIVATIONS[activation], _stream())
    if status == _lib.STK_ERR_UNSUPPORTED:
        return False
    _lib.check(status)
    return True


def dsd_scatter(shape, data, offsets, column_indices, offsets_t, column_indices_t, rhs, row_slots, weights, out):
    """out = padded_scatter(sparse @ rhs, top_k = 1, weights) without the padded result (stk_dsd_scatter): row r of
    the product goes to out[row_slots[r]]; bit-identical to dsd followed by padded_scatter.  False, with nothing
    launched, when the library has no such kernel for this case (the caller then makes the two calls); True otherwise."""
    _need_gpu(data, rhs, row_slots, out)
    m, k = shape
    n = rhs.shape[1]
    b = _blocking(data)
    assert k == rhs.shape[0], "incompatible dimensions"
    _validate_matmul_dims(m, k, n, b)
    tokens = out.shape[0]
    if b != 128 or n % 256 or not FUSION or data.shape[0] == 0 or tokens == 0:
        return False
    rhs = _dense_operand(rhs)
    data = data.detach()
    assert data.is_contiguous() and out.stride(1) == 1 and out.shape[1] == n
    assert data.dtype == rhs.dtype == out.dtype
    assert row_slots.dtype == torch.int32 and row_slots.is_contiguous() and row_slots.numel() >= m
    w = _weights32(weights, tokens)
    ci = _index(column_indices)
    plan = fusion_plan(offsets, column_indices, offsets_t, column_indices_t, blocking=b)
    with _on_device(out.device):
        ws = _dsd_workspace(out.device, m, n, b)
        status = _lib.load().stk_dsd_scatter(
            m, k, n, data.data_ptr(), _offsets(offsets).data_ptr(), ci.data_ptr(), rhs.data_ptr(), rhs.stride(0), rhs.stride(1),
            row_slots.data_ptr(), None if w is None else w.data_ptr(), tokens, out.data_ptr(), out.stride(0),
            data.shape[0], b, _value_dtype(out), _INDEX_DTYPES[ci.dtype], plan.data_ptr(),
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, _stream())
        if status == _lib.STK_ERR_UNSUPPORTED:
            return False
        if status != _lib.STK_OK and ws is not None:
            release_workspaces()
        _lib.check(status)
    return True
