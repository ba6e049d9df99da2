"""CPU oracle for the block-sparse matmul path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain numpy, the algorithms of the reference
(stanford-futuredata/stk 0.7.1) for the blocked-CSR-COO format and the
sdd / dsd / dds products.  It is the checker for the HIP kernels: only the test
suite, the smoke check and the benchmark's CPU-baseline leg may import it.  The
shipped package never does.

Every function cites the reference lines it follows (paths relative to the
reference checkout).  How each function is pinned (see tests/test_oracle.py):

  dense_mask        same numpy legacy-RNG call sequence + known-answer block mask
  to_sparse         known-answer vector, round trip, nnz count, row-major order
  to_dense          round trip against plain numpy block placement
  transpose_meta    known-answer vector, scipy CSR->CSC, permutation invariants
  row_indices       known-answer vector, np.repeat closed form
  sdd / dsd / dds   dense-masked float64 matmul (an independent formulation),
                    brute-force triple loops on tiny inputs, linearity
  activation /      torch.nn.functional.{relu, gelu, silu} (library routines written
  sdd_fused         independently), special values and limits; the composition itself is
                    activation(sdd) * multiplier on the pinned sdd
  dmoe_topology     to_sparse of the explicit block-diagonal dense pattern
  route             hand-worked vector, a slot-by-slot Python walk, sortedness and inverse
                    invariants (no reference code exists for it: the reference's callers do
                    this step; the definition is the one in include/stk_amd.h)
  padded_gather /   the same walk slot by slot on tiny inputs, gather -> scatter round
  padded_scatter    trip, hand-worked rounding cases (the order of the fp32 operations is
                    part of the definition, so the GPU result is compared bit for bit)

Tie order: the reference sorts block columns with a non-stable argsort
(stk/matrix.py:110), so the order of equal keys is implementation defined
there.  The canonical order used here is the stable one (ascending block id
inside each block column), which is what a CSR->CSC conversion yields.
"""
from collections import namedtuple
import math

import numpy as np

Topology = namedtuple(
    "Topology",
    "shape blocking row_indices column_indices offsets "
    "column_indices_t offsets_t block_offsets_t")


# --------------------------------------------------------------------------
# random block masks                       stk/random/random_ops.py:6-22
# --------------------------------------------------------------------------
def dense_mask(rows, cols, sparsity, blocking=1):
    """0/1 float32 matrix with round(nblocks * (1 - sparsity)) nonzero blocks.

    Follows stk/random/random_ops.py:6-22.  Draws from numpy's global legacy
    RNG with the same single call (np.random.choice without replacement), so
    np.random.seed(s) reproduces the reference's mask.
    """
    assert 0.0 <= sparsity <= 1.0
    assert rows % blocking == 0 and cols % blocking == 0
    br, bc = rows // blocking, cols // blocking
    keep = round(br * bc * (1 - sparsity))
    blocks = np.ones(br * bc)
    dropped = np.random.choice(blocks.size, blocks.size - keep, replace=False)
    blocks[dropped] = 0.0
    grid = blocks.reshape(br, bc)
    return np.kron(grid, np.ones((blocking, blocking))).astype(np.float32)


# --------------------------------------------------------------------------
# format conversion                        stk/ops/matrix_ops.py:36-85
# --------------------------------------------------------------------------
def block_mask(x, blocking):
    """Boolean [block_rows, block_cols]: block has a nonzero |x| sum.

    Follows stk/ops/matrix_ops.py:50-59 (sum of abs != 0).  A sum of absolute
    values is nonzero exactly when some element is not +-0 (NaN counts as
    nonzero because NaN != 0), so the test is done element-wise.
    """
    r, c = x.shape
    assert r % blocking == 0 and c % blocking == 0
    v = x.reshape(r // blocking, blocking, c // blocking, blocking)
    return np.logical_not(v == 0).any(axis=(1, 3))


def transpose_meta(shape, blocking, row_indices, column_indices):
    """(column_indices_t, offsets_t, block_offsets_t) for a blocked-CSR matrix.

    Follows stk/matrix.py:105-123 with the stable tie order: argsort of the
    block columns, gather of the block rows through it, a histogram of the
    block columns and its exclusive prefix sum.
    """
    block_cols = shape[1] // blocking
    order = np.argsort(np.asarray(column_indices).astype(np.int64), kind="stable")
    column_indices_t = np.asarray(row_indices)[order].astype(np.asarray(row_indices).dtype)
    block_offsets_t = order.astype(np.int32)
    per_col = np.bincount(np.asarray(column_indices).astype(np.int64), minlength=block_cols)
    offsets_t = np.concatenate([[0], np.cumsum(per_col)]).astype(np.int32)
    return column_indices_t, offsets_t, block_offsets_t


def to_sparse(x, blocking=1, index_dtype=np.int16):
    """Dense 2-D array -> (data [nnz, b, b], Topology).

    Follows stk/ops/matrix_ops.py:64-85: block mask, per-row counts scanned into
    int32 offsets, nonzero block coordinates in row-major order as int16, block
    contents gathered in that order, then transpose metadata (stk/matrix.py:150-157).
    """
    m = block_mask(x, blocking)
    offsets = np.concatenate([[0], np.cumsum(m.sum(axis=1))]).astype(np.int32)
    rows, cols = np.nonzero(m)  # row-major order, as torch.nonzero
    r, c = x.shape
    v = x.reshape(r // blocking, blocking, c // blocking, blocking).transpose(0, 2, 1, 3)
    data = np.ascontiguousarray(v[rows, cols]).reshape(-1, blocking, blocking)
    rows = rows.astype(index_dtype)
    cols = cols.astype(index_dtype)
    ct, ot, bt = transpose_meta(x.shape, blocking, rows, cols)
    return data, Topology(tuple(x.shape), blocking, rows, cols, offsets, ct, ot, bt)


def to_dense(shape, data, row_indices, column_indices):
    """Blocked -> dense with zeros elsewhere.  Follows stk/ops/matrix_ops.py:36-47
    (leading dimensions of `shape` are flattened into rows, :39)."""
    b = data.shape[-1]
    rows = int(np.prod(shape[:-1]))
    out = np.zeros((rows, shape[-1]), dtype=data.dtype)
    for p in range(data.shape[0]):
        i, j = int(row_indices[p]), int(column_indices[p])
        out[i * b:(i + 1) * b, j * b:(j + 1) * b] = data[p]
    return out.reshape(shape)


def row_indices(offsets, dtype=np.int16):
    """COO block-row index from CSR offsets.

    Follows stk/backend/triton_kernels.py:381-393: program `pid` stores `pid`
    into out[offsets[pid] : offsets[pid + 1]].
    """
    offsets = np.asarray(offsets)
    out = np.empty(int(offsets[-1]), dtype=dtype)
    for pid in range(len(offsets) - 1):
        for k in range(int(offsets[pid]), int(offsets[pid + 1])):
            out[k] = pid
    return out


# --------------------------------------------------------------------------
# products                                 stk/backend/triton_kernels.py
# --------------------------------------------------------------------------
def _f32(x):
    return np.asarray(x, dtype=np.float32)


def sdd(lhs, rhs, topo):
    """Sampled dense x dense: out[p] = lhs[r_p rows, :] @ rhs[:, c_p cols].

    Follows stk/backend/triton_kernels.py:34-68 (program p reads
    row_indices[p], column_indices[p], contracts over all of K with fp32
    accumulation, stores block p) and :332-379 (the inner-dimension assert).
    Returns float32 [nnz, b, b].
    """
    lhs, rhs = _f32(lhs), _f32(rhs)
    assert lhs.shape[1] == rhs.shape[0], "incompatible dimensions"
    b = topo.blocking
    nnz = len(topo.row_indices)
    out = np.empty((nnz, b, b), dtype=np.float32)
    for p in range(nnz):
        i, j = int(topo.row_indices[p]), int(topo.column_indices[p])
        out[p] = lhs[i * b:(i + 1) * b, :] @ rhs[:, j * b:(j + 1) * b]
    return out


_erf = np.vectorize(math.erf, otypes=[np.float64])


def activation(x, kind):
    """The activations a caller applies to the values of an sdd result, in float64:
    relu, gelu (0.5 x (1 + erf(x / sqrt 2))), gelu_tanh (0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))),
    the approximation MoE layers on top of stk.ops.sdd use by default), silu (x sigmoid(x)); None: identity."""
    x = np.asarray(x, dtype=np.float64)
    if kind in (None, "none"):
        return x
    if kind == "relu":
        return np.maximum(x, 0.0)
    if kind == "gelu":
        return 0.5 * x * (1.0 + _erf(x / math.sqrt(2.0)))
    if kind == "gelu_tanh":
        return 0.5 * x * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))
    if kind == "silu":
        return x / (1.0 + np.exp(-x))
    # the derivatives of the four (what a backward pass multiplies the incoming gradient with)
    if kind == "relu_grad":
        return (x > 0.0).astype(np.float64)
    if kind == "gelu_grad":
        return 0.5 * (1.0 + _erf(x / math.sqrt(2.0))) + x * np.exp(-0.5 * x * x) / math.sqrt(2.0 * math.pi)
    if kind == "gelu_tanh_grad":
        c = math.sqrt(2.0 / math.pi)
        t = np.tanh(c * (x + 0.044715 * x ** 3))
        return 0.5 * (1.0 + t) + 0.5 * x * (1.0 - t * t) * c * (1.0 + 3.0 * 0.044715 * x * x)
    if kind == "silu_grad":
        sg = 1.0 / (1.0 + np.exp(-x))
        return sg * (1.0 + x * (1.0 - sg))
    raise ValueError(kind)


def sdd_fused(lhs, rhs, topo, kind=None, multiplier=None):
    """activation(sdd(lhs, rhs, topo)) * multiplier: stk.ops.sdd (stk/ops/linear_ops.py:37-59) followed by an
    activation on the values and by stk.ops.mul (stk/ops/eltwise_ops.py:3-28: a.data * b.data on the shared
    topology).  Without intermediate rounding; float32 [nnz, b, b]."""
    out = activation(sdd(lhs, rhs, topo), kind)
    if multiplier is not None:
        assert multiplier.shape == out.shape
        out = out * np.asarray(multiplier, dtype=np.float64)
    return out.astype(np.float32)


def dsd(shape, data, topo, transpose_a, rhs):
    """op(sparse) x dense -> dense [shape[0], N], float32.

    `shape` is the logical (already transposed) size of the sparse operand.
    Follows stk/backend/triton_kernels.py:83-145 and :222-276.  Output block
    row m walks offsets[m]..offsets[m+1]; entry i uses block i and the rhs
    row panel column_indices[i].  With transpose_a the walk uses offsets_t /
    column_indices_t, the block id comes from block_offsets_t[i] and the block
    is read transposed (:128-133, :260-262).  Rows with no block are zero.
    """
    data, rhs = _f32(data), _f32(rhs)
    assert shape[1] == rhs.shape[0], "incompatible dimensions"
    b = topo.blocking
    out = np.zeros((shape[0], rhs.shape[1]), dtype=np.float32)
    offs, cols = (topo.offsets_t, topo.column_indices_t) if transpose_a else (topo.offsets, topo.column_indices)
    for m in range(shape[0] // b):
        acc = np.zeros((b, rhs.shape[1]), dtype=np.float32)
        for i in range(int(offs[m]), int(offs[m + 1])):
            blk = data[int(topo.block_offsets_t[i])].T if transpose_a else data[i]
            k = int(cols[i])
            acc += blk @ rhs[k * b:(k + 1) * b, :]
        out[m * b:(m + 1) * b] = acc
    return out


def dds(lhs, shape, data, topo, transpose_b):
    """dense x op(sparse) -> dense [M, shape[1]], float32.

    Follows stk/backend/triton_kernels.py:160-220 and :278-330.  Output block
    column n of a non-transposed sparse operand walks offsets_t[n].. with the
    block id from block_offsets_t[i] and the lhs column panel
    column_indices_t[i] (:209-211, :310-311); with transpose_b it walks
    offsets / column_indices with direct block ids and reads the block
    transposed (:206-207, :318-320).
    """
    lhs, data = _f32(lhs), _f32(data)
    assert lhs.shape[1] == shape[0], "incompatible dimensions"
    b = topo.blocking
    out = np.zeros((lhs.shape[0], shape[1]), dtype=np.float32)
    offs, cols = (topo.offsets, topo.column_indices) if transpose_b else (topo.offsets_t, topo.column_indices_t)
    for n in range(shape[1] // b):
        acc = np.zeros((lhs.shape[0], b), dtype=np.float32)
        for i in range(int(offs[n]), int(offs[n + 1])):
            blk = data[i].T if transpose_b else data[int(topo.block_offsets_t[i])]
            k = int(cols[i])
            acc += lhs[:, k * b:(k + 1) * b] @ blk
        out[:, n * b:(n + 1) * b] = acc
    return out


# --------------------------------------------------------------------------
# dense-equivalent path: the reference tests' comparator
#                                          stk/ops/linear_ops_test.py:83-96
# --------------------------------------------------------------------------
def dense_masked_sdd(lhs, rhs, topo):
    """to_dense(ones_like(topo)) * (lhs @ rhs), returned in blocked form."""
    b = topo.blocking
    ones = np.ones((len(topo.row_indices), b, b), dtype=np.float32)
    mask = to_dense(topo.shape, ones, topo.row_indices, topo.column_indices)
    full = (_f32(lhs) @ _f32(rhs)) * mask
    v = full.reshape(topo.shape[0] // b, b, topo.shape[1] // b, b).transpose(0, 2, 1, 3)
    return np.ascontiguousarray(v[topo.row_indices.astype(np.int64), topo.column_indices.astype(np.int64)])


def dense_equiv_dsd(data, topo, transpose_a, rhs):
    a = to_dense(topo.shape, _f32(data), topo.row_indices, topo.column_indices)
    return (a.T if transpose_a else a) @ _f32(rhs)


def dense_equiv_dds(lhs, data, topo, transpose_b):
    s = to_dense(topo.shape, _f32(data), topo.row_indices, topo.column_indices)
    return _f32(lhs) @ (s.T if transpose_b else s)


# --------------------------------------------------------------------------
# dropless-MoE block-diagonal topology (closed form; the reference has no
# builder, its callers construct this with stk.ops.row_indices and
# stk.Matrix(..., column_indices_t=...), stk/matrix.py:134-157)
# --------------------------------------------------------------------------
def dmoe_topology(tokens_per_expert, ffn, blocking, index_dtype=np.int16):
    """Topology of the [padded_tokens, experts * ffn] block-diagonal matrix.

    Expert e owns ceil(t_e / b) block rows and the ffn / b block columns
    starting at e * ffn / b.  Experts without tokens own no rows and their
    columns are empty.
    """
    t = np.asarray(tokens_per_expert, dtype=np.int64)
    b = blocking
    w = ffn // b
    rows_e = (t + b - 1) // b
    nrows = int(rows_e.sum())
    expert_of_row = np.repeat(np.arange(len(t)), rows_e)
    ri = np.repeat(np.arange(nrows), w).astype(index_dtype)
    ci = (expert_of_row[:, None] * w + np.arange(w)[None, :]).reshape(-1).astype(index_dtype)
    offsets = (np.arange(nrows + 1) * w).astype(np.int32)
    shape = (nrows * b, len(t) * ffn)
    ct, ot, bt = transpose_meta(shape, b, ri, ci)
    return Topology(shape, b, ri, ci, offsets, ct, ot, bt)


def padded_tokens_per_expert(tokens_per_expert, blocking):
    t = np.asarray(tokens_per_expert, dtype=np.int64)
    return (t + blocking - 1) // blocking * blocking


# --------------------------------------------------------------------------
# token routing around the dMoE products.  The reference has no code for this
# step (its callers sort the expert choices, pad the bins and copy the rows
# before they build stk.Matrix, stk/matrix.py:134-157); the definition is the
# one given with stk_route / stk_padded_gather / stk_padded_scatter in
# include/stk_amd.h.
# --------------------------------------------------------------------------
Route = namedtuple("Route", "indices bin_ids bins padded_bins slot_rows row_slots")


def route(top_experts, num_experts, blocking, padded_rows=None):
    """Stable sort of the slots by expert and their rows in the padded layout."""
    e = np.clip(np.asarray(top_experts, dtype=np.int64).reshape(-1), 0, num_experts - 1)
    indices = np.argsort(e, kind="stable")
    counts = np.bincount(e, minlength=num_experts)
    bins = np.cumsum(counts)
    padded_bins = np.cumsum((counts + blocking - 1) // blocking * blocking)
    first = bins - counts
    padded_first = np.concatenate([[0], padded_bins[:-1]])
    bin_ids = e[indices]
    rows_sorted = np.arange(e.size) - first[bin_ids] + padded_first[bin_ids]
    slot_rows = np.empty(e.size, dtype=np.int64)
    slot_rows[indices] = rows_sorted
    if padded_rows is None:
        padded_rows = int(padded_bins[-1])
    row_slots = np.full(padded_rows, -1, dtype=np.int64)
    inside = slot_rows < padded_rows
    row_slots[slot_rows[inside]] = np.nonzero(inside)[0]
    i32 = lambda a: a.astype(np.int32)
    return Route(i32(indices), i32(bin_ids), i32(bins), i32(padded_bins), i32(slot_rows), i32(row_slots))


def padded_gather(x, row_slots, top_k, weights=None):
    """float32 [padded_rows, cols]: row r = (weights[s] *) x[s // top_k], s = row_slots[r]; zeros for s < 0.
    The caller rounds to the 16-bit type."""
    x = _f32(x)
    s = np.asarray(row_slots, dtype=np.int64)
    out = np.zeros((s.size, x.shape[1]), dtype=np.float32)
    held = s >= 0
    rows = x[s[held] // top_k]
    if weights is not None:
        rows = np.asarray(weights, dtype=np.float32)[s[held]][:, None] * rows
    out[held] = rows
    return out


def padded_scatter(x, slot_rows, top_k, weights=None):
    """float32 [tokens, cols]: row t = sum over choice (in order) of (weights[s] *) x[slot_rows[s]],
    s = t * top_k + choice; every product and every sum rounded to fp32 on its own, the sum starting
    from the first product.  The caller rounds to the 16-bit type."""
    x = _f32(x)
    r = np.asarray(slot_rows, dtype=np.int64).reshape(-1, top_k)
    w = None if weights is None else np.asarray(weights, dtype=np.float32).reshape(-1, top_k)
    out = None
    for k in range(top_k):
        term = x[r[:, k]]
        if w is not None:
            term = w[:, k][:, None] * term
        out = term.copy() if out is None else out + term
    return out.astype(np.float32)


def padded_scatter_weight_gradient(x, grad, slot_rows, top_k):
    """float64 [slots]: <x[slot_rows[s]], grad[s // top_k]>."""
    x, grad = np.asarray(_f32(x), dtype=np.float64), np.asarray(_f32(grad), dtype=np.float64)
    r = np.asarray(slot_rows, dtype=np.int64)
    return np.einsum("sc,sc->s", x[r], grad[np.arange(r.size) // top_k])
