"""Pins the CPU oracle (oracle/stk_oracle.py) before anything is checked against it.

Each check is independent of the oracle's own formulas: committed known-answer
vectors (made with numpy/scipy only), scipy's CSR->CSC conversion, brute-force
loops on tiny inputs, float64 dense-masked products, closed forms and
invariants.  The parameter grids are those of the reference's tests
(stk/ops/matrix_ops_test.py:8-23, stk/random/random_ops_test.py:8-23,
stk/ops/linear_ops_test.py:21-43).
"""
import itertools
import json
import os

import numpy as np
import pytest
import scipy.sparse as sp

from oracle import stk_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")

# The known-answer vector for np.random.seed(0); mask(1024, 1024, 0.5, 128), typed in by hand from a
# derivation made with numpy and scipy alone (a second, independent source next to the fixture).
KAT = {
    "row_indices": [0,0,0,0,0,1,1,1,1,1,2,2,2,2,2,2,3,3,4,4,4,4,5,5,6,6,6,6,6,7,7,7],
    "column_indices": [0,1,3,5,6,0,1,4,5,7,0,1,3,4,5,7,0,1,4,5,6,7,4,7,0,1,2,3,5,0,1,3],
    "offsets": [0,5,10,16,18,22,24,29,32],
    "offsets_t": [0,6,12,13,17,21,26,28,32],
    "column_indices_t": [0,1,2,3,6,7,0,1,2,3,6,7,6,0,2,6,7,1,2,4,5,0,1,2,4,6,0,4,1,2,4,5],
    "block_offsets_t": [0,5,10,16,24,29,1,6,11,17,25,30,26,2,12,27,31,7,13,18,22,3,8,14,19,28,4,20,9,15,21,23],
}

FORMAT_CASES = [
    (8, 16, 0.0, 1), (8, 16, 0.5, 1), (8, 16, .95, 1), (16, 8, 0.0, 1), (16, 8, 0.5, 1), (16, 8, .95, 1),
    (8, 16, 0.0, 8), (8, 16, 0.5, 8), (8, 16, 1.0, 8), (16, 8, 0.0, 8), (16, 8, 0.5, 8), (16, 8, 1.0, 8),
    (128, 256, 0.5, 16), (256, 128, 0.75, 32), (512, 512, .875, 128),
]


def _topo_fields(t):
    return {k: np.asarray(getattr(t, k)).tolist() for k in KAT}


def test_config1_known_answer():
    fixture = json.load(open(os.path.join(GOLDEN, "config1_topology.json")))
    np.random.seed(0)
    mask = O.dense_mask(1024, 1024, 0.5, 128)
    assert mask.dtype == np.float32 and mask.shape == (1024, 1024)
    assert (mask[::128, ::128] != 0).astype(int).tolist() == fixture["mask"]
    data, topo = O.to_sparse(mask.astype(np.float16), 128)
    got = _topo_fields(topo)
    for k in KAT:
        assert got[k] == KAT[k], k
        assert got[k] == fixture[k], k
    assert data.shape == (32, 128, 128) and (data == 1).all()
    assert topo.row_indices.dtype == np.int16 and topo.column_indices.dtype == np.int16
    assert topo.offsets.dtype == np.int32 and topo.offsets_t.dtype == np.int32
    assert topo.block_offsets_t.dtype == np.int32 and topo.column_indices_t.dtype == np.int16


def test_random_topology_fixtures():
    for fx in json.load(open(os.path.join(GOLDEN, "random_topologies.json"))):
        mask = np.asarray(fx["mask"], dtype=np.float32)
        b = 4
        x = np.kron(mask, np.ones((b, b), dtype=np.float32))
        _, topo = O.to_sparse(x, b)
        got = _topo_fields(topo)
        for k in KAT:
            assert got[k] == fx[k], (fx["seed"], k)
        assert O.row_indices(topo.offsets).tolist() == fx["row_indices"]


@pytest.mark.parametrize("rows,cols,sparsity,blocking", FORMAT_CASES)
def test_dense_mask_properties(rows, cols, sparsity, blocking):
    # stk/random/random_ops_test.py:26-46
    np.random.seed(rows + cols)
    m = O.dense_mask(rows, cols, sparsity, blocking)
    assert m.shape == (rows, cols)
    nnz = round(rows // blocking * cols // blocking * (1 - sparsity)) * blocking ** 2
    assert np.count_nonzero(m) == nnz
    assert np.logical_or(m == 0, m == 1).all()
    # blocks are all-or-nothing
    v = m.reshape(rows // blocking, blocking, cols // blocking, blocking)
    assert (v.min(axis=(1, 3)) == v.max(axis=(1, 3))).all()


@pytest.mark.parametrize("rows,cols,sparsity,blocking", FORMAT_CASES)
def test_format_round_trip(rows, cols, sparsity, blocking):
    # stk/ops/matrix_ops_test.py:26-58
    rng = np.random.RandomState(7)
    np.random.seed(11)
    x = (rng.randn(rows, cols) * O.dense_mask(rows, cols, sparsity, blocking)).astype(np.float16)
    data, topo = O.to_sparse(x, blocking)
    nblocks = round(rows // blocking * cols // blocking * (1 - sparsity))
    assert data.size == nblocks * blocking ** 2
    assert len(topo.offsets) == rows // blocking + 1 and topo.offsets[-1] == nblocks
    # row-major nonzero order
    lin = topo.row_indices.astype(np.int64) * (cols // blocking) + topo.column_indices
    assert (np.diff(lin) > 0).all()
    dense = O.to_dense(topo.shape, data, topo.row_indices, topo.column_indices)
    assert dense.dtype == x.dtype and np.array_equal(dense, x)
    assert np.count_nonzero(dense) == np.count_nonzero(x)
    assert np.array_equal(O.row_indices(topo.offsets), topo.row_indices)


def test_block_mask_counts_nan_and_negative_zero():
    x = np.zeros((4, 6), dtype=np.float32)
    x[0, 0] = -0.0          # still a zero block
    x[2, 2] = np.nan        # NaN != 0 -> nonzero block
    x[3, 5] = -1e-30
    m = O.block_mask(x, 2)
    assert m.tolist() == [[False, False, False], [False, True, True]]


@pytest.mark.parametrize("seed", range(6))
def test_transpose_meta_vs_scipy_and_invariants(seed):
    rng = np.random.RandomState(seed)
    br, bc = rng.randint(1, 60), rng.randint(1, 60)
    mask = rng.rand(br, bc) < rng.choice([0.05, 0.3, 0.9])
    rows, cols = np.nonzero(mask)
    nnz = len(rows)
    ct, ot, bt = O.transpose_meta((br * 2, bc * 2), 2, rows.astype(np.int16), cols.astype(np.int16))
    offsets = np.concatenate([[0], np.cumsum(mask.sum(1))])
    csc = sp.csr_matrix((np.arange(1, nnz + 1), cols, offsets), shape=(br, bc)).tocsc()
    csc.sort_indices()
    assert ot.tolist() == csc.indptr.tolist()
    assert ct.tolist() == csc.indices.tolist()
    assert bt.tolist() == (csc.data - 1).tolist()
    # invariants
    assert sorted(bt.tolist()) == list(range(nnz))
    assert np.array_equal(rows[bt], ct)
    for c in range(bc):
        seg = bt[ot[c]:ot[c + 1]]
        assert (cols[seg] == c).all() and (np.diff(seg) > 0).all()


def test_transpose_meta_ties_are_stable_for_unsorted_rows():
    # columns not sorted inside a row and a duplicated coordinate: order must still be ascending block id
    rows = np.array([0, 0, 0, 1, 1, 1], dtype=np.int16)
    cols = np.array([2, 0, 2, 2, 1, 0], dtype=np.int16)
    ct, ot, bt = O.transpose_meta((4, 6), 2, rows, cols)
    assert bt.tolist() == [1, 5, 4, 0, 2, 3]
    assert ct.tolist() == [0, 1, 1, 0, 0, 1]
    assert ot.tolist() == [0, 2, 3, 6]


def test_row_indices_closed_form():
    offsets = np.array([0, 3, 3, 4, 9, 9], dtype=np.int32)
    assert O.row_indices(offsets).tolist() == np.repeat(np.arange(5), np.diff(offsets)).tolist()
    assert O.row_indices(np.array([0, 0, 0], dtype=np.int32)).tolist() == []


# ---------------------------------------------------------------- products
def _brute_mm(a, b):
    m, k = a.shape
    n = b.shape[1]
    out = np.zeros((m, n))
    for i in range(m):
        for j in range(n):
            s = 0.0
            for kk in range(k):
                s += float(a[i, kk]) * float(b[kk, j])
            out[i, j] = s
    return out


def _random_sparse(rng, rows, cols, sparsity, b):
    np.random.seed(rng.randint(1 << 30))
    x = (rng.randn(rows, cols) * O.dense_mask(rows, cols, sparsity, b)).astype(np.float32)
    data, topo = O.to_sparse(x, b)
    return x, data, topo


@pytest.mark.parametrize("trans", [False, True])
def test_products_brute_force_tiny(trans):
    rng = np.random.RandomState(3)
    b = 2
    # sparse operand logical shape [6, 8] (stored [8, 6] when transposed)
    stored = (8, 6) if trans else (6, 8)
    x, data, topo = _random_sparse(rng, *stored, 0.5, b)
    logical = x.T if trans else x
    rhs = rng.randn(8, 4).astype(np.float32)
    got = O.dsd(logical.shape, data, topo, trans, rhs)
    assert np.allclose(got, _brute_mm(logical, rhs), atol=1e-5)
    lhs = rng.randn(4, 6).astype(np.float32)
    got = O.dds(lhs, logical.shape, data, topo, trans)
    assert np.allclose(got, _brute_mm(lhs, logical), atol=1e-5)
    if not trans:
        a = rng.randn(6, 5).astype(np.float32)
        c = rng.randn(5, 8).astype(np.float32)
        full = _brute_mm(a, c)
        got = O.sdd(a, c, topo)
        for p in range(len(topo.row_indices)):
            i, j = topo.row_indices[p], topo.column_indices[p]
            assert np.allclose(got[p], full[i * b:(i + 1) * b, j * b:(j + 1) * b], atol=1e-5)


_SIZES = [(128, 128, 128, 0.0), (256, 256, 256, 0.5), (512, 256, 128, 0.8), (256, 128, 384, 0.75)]


@pytest.mark.parametrize("size,trans_a,trans_b,b", [
    (s, ta, tb, b) for s, (ta, tb), b in itertools.product(_SIZES, [(False, False), (False, True), (True, False), (True, True)], [32, 64])])
def test_products_vs_dense_float64(size, trans_a, trans_b, b):
    # same comparator as stk/ops/linear_ops_test.py:83-96,110-111,147-148: dense mm on the dense copy
    m, k, n, sparsity = size
    rng = np.random.RandomState(m + k + n + 2 * trans_a + trans_b)
    # dsd: sparse lhs, transposed sparse operand expressed through the flag
    stored = (k, m) if trans_a else (m, k)
    x, data, topo = _random_sparse(rng, *stored, sparsity, b)
    a64 = (x.T if trans_a else x).astype(np.float64)
    bmat = rng.randn(*((n, k) if trans_b else (k, n))).astype(np.float32)
    rhs = bmat.T if trans_b else bmat
    got = O.dsd(a64.shape, data, topo, trans_a, rhs)
    assert np.allclose(got, a64 @ rhs.astype(np.float64), rtol=1e-4, atol=1e-3)
    assert np.allclose(got, O.dense_equiv_dsd(data, topo, trans_a, rhs), rtol=1e-4, atol=1e-3)
    # dds: sparse rhs
    stored = (n, k) if trans_b else (k, n)
    x, data, topo = _random_sparse(rng, *stored, sparsity, b)
    b64 = (x.T if trans_b else x).astype(np.float64)
    amat = rng.randn(*((k, m) if trans_a else (m, k))).astype(np.float32)
    lhs = amat.T if trans_a else amat
    got = O.dds(lhs, b64.shape, data, topo, trans_b)
    assert np.allclose(got, lhs.astype(np.float64) @ b64, rtol=1e-4, atol=1e-3)
    assert np.allclose(got, O.dense_equiv_dds(lhs, data, topo, trans_b), rtol=1e-4, atol=1e-3)
    # sdd: dense operands as strided views
    _, _, topo = _random_sparse(rng, m, n, sparsity, b)
    got = O.sdd(lhs, rhs, topo)
    full = lhs.astype(np.float64) @ rhs.astype(np.float64)
    v = full.reshape(m // b, b, n // b, b).transpose(0, 2, 1, 3)
    want = v[topo.row_indices.astype(int), topo.column_indices.astype(int)]
    assert got.shape == want.shape
    assert np.allclose(got, want, rtol=1e-4, atol=1e-3)
    assert np.allclose(got, O.dense_masked_sdd(lhs, rhs, topo), rtol=1e-4, atol=1e-3)


def test_products_linearity_and_empty_rows():
    rng = np.random.RandomState(5)
    b = 16
    x, data, topo = _random_sparse(rng, 64, 96, 0.9, b)   # several empty block rows / columns
    r1, r2 = rng.randn(96, 32).astype(np.float32), rng.randn(96, 32).astype(np.float32)
    y = O.dsd(x.shape, data, topo, False, r1 + 2 * r2)
    assert np.allclose(y, O.dsd(x.shape, data, topo, False, r1) + 2 * O.dsd(x.shape, data, topo, False, r2), atol=1e-3)
    empty_rows = np.diff(topo.offsets) == 0
    assert empty_rows.any()
    for i in np.nonzero(empty_rows)[0]:
        assert (y[i * b:(i + 1) * b] == 0).all()
    # fully empty matrix
    _, data0, topo0 = _random_sparse(rng, 32, 32, 1.0, b)
    assert data0.shape[0] == 0
    assert (O.dsd((32, 32), data0, topo0, False, r1[:32]) == 0).all()
    assert (O.dds(r1.T[:, :32], (32, 32), data0, topo0, False) == 0).all()
    assert O.sdd(r1[:32, :8], r1.T[:8, :32], topo0).shape == (0, b, b)


def test_activations_against_torch_and_special_values():
    import torch
    import torch.nn.functional as F
    x = np.concatenate([np.linspace(-12, 12, 4801), [0.0, -0.0, 1e-8, -1e-8, 30.0, -30.0]])
    t = torch.from_numpy(x)
    for kind, fn in (("relu", F.relu), ("gelu", F.gelu), ("gelu_tanh", lambda v: F.gelu(v, approximate="tanh")), ("silu", F.silu)):
        assert np.allclose(O.activation(x, kind), fn(t).numpy(), rtol=1e-12, atol=1e-14), kind
        assert O.activation(np.zeros(3), kind).tolist() == [0.0, 0.0, 0.0]
        # identity for large positive arguments, zero for large negative ones
        assert np.allclose(O.activation(np.array([40.0, -40.0]), kind), [40.0, 0.0], atol=1e-12)
    assert np.array_equal(O.activation(x, None), x)
    # a dropped factor or a swapped constant shows at x = 1: gelu(1) = Phi(1), silu(1) = 1 / (1 + 1/e)
    assert abs(O.activation(1.0, "gelu") - 0.8413447460685429) < 1e-12
    assert abs(O.activation(1.0, "silu") - 0.7310585786300049) < 1e-12
    assert abs(O.activation(1.0, "gelu_tanh") - 0.8411919906082768) < 1e-9
    with pytest.raises(ValueError):
        O.activation(x, "swish")


def test_activation_derivatives_against_torch_autograd_and_differences():
    import torch
    import torch.nn.functional as F
    x = np.concatenate([np.linspace(-12, 12, 4801), [1e-8, -1e-8, 30.0, -30.0]])
    for kind, fn in (("relu", F.relu), ("gelu", F.gelu), ("gelu_tanh", lambda v: F.gelu(v, approximate="tanh")), ("silu", F.silu)):
        pts = x[x != 0.0] if kind == "relu" else x        # (relu'(0): torch says 0, and so does the oracle; checked below)
        t = torch.from_numpy(pts).requires_grad_(True)
        fn(t).sum().backward()
        got = O.activation(pts, kind + "_grad")
        assert np.allclose(got, t.grad.numpy(), rtol=1e-10, atol=1e-12), kind
        # central differences of the oracle's own function: a derivative of some other function would not match
        inner = pts[(np.abs(pts) > 1e-3) & (np.abs(pts) < 11)]
        h = 1e-6
        diff = (O.activation(inner + h, kind) - O.activation(inner - h, kind)) / (2 * h)
        assert np.allclose(O.activation(inner, kind + "_grad"), diff, rtol=1e-6, atol=1e-8), kind
        # one for large positive arguments, zero for large negative ones
        assert np.allclose(O.activation(np.array([40.0, -40.0]), kind + "_grad"), [1.0, 0.0], atol=1e-12)
    assert O.activation(np.zeros(1), "relu_grad").tolist() == [0.0]
    assert abs(O.activation(0.0, "gelu_grad") - 0.5) < 1e-15 and abs(O.activation(0.0, "silu_grad") - 0.5) < 1e-15
    assert abs(O.activation(0.0, "gelu_tanh_grad") - 0.5) < 1e-15


def test_sdd_fused_is_the_composition_of_its_parts():
    rng = np.random.RandomState(11)
    b = 16
    _, data, topo = _random_sparse(rng, 64, 96, 0.6, b)
    lhs, rhs = rng.randn(64, 40).astype(np.float32), rng.randn(40, 96).astype(np.float32)
    mult = rng.randn(*data.shape).astype(np.float32)
    plain = O.sdd(lhs, rhs, topo)
    assert np.array_equal(O.sdd_fused(lhs, rhs, topo), plain)
    assert np.allclose(O.sdd_fused(lhs, rhs, topo, "relu"), np.maximum(plain, 0))
    assert np.allclose(O.sdd_fused(lhs, rhs, topo, None, mult), plain * mult, rtol=1e-6)
    import torch
    want = torch.nn.functional.silu(torch.from_numpy(plain).double()).numpy() * mult
    assert np.allclose(O.sdd_fused(lhs, rhs, topo, "silu", mult), want, rtol=1e-5, atol=1e-6)


def test_inner_dimension_assert():
    rng = np.random.RandomState(0)
    x, data, topo = _random_sparse(rng, 32, 32, 0.5, 16)
    with pytest.raises(AssertionError):
        O.dsd((32, 32), data, topo, False, np.zeros((48, 16), np.float32))
    with pytest.raises(AssertionError):
        O.dds(np.zeros((16, 48), np.float32), (32, 32), data, topo, False)
    with pytest.raises(AssertionError):
        O.sdd(np.zeros((32, 8), np.float32), np.zeros((16, 32), np.float32), topo)


def test_dmoe_topology_matches_explicit_pattern():
    tokens = [130, 0, 64, 257, 1]     # ragged, one empty expert
    b, ffn = 8, 24
    topo = O.dmoe_topology(tokens, ffn, b)
    pad = O.padded_tokens_per_expert(tokens, b)
    assert pad.tolist() == [136, 0, 64, 264, 8]
    dense = np.zeros((int(pad.sum()), len(tokens) * ffn), dtype=np.float32)
    r0 = 0
    for e, p in enumerate(pad):
        dense[r0:r0 + p, e * ffn:(e + 1) * ffn] = 1
        r0 += p
    _, want = O.to_sparse(dense, b)
    assert topo.shape == want.shape
    for k in KAT:
        assert np.array_equal(getattr(topo, k), getattr(want, k)), k
        assert getattr(topo, k).dtype == getattr(want, k).dtype, k


# --------------------------------------------------------------------------
# token routing (defined in include/stk_amd.h; the reference has no code for it)
# --------------------------------------------------------------------------
# Worked by hand: 5 tokens, top-2 of 3 experts, blocking 4.  Expert 0 takes slots 1, 6; expert 1 slots 2, 5;
# expert 2 the other six; the bins are padded to 4, 4 and 8 rows.
ROUTE_KAT = {
    "top_experts": [[2, 0], [1, 2], [2, 1], [0, 2], [2, 2]],
    "indices": [1, 6, 2, 5, 0, 3, 4, 7, 8, 9],
    "bin_ids": [0, 0, 1, 1, 2, 2, 2, 2, 2, 2],
    "bins": [2, 4, 10],
    "padded_bins": [4, 8, 16],
    "slot_rows": [8, 0, 4, 9, 10, 5, 1, 11, 12, 13],
    "row_slots": [1, 6, -1, -1, 2, 5, -1, -1, 0, 3, 4, 7, 8, 9, -1, -1],
}


def _walk_route(experts, num_experts, blocking):
    """Slot-by-slot restatement of the definition, sharing no code with the oracle."""
    indices, bin_ids, bins, padded_bins, slot_rows, row_slots = [], [], [], [], [0] * len(experts), []
    for e in range(num_experts):
        mine = [s for s, x in enumerate(experts) if x == e]
        for s in mine:
            slot_rows[s] = len(row_slots)
            row_slots.append(s)
            indices.append(s)
            bin_ids.append(e)
        while len(row_slots) % blocking:
            row_slots.append(-1)
        bins.append(len(indices))
        padded_bins.append(len(row_slots))
    return indices, bin_ids, bins, padded_bins, slot_rows, row_slots


ROUTE_CASES = [  # (tokens, top_k, experts, blocking, seed)
    (0, 1, 4, 8, 0), (1, 1, 1, 128, 1), (7, 2, 3, 4, 2), (64, 1, 64, 128, 3), (300, 2, 5, 16, 4),
    (1000, 4, 64, 64, 5), (2050, 2, 100, 128, 6), (513, 1, 1024, 8, 7),
]


def route_experts(tokens, top_k, experts, seed):
    """top_k distinct experts per token, skewed so that some experts stay empty."""
    rng = np.random.default_rng(seed)
    k = min(top_k, experts)
    score = rng.random((tokens, experts)) * (1.0 + np.arange(experts)[None, :] % 3)
    top = np.argsort(-score, axis=1, kind="stable")[:, :k]
    if k < top_k:
        top = np.concatenate([top] * top_k, axis=1)[:, :top_k]
    return top.astype(np.int32)


def test_route_known_answer():
    r = O.route(ROUTE_KAT["top_experts"], 3, 4)
    for k in r._fields:
        assert getattr(r, k).tolist() == ROUTE_KAT[k], k
        assert getattr(r, k).dtype == np.int32


@pytest.mark.parametrize("tokens,top_k,experts,blocking,seed", ROUTE_CASES)
def test_route_against_walk_and_invariants(tokens, top_k, experts, blocking, seed):
    top = route_experts(tokens, top_k, experts, seed)
    flat = top.reshape(-1)
    r = O.route(top, experts, blocking)
    want = _walk_route(flat.tolist(), experts, blocking)
    for got, w, name in zip(r, want, r._fields):
        assert got.tolist() == w, name
    # what the definition implies: a sorted permutation, ascending slot inside an expert, mutually inverse maps
    assert sorted(r.indices.tolist()) == list(range(flat.size))
    assert np.all(np.diff(r.bin_ids) >= 0)
    same = np.diff(r.bin_ids) == 0
    assert np.all(np.diff(r.indices)[same] > 0)
    assert np.all(r.padded_bins % blocking == 0) and np.all(r.padded_bins >= r.bins)
    held = r.row_slots >= 0
    assert held.sum() == flat.size
    assert np.array_equal(r.slot_rows[r.row_slots[held]], np.nonzero(held)[0])
    # a larger layout only adds padding rows at the end
    big = O.route(top, experts, blocking, padded_rows=r.row_slots.size + 2 * blocking)
    assert np.array_equal(big.row_slots[:r.row_slots.size], r.row_slots) and np.all(big.row_slots[r.row_slots.size:] == -1)
    assert np.array_equal(big.slot_rows, r.slot_rows)


def _f32_walk_scatter(x, slot_rows, top_k, weights):
    tokens = len(slot_rows) // top_k
    out = np.zeros((tokens, x.shape[1]), dtype=np.float32)
    for t in range(tokens):
        for c in range(x.shape[1]):
            acc = None
            for k in range(top_k):
                s = t * top_k + k
                v = np.float32(x[slot_rows[s], c])
                if weights is not None:
                    v = np.float32(np.float32(weights[s]) * v)
                acc = v if acc is None else np.float32(acc + v)
            out[t, c] = acc
    return out


@pytest.mark.parametrize("top_k,weighted", [(1, False), (1, True), (2, False), (2, True), (3, True)])
def test_padded_copies_against_walk(top_k, weighted):
    rng = np.random.default_rng(top_k * 2 + weighted)
    tokens, experts, blocking, cols = 9, 4, 4, 8
    top = route_experts(tokens, top_k, experts, 11 + top_k)
    r = O.route(top, experts, blocking)
    x = rng.standard_normal((tokens, cols)).astype(np.float32)
    w = rng.random(tokens * top_k).astype(np.float32) if weighted else None
    g = O.padded_gather(x, r.row_slots, top_k, w)
    assert g.dtype == np.float32 and g.shape == (r.row_slots.size, cols)
    for row, s in enumerate(r.row_slots):
        want = np.zeros(cols, np.float32) if s < 0 else (x[s // top_k] if w is None else np.float32(w[s]) * x[s // top_k])
        assert np.array_equal(g[row], want)
    y = rng.standard_normal((r.row_slots.size, cols)).astype(np.float32)
    got = O.padded_scatter(y, r.slot_rows, top_k, w)
    assert got.dtype == np.float32
    assert np.array_equal(got, _f32_walk_scatter(y, r.slot_rows.tolist(), top_k, w))
    # gather then scatter without weights adds every token's row top_k times (exact for k = 1, 2, 4)
    if top_k in (1, 2):
        assert np.array_equal(O.padded_scatter(O.padded_gather(x, r.row_slots, top_k), r.slot_rows, top_k), top_k * x)
    # weight gradient: the derivative of sum(scatter * grad) with respect to each weight, against a direct sum
    grad = rng.standard_normal((tokens, cols)).astype(np.float32)
    dw = O.padded_scatter_weight_gradient(y, grad, r.slot_rows, top_k)
    for s in range(tokens * top_k):
        assert abs(dw[s] - float(np.dot(y[r.slot_rows[s]].astype(np.float64), grad[s // top_k].astype(np.float64)))) < 1e-9


def test_padded_scatter_sum_is_fp32_in_choice_order():
    # 2^24 + 1 + 1: in fp32, (2^24 + 1) + 1 = 2^24 + 2 is wrong by rounding order, ((2^24) + 1) = 2^24 then + 1 = 2^24;
    # summed the other way round, 1 + 1 = 2 first, it would be 2^24 + 2
    x = np.array([[2.0 ** 24], [1.0], [1.0]], dtype=np.float32)
    assert O.padded_scatter(x, [0, 1, 2], 3)[0, 0] == np.float32(2.0 ** 24)
    assert O.padded_scatter(x, [1, 2, 0], 3)[0, 0] == np.float32(2.0 ** 24 + 2)
    # -0.0 survives a lone term (the sum starts from the first product, not from +0)
    assert np.signbit(O.padded_scatter(np.array([[-0.0]], dtype=np.float32), [0], 1)[0, 0])
