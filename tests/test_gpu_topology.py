"""GPU parity, integer side: row_indices, transpose metadata, to_sparse, to_dense.

Everything runs through the C ABI (stk_amd.backend.hip_kernels -> libstk_amd.so)
on device tensors and must match the oracle and the committed fixtures bit for bit.
"""
import json
import os

import numpy as np
import pytest
import torch

import stk_amd as stk
from oracle import stk_oracle as O
from stk_amd.backend import hip_kernels
from tests import _util as U
from tests.test_oracle import FORMAT_CASES, GOLDEN, KAT

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def test_config1_known_answer_on_device():
    np.random.seed(0)
    x = stk.random.dense_mask(1024, 1024, 0.5, 128).half().to(DEV)
    m = stk.ops.to_sparse(x, 128)
    assert m.is_cuda and m.data.shape == (32, 128, 128) and bool((m.data == 1).all())
    for k, want in KAT.items():
        assert getattr(m, k).cpu().tolist() == want, k
    assert m.row_indices.dtype == torch.int16 and m.offsets_t.dtype == torch.int32 and m.block_offsets_t.dtype == torch.int32
    got = stk.ops.row_indices(m.size(), m.data, m.offsets, m.column_indices)
    assert got.dtype == torch.int16 and got.cpu().tolist() == KAT["row_indices"]
    assert torch.equal(stk.ops.to_dense(m), x)


def test_random_topology_fixtures_on_device():
    for fx in json.load(open(os.path.join(GOLDEN, "random_topologies.json"))):
        mask = torch.tensor(fx["mask"], dtype=torch.float16)
        x = mask.repeat_interleave(4, 0).repeat_interleave(4, 1).to(DEV)
        m = stk.ops.to_sparse(x, 4)
        for k in KAT:
            assert getattr(m, k).cpu().tolist() == fx[k], (fx["seed"], k)
        assert torch.equal(stk.ops.to_dense(m), x)


@pytest.mark.parametrize("rows,cols,sparsity,blocking", FORMAT_CASES)
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_format_round_trip(rows, cols, sparsity, blocking, dtype):
    # stk/ops/matrix_ops_test.py:26-58, on the device
    np.random.seed(rows * 3 + cols)
    torch.manual_seed(rows + cols)
    x = (torch.randn(rows, cols) * stk.random.dense_mask(rows, cols, sparsity, blocking)).to(dtype)
    m = stk.ops.to_sparse(x.to(DEV), blocking)
    if dtype == torch.float16:
        m.validate()
    data, topo = O.to_sparse(x.numpy(), blocking)
    U.assert_topology_equal(m, topo, "to_sparse")
    assert np.array_equal(m.data.cpu().numpy(), data)
    nnz = round(rows // blocking * cols // blocking * (1 - sparsity)) * blocking ** 2
    assert m.nnz == nnz
    dense = stk.ops.to_dense(m)
    assert dense.shape == x.shape and dense.dtype == dtype
    assert torch.equal(dense.cpu(), x)
    assert torch.count_nonzero(dense).item() == torch.count_nonzero(x).item()


def test_to_sparse_nan_negative_zero_and_strided_input():
    x = torch.zeros(8, 12, dtype=torch.bfloat16)
    x[0, 0] = -0.0
    x[4, 4] = float("nan")
    x[7, 11] = 1e-30
    m = stk.ops.to_sparse(x.to(DEV), 4)
    assert m.row_indices.cpu().tolist() == [1, 1] and m.column_indices.cpu().tolist() == [1, 2]
    # a column slice of a wider tensor: row stride != cols
    wide = torch.randn(16, 64, device=DEV).half()
    wide[:, 8:16] = 0
    view = wide[:, :32]
    m = stk.ops.to_sparse(view, 8)
    data, topo = O.to_sparse(view.cpu().numpy(), 8)
    U.assert_topology_equal(m, topo)
    assert np.array_equal(m.data.cpu().numpy(), data)


@pytest.mark.parametrize("index_dtype", [torch.int16, torch.int32])
@pytest.mark.parametrize("seed", range(5))
def test_transpose_meta_random_patterns(seed, index_dtype):
    rng = np.random.RandomState(seed)
    br, bc = [(7, 300), (300, 7), (129, 257), (1, 1), (600, 4100)][seed]
    mask = rng.rand(br, bc) < [0.3, 0.3, 0.05, 1.0, 0.02][seed]
    rows, cols = np.nonzero(mask)
    npdt = np.int16 if index_dtype == torch.int16 else np.int32
    ct, ot, bt = O.transpose_meta((br * 2, bc * 2), 2, rows.astype(npdt), cols.astype(npdt))
    data = torch.empty(len(rows), 2, 2, device=DEV, dtype=torch.float16)
    g_ct, g_ot, g_bt = hip_kernels.transpose_meta((br * 2, bc * 2), data, _dev(rows.astype(npdt)), _dev(cols.astype(npdt)), None)
    assert g_ct.dtype == index_dtype and g_ot.dtype == torch.int32 and g_bt.dtype == torch.int32
    assert np.array_equal(g_ot.cpu().numpy(), ot)
    assert np.array_equal(g_bt.cpu().numpy(), bt)
    assert np.array_equal(g_ct.cpu().numpy(), ct)


def test_transpose_meta_is_a_stable_sort_for_any_input():
    # unsorted columns inside rows, repeated coordinates, many ties: still ascending block id per column
    rng = np.random.RandomState(9)
    nnz, bc = 50000, 3
    rows = np.sort(rng.randint(0, 200, nnz)).astype(np.int16)
    cols = rng.randint(0, bc, nnz).astype(np.int16)
    ct, ot, bt = O.transpose_meta((400, bc * 2), 2, rows, cols)
    data = torch.empty(nnz, 2, 2, device=DEV, dtype=torch.float16)
    g_ct, g_ot, g_bt = hip_kernels.transpose_meta((400, bc * 2), data, _dev(rows), _dev(cols), None)
    assert np.array_equal(g_bt.cpu().numpy(), bt) and np.array_equal(g_ot.cpu().numpy(), ot) and np.array_equal(g_ct.cpu().numpy(), ct)


@pytest.mark.parametrize("index", [np.int16, np.int32])
@pytest.mark.parametrize("nnz,bc", [(16384, 700), (16385, 700), (300000, 5000), (1000, 1), (4097, 256), (4097, 257), (9000, 20000)])
def test_transpose_meta_at_the_sizes_where_the_method_changes(nnz, bc, index):
    # up to 16384 blocks one workgroup sorts everything in one launch; beyond that the passes are launches of their
    # own.  Many empty columns (also in front and at the end), one column, one or two digits.
    rng = np.random.RandomState(nnz % 97)
    rows = np.sort(rng.randint(0, 3000, nnz)).astype(index)
    cols = (bc // 50 + rng.randint(0, max(1, bc - bc // 25), nnz)).astype(index)
    ct, ot, bt = O.transpose_meta((6000, bc * 2), 2, rows, cols)
    data = torch.empty(nnz, 2, 2, device=DEV, dtype=torch.float16)
    g_ct, g_ot, g_bt = hip_kernels.transpose_meta((6000, bc * 2), data, _dev(rows), _dev(cols), None)
    assert np.array_equal(g_bt.cpu().numpy(), bt) and np.array_equal(g_ot.cpu().numpy(), ot) and np.array_equal(g_ct.cpu().numpy(), ct)


def test_empty_matrix():
    x = torch.zeros(64, 128, dtype=torch.float16, device=DEV)
    m = stk.ops.to_sparse(x, 16)
    assert m.nnz == 0 and m.offsets.cpu().tolist() == [0] * 5 and m.offsets_t.cpu().tolist() == [0] * 9
    assert m.block_offsets_t.numel() == 0 and m.column_indices_t.numel() == 0
    assert torch.equal(stk.ops.to_dense(m), x)
    assert stk.ops.row_indices(m.size(), m.data, m.offsets, m.column_indices).numel() == 0


@pytest.mark.parametrize("name", ["c3_top1", "c4_zipf_top2", "c5_b64", "c5_skew"])
def test_dmoe_topologies_full_size(name):
    # the block-diagonal topologies of the benchmark configurations, at full size
    if name == "c3_top1":
        tokens, ffn, b = U.dmoe_tokens_top1(16384, 64, 0), 4096, 128
    elif name == "c4_zipf_top2":
        tokens, ffn, b = U.dmoe_tokens_zipf_top2(32768, 64, 0), 8192, 128
    elif name == "c5_b64":
        tokens, ffn, b = U.dmoe_tokens_top1(16384, 64, 0), 4096, 64
    else:
        tokens, ffn, b = U.dmoe_tokens_skewed(16384, 64, 0), 4096, 64
    topo = O.dmoe_topology(tokens, ffn, b)
    nnz = len(topo.row_indices)
    data = torch.empty(nnz, 1, 1, device=DEV, dtype=torch.float16).expand(nnz, b, b)  # metadata only: no block storage
    offsets = _dev(topo.offsets)
    ci = _dev(topo.column_indices)
    ri = stk.ops.row_indices(topo.shape, data, offsets, ci)
    assert np.array_equal(ri.cpu().numpy(), topo.row_indices)
    m = stk.Matrix(torch.Size(topo.shape), data, ri, ci, offsets)   # builds the transpose metadata on the device
    U.assert_topology_equal(m, topo, name)
    # invariants that hold at any size
    bt = m.block_offsets_t.long()
    assert torch.equal(torch.sort(bt).values, torch.arange(nnz, device=DEV))
    assert torch.equal(m.row_indices[bt], m.column_indices_t)
    assert torch.equal(torch.sort(m.column_indices[bt].int(), stable=True).values, m.column_indices[bt].int())


def _greedy_roles(offsets, indices):
    """Plain statement of the fusion plan: runs of identical non-empty lines paired from the start of the run."""
    lines = len(offsets) - 1
    seg = [tuple(indices[offsets[i]:offsets[i + 1]]) for i in range(lines)]
    role = [0] * lines
    i = 0
    while i < lines:
        if i + 1 < lines and len(seg[i]) > 0 and seg[i] == seg[i + 1]:
            role[i], role[i + 1] = 1, 2
            i += 2
        else:
            i += 1
    return role


def _greedy_roles_with_threes(offsets, indices):
    """The same pairing, except that the last three lines of an odd run of three or more form one group (role 3)."""
    lines = len(offsets) - 1
    seg = [tuple(indices[offsets[i]:offsets[i + 1]]) for i in range(lines)]
    role = [0] * lines
    i = 0
    while i < lines:
        n = 1
        while i + n < lines and len(seg[i]) > 0 and seg[i + n] == seg[i]:
            n += 1
        j = 0
        while n - j >= 2:
            if n - j == 3:
                role[i + j:i + j + 3] = [3, 2, 2]
                j += 3
            else:
                role[i + j:i + j + 2] = [1, 2]
                j += 2
        i += n
    return role


@pytest.mark.parametrize("name", ["dmoe", "skewed", "random", "dense", "empty", "runs", "many", "tall"])
def test_fusion_plan_roles(name):
    if name == "dmoe":
        topo = O.dmoe_topology([300, 0, 129, 1, 640, 128, 77, 256, 512], 512, 128)
    elif name == "skewed":
        topo = O.dmoe_topology([3000, 900, 400, 300] + [128] * 28, 512, 128)
    else:
        rng = np.random.RandomState(1)
        if name == "random":
            mask = rng.rand(37, 23) < 0.3
        elif name == "dense":
            mask = np.ones((9, 5), bool)
        elif name == "empty":
            mask = np.zeros((6, 4), bool)
        elif name == "many":    # more lone rows than the plan sorts (they stay ascending); columns of about 100 blocks
            mask = rng.rand(5000, 300) < 0.02
        elif name == "tall":    # columns of more than 255 blocks: equal keys, ascending among themselves
            mask = rng.rand(600, 7) < 0.7
        else:   # runs of 1..5 identical rows, some empty rows in between
            rows = []
            for n in [1, 2, 3, 4, 5, 2, 1, 3, 9, 6]:
                pattern = rng.rand(11) < 0.4
                rows += [pattern] * n + [np.zeros(11, bool)]
            mask = np.array(rows)
        x = np.kron(mask, np.ones((2, 2), dtype=np.float32))
        _, topo = O.to_sparse(x, 2)
    br, bc = len(topo.offsets) - 1, len(topo.offsets_t) - 1
    nnz = len(topo.column_indices)
    plan = hip_kernels.fusion_plan(_dev(topo.offsets), _dev(topo.column_indices), _dev(topo.offsets_t), _dev(topo.column_indices_t))
    whole = plan.cpu().numpy()
    max_tiles = (nnz + br + 1) // 2
    sdd_bytes = 8 + 8 * max_tiles
    got = whole[sdd_bytes:]
    assert got[:br].tolist() == _greedy_roles(topo.offsets, topo.column_indices)
    assert got[br:br + bc].tolist() == _greedy_roles(topo.offsets_t, topo.column_indices_t)
    tall = got[2 * (br + bc):]
    assert tall[:br].tolist() == _greedy_roles_with_threes(topo.offsets, topo.column_indices)
    assert tall[br:br + bc].tolist() == _greedy_roles_with_threes(topo.offsets_t, topo.column_indices_t)
    # behind the roles: ten counts, then five lists per direction (role 1, role 0, tall 1, tall 3, tall 0), longest lines first
    off = (3 * (br + bc) + 3) // 4 * 4
    lists = got[off:off + 4 * 5 * (2 + br + bc)].view(np.int32)
    for d, (lines, roles, talls) in enumerate([(br, got[:br], tall[:br]), (bc, got[br:br + bc], tall[br:br + bc])]):
        base = 10 + (5 * br if d else 0)
        offs = topo.offsets_t if d else topo.offsets
        for kind, (src, want) in enumerate([(roles, 1), (roles, 0), (talls, 1), (talls, 3), (talls, 0)]):
            expect = np.nonzero(src == want)[0].tolist()
            expect = _longest_first(expect, offs)   # every list: longest first, equal lengths in ascending order
            assert int(lists[5 * d + kind]) == len(expect)
            assert lists[base + kind * lines: base + kind * lines + len(expect)].tolist() == expect
    # behind the lists, per direction: slice counts for dsd (1 .. 4) and the hint that the blocks are spread
    # unevenly over equal eighths of the lines
    hints = got[off + 4 * 5 * (2 + br + bc):]
    for d, (lines, offs) in enumerate([(br, topo.offsets), (bc, topo.offsets_t)]):
        h = hints[32 * d:32 * d + 32]
        assert all(1 <= int(v) <= 4 for v in h[:16])
        shares = [int(offs[(c + 1) * lines // 8]) - int(offs[c * lines // 8]) for c in range(8)]
        assert int(h[16]) == int(any(32 * sh > 5 * int(offs[lines]) for sh in shares)), (d, shares)
        # and per list the entries that go to one compute die at a time: a quarter of a die's share of the list's
        # blocks in entries as long as the first one, rounded down to a power of two between 1 and 32
        base = 10 + (5 * br if d else 0)
        for kind in range(5):
            count = int(lists[5 * d + kind])
            entries = 1
            if count:
                members = lists[base + kind * lines: base + kind * lines + count].tolist()
                blocks = [int(offs[i + 1]) - int(offs[i]) for i in members]
                fit = sum(blocks) // (32 * max(blocks[0], 1))
                while entries < 32 and 2 * entries <= fit:
                    entries *= 2
            assert int(h[17 + kind]) == entries, (d, kind, count)
        # and from how many 128-wide tiles of the dense operand on the launches over single lines deal their tiles to
        # the compute dies by stripes of the dense operand: ceil(7 nnz / (G - K)), G = the blocks of one line per list
        # entry, K = the lines of the other direction (0: never; beyond 255: never); byte 22 for the lists with threes,
        # byte 23 for the lists of pairs and lone lines
        others = bc if d == 0 else br
        for byte, kinds in ((22, (2, 3, 4)), (23, (0, 1))):
            g_blocks = 0
            for kind in kinds:
                count = int(lists[5 * d + kind])
                members = lists[base + kind * lines: base + kind * lines + count].tolist()
                g_blocks += sum(int(offs[i + 1]) - int(offs[i]) for i in members)
            saved = g_blocks - others
            want = 0
            if saved > 0:
                want = max(1, -(-7 * int(offs[lines]) // saved))
                want = 0 if want > 255 else want
            assert int(h[byte]) == want, (d, byte, g_blocks, others)
    # in front: the tiles of sdd
    sdd = whole[:8 + 8 * max_tiles].view(np.int32)
    assert sdd[2:2 + 2 * sdd[0]].reshape(-1, 2).tolist() == _sdd_tiles(topo.offsets, topo.column_indices, 2, 2)
    # and for 64-blocks: tiles of up to 4 x 4 blocks
    plan64 = hip_kernels.fusion_plan(_dev(topo.offsets.copy()), _dev(topo.column_indices), blocking=64).cpu().numpy()
    sdd64 = plan64[:8 + 8 * max_tiles].view(np.int32)
    assert sdd64[2:2 + 2 * sdd64[0]].reshape(-1, 2).tolist() == _sdd_tiles(topo.offsets, topo.column_indices, 4, 4)
    # a plan for 64-blocks built with both directions: groups of up to four identical lines; both role arrays hold
    # the size of the group at its first line, and the lists are fours, (none), pairs, threes, lone lines
    both64 = hip_kernels.fusion_plan(_dev(topo.offsets.copy()), _dev(topo.column_indices), _dev(topo.offsets_t), _dev(topo.column_indices_t),
                                     blocking=64).cpu().numpy()[sdd_bytes:]
    want_rows, want_cols = _groups_of_up_to_four(topo.offsets, topo.column_indices), _groups_of_up_to_four(topo.offsets_t, topo.column_indices_t)
    assert both64[:br].tolist() == want_rows and both64[br:br + bc].tolist() == want_cols
    assert both64[2 * (br + bc):2 * (br + bc) + br].tolist() == want_rows
    lists64 = both64[off:off + 4 * 5 * (2 + br + bc)].view(np.int32)
    for d, (lines, sizes) in enumerate([(br, np.array(want_rows)), (bc, np.array(want_cols))]):
        base = 10 + (5 * br if d else 0)
        offs = topo.offsets_t if d else topo.offsets
        for kind, size in enumerate([4, None, 2, 3, 1]):
            expect = [] if size is None else np.nonzero(sizes == size)[0].tolist()
            expect = _longest_first(expect, offs)
            assert int(lists64[5 * d + kind]) == len(expect), (d, kind)
            assert lists64[base + kind * lines: base + kind * lines + len(expect)].tolist() == expect
    rows_only = hip_kernels.fusion_plan(_dev(topo.offsets), _dev(topo.column_indices)).cpu().numpy()
    assert rows_only[:8 + 8 * int(sdd[0])].tolist() == whole[:8 + 8 * int(sdd[0])].tolist()
    assert rows_only[sdd_bytes:sdd_bytes + br].tolist() == got[:br].tolist()


def _longest_first(lines, offsets):
    """Lines in order of descending min(blocks, 255), equal lengths ascending (lists of more than 4096 stay ascending)."""
    if len(lines) > 4096:
        return lines
    return sorted(lines, key=lambda i: (-min(int(offsets[i + 1]) - int(offsets[i]), 255), i))


def _groups_of_up_to_four(offsets, indices):
    """Size of the group that starts at each line (0 for a line inside a group): a run of identical, non-empty
    lines is cut from its start into fours while they last; the three, two or one lines left form one more group.
    Lines with more than nnz / compute units blocks (a tile over four of them would exceed a compute unit's share
    of a product with four tiles in the other dimension) are cut into pairs instead."""
    lines = len(offsets) - 1
    seg = [tuple(indices[offsets[i]:offsets[i + 1]]) for i in range(lines)]
    share = max(1, int(offsets[lines]) * 4 // torch.cuda.get_device_properties(0).multi_processor_count)
    size = [0] * lines
    i = 0
    while i < lines:
        n = 1
        while i + n < lines and len(seg[i]) > 0 and seg[i + n] == seg[i]:
            n += 1
        if 4 * len(seg[i]) > share:
            for a in range(0, n, 2):
                size[i + a] = min(2, n - a)
        else:
            for a, r in _fours(n):
                size[i + a] = r
        i += n
    return size


def _fours(n):
    """(first line, lines) of the groups a run of n identical lines is cut into: fours from the start, then the
    three, two or one lines left - but a four and one line left over become a three and a pair."""
    groups, a = [], 0
    while a < n:
        left = n - a
        r = 4 if left >= 6 or left == 4 else (3 if left == 5 else left)
        groups.append((a, r))
        a += r
    return groups


def _sdd_tiles(offsets, indices, most_rows, most_cols):
    """Plain statement of the sdd tile list: row by row; a run of identical rows is cut from its start into groups
    (most_rows 4: fours while they last, then the three, two or one rows that are left as one more group; 2: pairs,
    with the last three rows of an odd run of three or more as one group), and the first row of a group owns one
    tile per `most_cols` neighbouring blocks (per block for a group of three when most_cols is 2):
    (first block, rows | cols << 8)."""
    rows = len(offsets) - 1
    seg = [tuple(indices[offsets[i]:offsets[i + 1]]) for i in range(rows)]
    tiles = []
    i = 0
    while i < rows:
        n = 1
        while i + n < rows and len(seg[i]) > 0 and seg[i + n] == seg[i]:
            n += 1
        nseg = len(seg[i])
        a = 0
        while a < n:
            if most_rows == 4:
                r = dict(_fours(n))[a]
            else:
                r = 3 if n - a == 3 else min(2, n - a)
            wide = 1 if (r == 3 and most_cols == 2) else most_cols
            tiles += [[offsets[i + a] + j, r | (min(wide, nseg - j) << 8)] for j in range(0, nseg, wide)]
            a += r
        i += n
    return tiles


_DMOE_BUILDER_CASES = [
    ([300, 0, 129, 1, 640, 128, 77, 256], 4, 128, torch.int16),
    ([128], 1, 128, torch.int16),
    ([0, 0, 5], 3, 64, torch.int16),
    ([64, 64, 0, 0], 2, 64, torch.int32),
    ([1] * 40, 7, 8, torch.int32),
]


@pytest.mark.parametrize("tokens,width,blocking,index_dtype", _DMOE_BUILDER_CASES)
def test_dmoe_topology_builder_matches_oracle_and_sort(tokens, width, blocking, index_dtype):
    topo = O.dmoe_topology(tokens, width * blocking, blocking, np.int16 if index_dtype == torch.int16 else np.int32)
    pad = O.padded_tokens_per_expert(tokens, blocking)
    bins = torch.from_numpy(np.cumsum(pad).astype(np.int32)).to(DEV)
    block_rows = int(pad.sum()) // blocking
    m = stk.ops.dmoe_topology(bins, blocking, block_rows, width, dtype=torch.float16, index_dtype=index_dtype)
    assert tuple(m.size()) == tuple(topo.shape) and m.row_indices.dtype == index_dtype
    U.assert_topology_equal(m, topo, "builder")
    if index_dtype == torch.int16:
        m.validate()      # the reference's own consistency check (float16 values, 16-bit indices)
    # the sort-based path on the same pattern gives the same transpose metadata
    ct, ot, bt = hip_kernels.transpose_meta(m.size(), m.data, m.row_indices, m.column_indices, m.offsets)
    assert torch.equal(ct, m.column_indices_t) and torch.equal(ot, m.offsets_t) and torch.equal(bt, m.block_offsets_t)
    ri = torch.empty_like(m.row_indices)
    hip_kernels.row_indices(m.size(), m.data, m.offsets, m.column_indices, ri)
    assert torch.equal(ri, m.row_indices)


def test_dmoe_topology_builder_full_size_and_in_a_product():
    tokens = U.dmoe_tokens_zipf_top2(32768, 64, 0)          # 65536 token slots, skewed
    pad = O.padded_tokens_per_expert(tokens, 128)
    topo = O.dmoe_topology(tokens, 8192, 128)
    bins = torch.from_numpy(np.cumsum(pad).astype(np.int32)).to(DEV)
    m = stk.ops.dmoe_topology(bins, 128, int(pad.sum()) // 128, 64)
    U.assert_topology_equal(m, topo, "builder, 65536 slots")
    # a small one straight into sdd: equals the dense product under the mask
    tokens = np.array([200, 0, 384, 129])
    pad = O.padded_tokens_per_expert(tokens, 128)
    topo = O.dmoe_topology(tokens, 256, 128)
    bins = torch.from_numpy(np.cumsum(pad).astype(np.int32)).to(DEV)
    m = stk.ops.dmoe_topology(bins, 128, int(pad.sum()) // 128, 2)
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(m.size()[0], 64, generator=g) * 0.1).bfloat16().to(DEV)
    w = (torch.randn(64, m.size()[1], generator=g) * 0.1).bfloat16().to(DEV)
    U.assert_close(stk.ops.sdd(x, w, m).data, O.sdd(U.np32(x), U.np32(w), topo), torch.bfloat16, "sdd on a built topology")


def test_dmoe_topology_builder_rejects_bad_arguments():
    bins = torch.tensor([128], dtype=torch.int32, device=DEV)
    with pytest.raises(AssertionError):
        hip_kernels.dmoe_topology(bins, 128, 1, 0)
    with pytest.raises(AssertionError):                      # 40000 block columns do not fit 16-bit indices
        hip_kernels.dmoe_topology(bins, 128, 1, 40000)


def test_to_sparse_of_a_large_sparse_matrix_keeps_only_what_it_uses():
    # 1024 x 1024 blocks of 8 with 37 of them nonzero: the index tensors and the offsets own their storage, so that a
    # Matrix does not hold on to the buffers sized for every block that the conversion works in
    rows = cols = 8192
    x = torch.zeros(rows, cols, dtype=torch.float16, device=DEV)
    g = torch.Generator().manual_seed(4)
    where = torch.randperm(1024 * 1024, generator=g)[:37]
    for w in where.tolist():
        x[(w // 1024) * 8 + 3, (w % 1024) * 8 + 5] = 1.0
    m = stk.ops.to_sparse(x, 8)
    assert m.row_indices.numel() == 37
    for t, elems in ((m.row_indices, 37), (m.column_indices, 37), (m.offsets, 1025)):
        assert t.untyped_storage().nbytes() <= max(512, 2 * elems * t.element_size()), t.untyped_storage().nbytes()
    data, topo = O.to_sparse(x.cpu().numpy(), 8)
    U.assert_topology_equal(m, topo, "large sparse")
    assert torch.equal(stk.ops.to_dense(m), x)
