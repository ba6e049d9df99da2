"""Random differential test: the three products and all their gradients on random topologies against the dense
fp32 comparator that the tolerance is stated for (to_dense + torch.matmul, masked to the topology), on the GPU.

Each case draws a block size, a value type, an index type, a pattern (uniformly random blocks, runs of identical
rows, block-diagonal experts with and without empty experts), transposes for both operands and the dense extents.
The seeds are fixed, so a failure names a case that can be run again.  Tolerance: |got - want| <= atol + 1e-2 |want|
with atol 1e-2 (bfloat16) / 5e-3 (float16), and, because operands of this size leave that bound loose, also
max |got - want| <= 2^-6 (2^-9) of the largest |want| - a dropped or doubled block fails it.
"""
import numpy as np
import pytest
import torch

import stk_amd as stk

pytestmark = pytest.mark.gpu
DEV = "cuda"
CASES_PER_TEST = 40


def _check(name, got, want, dtype, info):
    got, want = got.float(), want.float()
    atol = 1e-2 if dtype == torch.bfloat16 else 5e-3
    err = (got - want).abs()
    assert torch.isfinite(got).all(), (name, info)
    assert bool((err <= atol + 1e-2 * want.abs()).all()), (name, info, err.max().item())
    scale_free = 2.0 ** -6 if dtype == torch.bfloat16 else 2.0 ** -9
    assert err.max().item() <= scale_free * want.abs().max().item() + 1e-30, (name, info, err.max().item(), want.abs().max().item())


def _pattern(rng):
    kind = rng.choice(["random", "runs", "experts", "wide experts"])
    if kind == "random":
        mask = rng.rand(int(rng.randint(1, 24)), int(rng.randint(1, 24))) < rng.choice([0.1, 0.3, 0.6, 1.0])
    elif kind == "runs":      # runs of identical block rows (fused tiles), some of them empty
        rows, cols = int(rng.randint(2, 40)), int(rng.randint(2, 24))
        patterns = rng.rand(4, cols) < 0.5
        mask = patterns[np.sort(rng.randint(0, 4, rows))]
    else:                     # block-diagonal: experts of 0 .. 8 block rows
        experts = int(rng.randint(1, 12))
        per = int(rng.choice([1, 2, 4, 8] if kind == "experts" else [16, 32]))
        rows_of = rng.randint(0, 5 if kind == "experts" else 9, experts)
        if rows_of.sum() == 0:
            rows_of[0] = 1
        mask = np.zeros((int(rows_of.sum()), experts * per), bool)
        r0 = 0
        for e, n in enumerate(rows_of):
            mask[r0:r0 + n, e * per:(e + 1) * per] = True
            r0 += n
    return str(kind), mask


def _like(s, data):
    return stk.Matrix(s.size(), data, s.row_indices, s.column_indices, s.offsets, s.column_indices_t, s.offsets_t, s.block_offsets_t)


@pytest.mark.parametrize("batch", range(5))
def test_random_products_and_gradients_against_dense_fp32(batch):
    for case in range(CASES_PER_TEST):
        seed = 7000 + batch * CASES_PER_TEST + case
        rng = np.random.RandomState(seed)
        torch.manual_seed(seed)
        b = int(rng.choice([128, 128, 64]))
        dtype = torch.bfloat16 if rng.rand() < 0.5 else torch.float16
        kind, mask = _pattern(rng)
        m, k = mask.shape[0] * b, mask.shape[1] * b
        n = b * int(rng.choice([1, 2, 3, 4, 8, rng.randint(1, 12)]))
        inner = b * int(rng.choice([1, 2, 4, 8, rng.randint(1, 12)]))
        ta, tb = bool(rng.rand() < 0.5), bool(rng.rand() < 0.5)
        idx32 = bool(rng.rand() < 0.2)
        info = dict(seed=seed, blocking=b, dtype=str(dtype), pattern=kind, shape=(m, k), n=n, inner=inner, ta=ta, tb=tb, idx32=idx32)
        dense_mask = torch.from_numpy(np.kron(mask, np.ones((b, b), dtype=np.float32))).to(DEV)
        vals = (torch.randn(m, k, device=DEV) * 0.5).to(dtype) * dense_mask.to(dtype)
        vals = torch.where((dense_mask > 0) & (vals == 0), torch.ones_like(vals), vals)   # to_sparse keeps every block of the mask
        s = stk.ops.to_sparse(vals, b)
        assert s.nnz == int(mask.sum()) * b * b, info
        if idx32:
            s = stk.Matrix(s.size(), s.data, s.row_indices.int(), s.column_indices.int(), s.offsets, s.column_indices_t.int(), s.offsets_t,
                           s.block_offsets_t)
        sd = vals.float()

        def randn(*shape):
            return (torch.randn(*shape, device=DEV) * 0.5).to(dtype)

        def view(t, transposed):    # the same values, as a .t() view of a contiguous tensor or contiguous
            return (t.t().contiguous().t() if transposed else t).detach().requires_grad_(True)

        # dsd: op(S) rhs and its two gradients
        rhs = randn(m if ta else k, n)
        values, rhs_arg = s.data.detach().clone().requires_grad_(True), view(rhs, tb)
        sm = _like(s, values)
        out = stk.ops.dsd(sm.t() if ta else sm, rhs_arg)
        _check("dsd", out, (sd.t() if ta else sd) @ rhs.float(), dtype, info)
        dy = randn(*out.shape)
        out.backward(dy)
        _check("dsd: gradient of rhs", rhs_arg.grad, (sd if ta else sd.t()) @ dy.float(), dtype, info)
        ds = (rhs.float() @ dy.float().t()) if ta else (dy.float() @ rhs.float().t())
        _check("dsd: gradient of the values", stk.ops.to_dense(_like(s, values.grad)), ds * dense_mask, dtype, info)

        # dds: lhs op(S) and its two gradients
        lhs = randn(n, k if tb else m)
        values, lhs_arg = s.data.detach().clone().requires_grad_(True), view(lhs, ta)
        sm = _like(s, values)
        out = stk.ops.dds(lhs_arg, sm.t() if tb else sm)
        _check("dds", out, lhs.float() @ (sd.t() if tb else sd), dtype, info)
        dy = randn(*out.shape)
        out.backward(dy)
        _check("dds: gradient of lhs", lhs_arg.grad, dy.float() @ (sd if tb else sd.t()), dtype, info)
        ds = (dy.float().t() @ lhs.float()) if tb else (lhs.float().t() @ dy.float())
        _check("dds: gradient of the values", stk.ops.to_dense(_like(s, values.grad)), ds * dense_mask, dtype, info)

        # sdd: lhs rhs on the pattern and its two gradients
        lhs, rhs = randn(m, inner), randn(inner, k)
        lhs_arg, rhs_arg = view(lhs, ta), view(rhs, tb)
        out = stk.ops.sdd(lhs_arg, rhs_arg, s)
        _check("sdd", stk.ops.to_dense(out), (lhs.float() @ rhs.float()) * dense_mask, dtype, info)
        dvalues = randn(*out.data.shape)
        out.data.backward(dvalues)
        ds = stk.ops.to_dense(_like(s, dvalues)).float()
        _check("sdd: gradient of lhs", lhs_arg.grad, ds @ rhs.float().t(), dtype, info)
        _check("sdd: gradient of rhs", rhs_arg.grad, lhs.float().t() @ ds, dtype, info)


def _same(name, got, want, info):
    got = got.cpu().numpy() if torch.is_tensor(got) else np.asarray(got)
    want = want.cpu().numpy() if torch.is_tensor(want) else want
    assert got.shape == np.asarray(want).shape and np.array_equal(got, want), (name, info)


@pytest.mark.parametrize("batch", range(3))
def test_random_routings_and_formats_bit_exact_against_the_oracle(batch):
    # the integer paths: routing, the row copy into the padded layout, the dMoE topology of that routing, and
    # to_sparse / transpose metadata / row_indices / to_dense on a random pattern, bit for bit against numpy
    from oracle import stk_oracle as O
    meta = ("offsets", "row_indices", "column_indices", "offsets_t", "column_indices_t", "block_offsets_t")
    for case in range(25):
        seed = 9000 + 25 * batch + case
        rng = np.random.RandomState(seed)
        tokens = int(rng.choice([1, 7, 100, 1000, 5000, rng.randint(1, 20000)]))
        top_k = int(rng.choice([1, 1, 2, 2, 4, 3]))
        experts = int(rng.choice([1, 2, 8, 64, 100, rng.randint(max(top_k, 1), 300)]))
        blocking = int(rng.choice([8, 64, 128]))
        skew = float(rng.choice([0.0, 1.2, 3.0]))
        p = np.arange(1, experts + 1, dtype=np.float64) ** -skew
        top = rng.choice(experts, size=(tokens, top_k), p=p / p.sum()).astype(np.int32)
        info = dict(seed=seed, tokens=tokens, top_k=top_k, experts=experts, blocking=blocking, skew=skew)
        want = O.route(top, experts, blocking)
        r = stk.ops.route(torch.from_numpy(top).to(DEV), experts, blocking)
        for f in want._fields:
            _same("route " + f, getattr(r, f), getattr(want, f), info)
        x = torch.randn(tokens, 8 * int(rng.randint(1, 40)), generator=torch.Generator().manual_seed(seed)).to(torch.bfloat16)
        _same("gather", stk.ops.padded_gather(x.to(DEV), r).float(), O.padded_gather(x.float().numpy(), want.row_slots, top_k), info)
        if blocking >= 64 and experts <= 64:
            per = int(rng.choice([1, 2, 4]))
            t = stk.ops.dmoe_topology(r.padded_bins, blocking, int(want.padded_bins[-1]) // blocking, per, dtype=torch.bfloat16)
            wt = O.dmoe_topology(np.diff(np.concatenate([[0], want.bins])), per * blocking, blocking)
            for f in meta:
                _same("dmoe_topology " + f, getattr(t, f), getattr(wt, f), info)
        b = int(rng.choice([1, 2, 16, 64, 128]))
        br, bc = int(rng.randint(1, 60)), int(rng.randint(1, 60))
        mask = rng.rand(br, bc) < rng.choice([0.0, 0.05, 0.3, 0.9])
        xd = (np.kron(mask, np.ones((b, b))) * rng.randn(br * b, bc * b)).astype(np.float16)
        info = dict(seed=seed, blocking=b, block_rows=br, block_cols=bc)
        s = stk.ops.to_sparse(torch.from_numpy(xd).to(DEV), b)
        wd, wt = O.to_sparse(xd, b)
        _same("to_sparse values", s.data, wd, info)
        for f in meta:
            _same("to_sparse " + f, getattr(s, f), getattr(wt, f), info)
        _same("to_dense", stk.ops.to_dense(s), xd, info)
        _same("row_indices", stk.ops.row_indices(s.size(), s.data, s.offsets, s.column_indices), wt.row_indices, info)


@pytest.mark.parametrize("batch", range(2))
def test_random_routed_products_bit_exact_against_the_two_launches(batch):
    """stk_sdd_gather, stk_dsd_scatter and the sums kept by stk_sdd_fused_sums on random routings and sizes: the
    products on the token rows must give the bits of copy + product (where the library has no kernel for a case the
    ops run the two launches, and the comparison holds trivially)."""
    from stk_amd.backend import hip_kernels
    fused = {"gather": 0, "scatter": 0}
    for case in range(12):
        seed = 9100 + batch * 12 + case
        rng = np.random.RandomState(seed)
        torch.manual_seed(seed)
        dtype = [torch.bfloat16, torch.float16][int(rng.randint(2))]
        experts = int(rng.choice([2, 5, 8, 16, 33]))
        top_k = int(rng.choice([1, 1, 2]))
        tokens = int(rng.choice([300, 1500, 4000, 9000]))
        hidden = int(rng.choice([128, 256, 384, 512, 1024]))
        ffn = int(rng.choice([128, 384, 1024, 2560]))
        skew = float(rng.choice([0.0, 1.5, 4.0]))
        if case < 2:     # enough blocks x columns for the eight-wavefront dsd, whose store the scatter is part of
            experts, top_k, tokens, hidden, ffn = 8, 1, 9000, [1024, 512][case], [2560, 5120][case]
        info = dict(seed=seed, dtype=dtype, experts=experts, top_k=top_k, tokens=tokens, hidden=hidden, ffn=ffn, skew=skew)
        logits = torch.randn(tokens, experts)
        logits[:, 0] += skew
        if experts > 2:
            logits[:, 1] = -1e9                      # an expert without tokens
        top = logits.topk(top_k, dim=1).indices.to(torch.int32).to(DEV)
        capacity = stk.ops.route_capacity(tokens * top_k, experts, 128) if rng.rand() < 0.3 else None
        r = stk.ops.route(top, experts, 128, padded_rows=capacity)
        rows = r.row_slots.numel()
        topo = stk.ops.dmoe_topology(r.padded_bins, 128, rows // 128, ffn // 128, dtype=dtype)
        x = torch.randn(tokens, hidden).to(dtype).to(DEV)
        w1 = (torch.randn(hidden, experts * ffn) * 0.05).to(dtype).to(DEV)
        w2 = (torch.randn(experts * ffn, hidden) * 0.05).to(dtype).to(DEV)
        if rng.rand() < 0.5:
            w1 = w1.t().contiguous().t()
        if rng.rand() < 0.5:
            w2 = w2.t().contiguous().t()
        activation = [None, "relu", "gelu_tanh", "silu"][int(rng.randint(4))]
        weights = (torch.rand(tokens, top_k, device=DEV) + 0.5) if rng.rand() < 0.5 else None
        padded = stk.ops.padded_gather(x, r)
        want_h = stk.ops.sdd_fused(padded, w1, topo, activation)
        got_h = stk.ops.gather_sdd(x, r, w1, topo, activation)
        _same("gather_sdd", got_h.data.view(torch.int16), want_h.data.view(torch.int16), info)
        want_y = stk.ops.padded_scatter(stk.ops.dsd(want_h, w2), r, weights)
        got_y = stk.ops.dsd_scatter(want_h, w2, r, weights)
        _same("dsd_scatter", got_y.view(torch.int16), want_y.view(torch.int16), info)
        # which cases reached the kernels
        out = torch.empty_like(topo.data)
        fused["gather"] += bool(hip_kernels.sdd_gather(x, r.row_slots, top_k, w1, topo.size(), out, topo.offsets, topo.row_indices,
                                                       topo.column_indices, activation))
        if top_k == 1:
            y = torch.empty(tokens, hidden, dtype=dtype, device=DEV)
            fused["scatter"] += bool(hip_kernels.dsd_scatter(want_h.size(), want_h.data, want_h.offsets, want_h.column_indices, want_h.offsets_t,
                                                             want_h.column_indices_t, w2, r.row_slots, weights, y))
        # the kept sums are the plain product
        if activation is not None:
            sums = torch.empty_like(topo.data)
            again = torch.empty_like(topo.data)
            hip_kernels.sdd_fused(padded, w1, topo.size(), again, topo.offsets, topo.row_indices, topo.column_indices, activation, sums=sums)
            _same("sums", sums.view(torch.int16), stk.ops.sdd(padded, w1, topo).data.view(torch.int16), info)
            _same("fused beside sums", again.view(torch.int16), want_h.data.view(torch.int16), info)
    assert fused["gather"] >= 8, fused     # every case at blocking 128 has the gathered product
    assert fused["scatter"] >= 2, fused
