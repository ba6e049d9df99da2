#!/usr/bin/env python3
"""Benchmark of the block-sparse products on the dMoE FFN forward topology.

Workload (one GPU): 16384 tokens routed top-1 over 64 experts (N(0,1) logits,
seed 0), per-expert token counts padded to 128, hidden 1024, ffn 4096, bf16:
the block-diagonal topology [T', 64 * 4096] with 128 x 128 blocks.  One step is
    h   = sdd(x, W1, topo)        x [T', 1024], W1 [1024, 64 * 4096]
    y   = dsd(h, W2)              W2 [64 * 4096, 1024]
    dW1 = dds(x^T, h)             the layer-0 weight-gradient shape (walks the CSC metadata)
and the metric is effective TFLOP/s over nonzero blocks, nnz * 2 * 128^2 * 1024
FLOP per product.  Inputs are synthetic and resident in HBM before timing.

Order of the run: the same-problem dense GEMMs and the routing are timed first (they also bring
the GPU to its steady clocks: the first ~100 ms of work after an idle period run up to 15 % slower),
then W untimed steps, then K steps timed by the wall clock between two synchronisations with nothing
but the three launches inside (`value`, `ms_per_step`), then K more steps with a HIP event between the
launches (`per_op_ms`, `roofline`), then each product K times back to back between one pair of events
(`per_op_back_to_back_ms`).

The JSON line also carries
  dense      same-problem dense bf16 GEMMs (torch.bmm over experts with the same
             FLOPs and weight bytes) timed in the same run, and our fraction of them; the same
             batched products at 256 and 384 rows per expert (`whole_tiles`) and the single
             GEMM of equal FLOPs (`frac_of_single_gemm`) beside them
  roofline   algorithmic bytes (or FLOPs) of the slowest of the three kernels over
             its mean duration from HIP events on the launch stream; `traffic` is read
             from the rocprofv3 counter summary under profiles/ (its source and commit are
             named; null with `traffic_stale` when the kernel sources have changed since)
  routing    the token routing on either side of the products on the same workload
             (sort into padded expert bins, gather, scatter), timed outside the step
  other_configs  per-product times on the other configurations of BASELINE.json with their
             dense comparators (--configs none leaves them out)
  cpu_baseline  the reference's dense-equivalent CPU path (to_dense + torch.matmul + mask, fp32)
             restated on the oracle's format helpers and timed on the host cores on a bounded,
             scaled-down sample of the same workload; the oracle's block walk beside it
"""
import argparse
import gc
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

TOKENS, EXPERTS, HIDDEN, FFN, BLOCK = 16384, 64, 1024, 4096, 128
PEAK_BF16_TFLOPS = 2500.0    # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0        # MI355X HBM3E


def build_workload(dev, seed=0):
    import stk_amd as stk
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(TOKENS, EXPERTS, generator=g)
    tokens_per_expert = torch.bincount(logits.argmax(dim=1), minlength=EXPERTS)
    block_rows_e = (tokens_per_expert + BLOCK - 1) // BLOCK
    nrows = int(block_rows_e.sum())
    # block-diagonal topology, transpose metadata included, from the library's one-launch builder
    padded_bins = torch.cumsum(block_rows_e * BLOCK, 0).to(torch.int32).to(dev)
    topo = stk.ops.dmoe_topology(padded_bins, BLOCK, nrows, FFN // BLOCK, dtype=torch.bfloat16)
    shape = topo.size()
    x = (torch.randn(shape[0], HIDDEN, generator=g) * 0.02).to(torch.bfloat16).to(dev)
    w1 = (torch.randn(HIDDEN, shape[1], generator=g) * 0.02).to(torch.bfloat16).to(dev)
    w2 = (torch.randn(shape[1], HIDDEN, generator=g) * 0.02).to(torch.bfloat16).to(dev)
    return topo, x, w1, w2, tokens_per_expert.numpy(), block_rows_e.numpy()


def algorithmic_bytes(nnz, rows, block_rows_e):
    """Compulsory HBM bytes per launch, every operand counted once."""
    blocks = nnz * BLOCK * BLOCK * 2
    weights = int((block_rows_e > 0).sum()) * HIDDEN * FFN * 2
    tokens = rows * HIDDEN * 2
    idx = nnz * 4
    return {
        "sdd": tokens + weights + blocks + idx,           # read x, W1 (touched experts); write h
        "dsd": blocks + weights + tokens + idx,           # read h, W2; write y
        "dds": tokens + blocks + HIDDEN * EXPERTS * FFN * 2 + idx + nnz * 4,   # read x, h; write dW1 (all columns)
    }


def time_events(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for s, e in ev:
        s.record()
        fn()
        e.record()
    torch.cuda.synchronize()
    return float(np.median([s.elapsed_time(e) for s, e in ev]))


def time_batch(fn, calls):
    """Mean time of `calls` launches issued back to back between one pair of events."""
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(calls):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / calls


def dense_comparators(rows, dev, steps, warmup):
    """Same-problem dense GEMMs: every expert gets rows/EXPERTS token rows, so FLOPs
    and weight bytes equal the block-sparse products'."""
    te = max(BLOCK, int(round(rows / EXPERTS / 8)) * 8)
    xe = (torch.randn(EXPERTS, te, HIDDEN, device=dev) * 0.02).bfloat16()
    w1 = (torch.randn(EXPERTS, HIDDEN, FFN, device=dev) * 0.02).bfloat16()
    w2 = (torch.randn(EXPERTS, FFN, HIDDEN, device=dev) * 0.02).bfloat16()
    he = torch.bmm(xe, w1)
    flops = 2.0 * EXPERTS * te * HIDDEN * FFN
    out = {"tokens_per_expert": te}
    fns = {"sdd": lambda: torch.bmm(xe, w1), "dsd": lambda: torch.bmm(he, w2), "dds": lambda: torch.bmm(xe.transpose(1, 2), he)}
    for k, fn in fns.items():
        out[k + "_like_ms"] = time_events(fn, steps, warmup)              # one pair of events per call, median
        out[k + "_like_back_to_back_ms"] = time_batch(fn, steps)          # one pair of events around `steps` calls
        out[k + "_like_tflops"] = flops / (out[k + "_like_ms"] * 1e-3) / 1e12
    # one plain GEMM with the same FLOPs (reads 1/64 of the weights): upper bound
    xa = (torch.randn(EXPERTS * te, HIDDEN, device=dev) * 0.02).bfloat16()
    wa = (torch.randn(HIDDEN, FFN, device=dev) * 0.02).bfloat16()
    ms = time_events(lambda: torch.mm(xa, wa), steps, warmup)
    out["single_gemm_tflops"] = flops / (ms * 1e-3) / 1e12
    del xe, he, xa
    # the same batched products with 256 and 384 token rows per expert: whole macro-tiles of the library's kernels
    # (the mean of the routed counts, 314 rows here, is a ragged size for them), so that the comparator is not one
    # the library happens to be slow at
    out["whole_tiles"] = {}
    for t in (256, 384):
        xt = (torch.randn(EXPERTS, t, HIDDEN, device=dev) * 0.02).bfloat16()
        ht = torch.bmm(xt, w1)
        f = 2.0 * EXPERTS * t * HIDDEN * FFN
        fns = {"sdd": lambda: torch.bmm(xt, w1), "dsd": lambda: torch.bmm(ht, w2), "dds": lambda: torch.bmm(xt.transpose(1, 2), ht)}
        out["whole_tiles"][str(t)] = {k + "_like_tflops": f / (time_events(fn, steps, warmup) * 1e-3) / 1e12 for k, fn in fns.items()}
        del xt, ht
    return out


def _blas_threads():
    try:
        from threadpoolctl import threadpool_info
        return int(max([p.get("num_threads", 1) for p in threadpool_info()] or [1]))
    except Exception:
        return os.cpu_count() or 1


def cpu_block_walk(tokens_per_expert, budget_s):
    """The CPU oracle's block walk (numpy port of the reference kernels) on the experts of the same workload,
    one expert at a time, cycling over them until the time budget is used."""
    from oracle import stk_oracle as O
    rng = np.random.RandomState(0)
    max_rows = int(max((int(t) + BLOCK - 1) // BLOCK * BLOCK for t in tokens_per_expert))
    # operands drawn once (outside the timed part); every expert takes its rows of x
    x_all = rng.randn(max_rows, HIDDEN).astype(np.float32) * 0.02
    w1 = rng.randn(HIDDEN, FFN).astype(np.float32) * 0.02
    w2 = rng.randn(FFN, HIDDEN).astype(np.float32) * 0.02
    done_flops, elapsed, used = 0.0, 0.0, 0
    while elapsed < budget_s:
        for e, t in enumerate(tokens_per_expert):
            if t == 0:
                continue
            topo = O.dmoe_topology([t], FFN, BLOCK)
            x = x_all[:topo.shape[0]]
            t0 = time.perf_counter()
            h = O.sdd(x, w1, topo)
            O.dsd(topo.shape, h, topo, False, w2)
            O.dds(x.T, topo.shape, h, topo, False)
            elapsed += time.perf_counter() - t0
            done_flops += 3 * len(topo.row_indices) * 2.0 * BLOCK * BLOCK * HIDDEN
            used += 1
            if elapsed >= budget_s:
                break
    return {"value": done_flops / elapsed / 1e12, "unit": "TFLOP/s", "cores": _blas_threads(),
            "sample": f"oracle sdd+dsd+dds (fp32 numpy block walk, one expert at a time) over {used} expert problems of the same "
                      f"topology ({used / EXPERTS:.1f} passes over the {EXPERTS} experts), {elapsed:.1f} s of CPU work"}


def cpu_baseline(tokens_per_expert, budget_s=8.0, group=4):
    """The reference's dense-equivalent path on the host cores: to_dense(S), torch.matmul in fp32, and the
    result masked to the topology (what stk's own tests compare its kernels with).  The whole topology as a
    dense matrix would hold 20096 x 262144 values, so the experts are taken `group` at a time: each problem is
    the block-diagonal topology of `group` consecutive experts with their real token counts, and the dense
    product does `group` times the nonzero FLOPs (the full topology would do 64 times).  Throughput is counted
    over the nonzero blocks only, as for the GPU.  The format helpers are the oracle's."""
    from oracle import stk_oracle as O
    g = torch.Generator().manual_seed(0)
    threads = torch.get_num_threads()
    cols = group * FFN
    max_rows = int(max(sum((int(t) + BLOCK - 1) // BLOCK * BLOCK for t in tokens_per_expert[e0:e0 + group]) for e0 in range(0, EXPERTS, group)))
    # operands drawn once (outside the timed part); every problem takes its rows of x
    x_all = torch.randn(max_rows, HIDDEN, generator=g) * 0.02
    w1 = torch.randn(HIDDEN, cols, generator=g) * 0.02
    w2 = torch.randn(cols, HIDDEN, generator=g) * 0.02
    done_flops, elapsed, problems = 0.0, 0.0, 0
    while elapsed < budget_s:
        for e0 in range(0, EXPERTS, group):
            counts = [int(t) for t in tokens_per_expert[e0:e0 + group]]
            if sum(counts) == 0:
                continue
            topo = O.dmoe_topology(counts, FFN, BLOCK)
            rows = topo.shape[0]
            x = x_all[:rows]
            blocks = torch.zeros(rows // BLOCK, cols // BLOCK)
            blocks[torch.from_numpy(topo.row_indices.astype(np.int64)), torch.from_numpy(topo.column_indices.astype(np.int64))] = 1.0
            mask = blocks.repeat_interleave(BLOCK, 0).repeat_interleave(BLOCK, 1)     # to_dense of a matrix of ones
            t0 = time.perf_counter()
            h_dense = torch.matmul(x, w1) * mask                             # sdd: dense product, masked to the topology
            y = torch.matmul(h_dense, w2)                                    # dsd: to_dense(h) @ W2
            dw1 = torch.matmul(x.t(), h_dense)                               # dds: x^T @ to_dense(h)
            elapsed += time.perf_counter() - t0
            del y, dw1
            done_flops += 3 * len(topo.row_indices) * 2.0 * BLOCK * BLOCK * HIDDEN
            problems += 1
            if elapsed >= budget_s:
                break
    out = {"value": done_flops / elapsed / 1e12, "unit": "TFLOP/s", "cores": int(threads), "kind": "port",
           "host_cpu_count": os.cpu_count(), "torch_num_threads": int(threads),
           "sample": f"dense-equivalent sdd+dsd+dds (torch.matmul fp32 on dense operands, sdd masked to the topology) over {problems} "
                     f"problems of {group} consecutive experts of the same topology with their real token counts (1/{EXPERTS // group} "
                     f"of the experts each, so the dense products do {group}x the nonzero FLOPs; the full topology would do "
                     f"{EXPERTS}x), {elapsed:.1f} s of CPU work; TFLOP/s counted over nonzero blocks"}
    out["block_walk"] = cpu_block_walk(tokens_per_expert, budget_s)
    return out


def routing_times(dev, steps, warmup, seed=0):
    """The step on either side of the products, on the same workload: the (token, expert) choices sorted into
    padded expert bins (stk_route, four short launches), the token rows copied into the padded layout
    (stk_padded_gather) and back (stk_padded_scatter).  Compulsory bytes: every row read once and written once."""
    import stk_amd as stk
    from stk_amd.backend import hip_kernels
    g = torch.Generator().manual_seed(seed)
    top = torch.randn(TOKENS, EXPERTS, generator=g).argmax(dim=1, keepdim=True).to(torch.int32).to(dev)
    r = stk.ops.route(top, EXPERTS, BLOCK)
    rows = r.row_slots.numel()
    x = (torch.randn(TOKENS, HIDDEN, generator=g) * 0.02).to(torch.bfloat16).to(dev)
    padded = hip_kernels.padded_gather(x, r.row_slots, 1)
    assert torch.equal(hip_kernels.padded_scatter(padded, r.slot_rows, 1), x)
    out = {"padded_rows": rows}
    out["route_ms"] = time_events(lambda: hip_kernels.route(top, EXPERTS, BLOCK, rows), steps, warmup)
    # the copies through the C ABI into outputs allocated once, back to back between one pair of events: a launch
    # of 12 us is otherwise timed together with the allocation and the host's launch latency (the *_op_ms figures)
    from stk_amd.backend import _lib
    lib, stream = _lib.load(), torch.cuda.current_stream().cuda_stream
    gathered, scattered = torch.empty_like(padded), torch.empty_like(x)

    def gather_launch():
        _lib.check(lib.stk_padded_gather(x.data_ptr(), TOKENS, HIDDEN, HIDDEN, r.row_slots.data_ptr(), None, 1, rows,
                                         gathered.data_ptr(), HIDDEN, _lib.STK_BF16, stream))

    def scatter_launch():
        _lib.check(lib.stk_padded_scatter(padded.data_ptr(), rows, HIDDEN, HIDDEN, r.slot_rows.data_ptr(), None, 1, TOKENS,
                                          scattered.data_ptr(), HIDDEN, _lib.STK_BF16, stream))

    def back_to_back(fn, calls=40):
        for _ in range(warmup):
            fn()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(calls):
            fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / calls

    for name, launch, op, nbytes in (
            ("gather", gather_launch, lambda: hip_kernels.padded_gather(x, r.row_slots, 1), (TOKENS + rows) * HIDDEN * 2 + rows * 4),
            ("scatter", scatter_launch, lambda: hip_kernels.padded_scatter(padded, r.slot_rows, 1), 2 * TOKENS * HIDDEN * 2 + TOKENS * 4)):
        ms = back_to_back(launch)
        out[name + "_ms"] = ms
        out[name + "_gbs"] = nbytes / (ms * 1e-3) / 1e9
        out[name + "_frac_of_hbm_peak"] = out[name + "_gbs"] / PEAK_HBM_GBS
        out[name + "_op_ms"] = time_events(op, steps, warmup)
    assert torch.equal(gathered, padded) and torch.equal(scattered, x)
    out["routed_forward"] = routed_forward_times(x, r, warmup)
    return out


def routed_forward_times(x, r, warmup, calls=20):
    """The forward pass of the routed layer on the benchmark workload, tokens in and tokens out, as the four launches
    gather -> sdd(gelu) -> dsd -> scatter and as the two launches that read and write the token rows in place
    (stk_sdd_gather, stk_dsd_scatter); outputs allocated once, `calls` passes back to back between one pair of events."""
    import stk_amd as stk
    from stk_amd.backend import hip_kernels
    dev, rows = x.device, r.row_slots.numel()
    topo = stk.ops.dmoe_topology(r.padded_bins, BLOCK, rows // BLOCK, FFN // BLOCK, dtype=torch.bfloat16)
    w1 = (torch.randn(HIDDEN, EXPERTS * FFN, device=dev) * 0.02).bfloat16()
    w2 = (torch.randn(EXPERTS * FFN, HIDDEN, device=dev) * 0.02).bfloat16()
    meta = (topo.offsets, topo.row_indices, topo.column_indices)
    walk = (topo.offsets, topo.row_indices, topo.column_indices, topo.offsets_t, topo.column_indices_t, topo.block_offsets_t)
    h = torch.empty_like(topo.data)
    padded_y, y4, y2 = torch.empty(rows, HIDDEN, dtype=x.dtype, device=dev), None, torch.empty_like(x)

    def four():
        nonlocal y4
        padded = hip_kernels.padded_gather(x, r.row_slots, 1)
        hip_kernels.sdd_fused(padded, w1, topo.size(), h, *meta, "gelu_tanh")
        hip_kernels.dsd(topo.size(), h, *walk, False, w2, padded_y)
        y4 = hip_kernels.padded_scatter(padded_y, r.slot_rows, 1)

    def two():
        assert hip_kernels.sdd_gather(x, r.row_slots, 1, w1, topo.size(), h, *meta, "gelu_tanh")
        assert hip_kernels.dsd_scatter(topo.size(), h, topo.offsets, topo.column_indices, topo.offsets_t, topo.column_indices_t, w2,
                                       r.row_slots, None, y2)

    def back_to_back(fn):
        for _ in range(warmup):
            fn()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(calls):
            fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / calls

    out = {"four_launches_ms": back_to_back(four), "two_launches_ms": back_to_back(two)}
    out["saved_us"] = (out["four_launches_ms"] - out["two_launches_ms"]) * 1e3
    out["bit_identical"] = bool(torch.equal(y4, y2))
    return out


def gradient_pair_times(topo, x, w1, calls):
    """The two operand gradients of sdd on the benchmark topology, dsd(dS, W1^T) and dds(x^T, dS), as the one launch of
    stk_dsd_dds and as two launches (stk_dsd without its workspace, stk_dds); `calls` times each, back to back."""
    from stk_amd.backend import hip_kernels
    ds = torch.empty_like(topo.data).normal_(0, 0.02)
    meta = (topo.offsets, topo.row_indices, topo.column_indices, topo.offsets_t, topo.column_indices_t, topo.block_offsets_t)
    dx, dw1 = torch.empty_like(x), torch.empty_like(w1)
    slicing, hip_kernels.SLICE_LAST_ROUND = hip_kernels.SLICE_LAST_ROUND, False

    def joint():
        hip_kernels.dsd_dds(topo.size(), ds, *meta, w1.t(), dx, x.t(), dw1)

    def two():
        hip_kernels.dsd(topo.size(), ds, *meta, False, w1.t(), dx)
        hip_kernels.dds(x.t(), topo.size(), ds, *meta, False, dw1)

    try:
        for fn in (joint, two):
            for _ in range(3):
                fn()
        out = {"joint_launch_ms": time_batch(joint, calls), "two_launches_ms": time_batch(two, calls)}
    finally:
        hip_kernels.SLICE_LAST_ROUND = slicing
    out["note"] = "dsd(dS,W1^T) + dds(x^T,dS): stk_dsd_dds against stk_dsd (no workspace) followed by stk_dds, back to back"
    return out


def dsd_gradient_pair_times(topo, x, w1, w2, calls):
    """The two gradients of dsd(h, W2) on the benchmark topology, sdd(dy, W2^T) on the pattern and dsd(h^T, dy), as the one
    launch of stk_sdd_dsd and as two launches (stk_sdd, stk_dsd without its workspace); `calls` times each, back to back."""
    from stk_amd.backend import hip_kernels
    import stk_amd as stk
    h = stk.ops.sdd(x, w1, topo).data
    dy = torch.empty_like(x).normal_(0, 0.02)
    meta = (topo.offsets, topo.row_indices, topo.column_indices, topo.offsets_t, topo.column_indices_t, topo.block_offsets_t)
    dh, dw2 = torch.empty_like(h), torch.empty_like(w2)
    rows, cols = topo.size()
    slicing, hip_kernels.SLICE_LAST_ROUND = hip_kernels.SLICE_LAST_ROUND, False

    def joint():
        hip_kernels.sdd_dsd((rows, cols), dy, w2.t(), dh, h, *meta, True, dy, dw2)

    def two():
        hip_kernels.sdd(dy, w2.t(), (rows, cols), dh, topo.offsets, topo.row_indices, topo.column_indices, block_order=topo.block_offsets_t)
        hip_kernels.dsd((cols, rows), h, *meta, True, dy, dw2)

    try:
        for fn in (joint, two):
            for _ in range(3):
                fn()
        out = {"joint_launch_ms": time_batch(joint, calls), "two_launches_ms": time_batch(two, calls)}
    finally:
        hip_kernels.SLICE_LAST_ROUND = slicing
    out["note"] = "sdd(dy,W2^T) + dsd(h^T,dy): stk_sdd_dsd against stk_sdd followed by stk_dsd (no workspace), back to back"
    return out


def _expert_choices(name, seed=0):
    """[tokens, top_k] int32 expert choices of the dMoE configurations of BASELINE.json."""
    g = torch.Generator().manual_seed(seed)
    if name == "4":      # Zipf(s = 1.2)-skewed popularity, top-2 by the Gumbel trick
        logp = -1.2 * torch.log(torch.arange(1, EXPERTS + 1, dtype=torch.float64))
        u = torch.rand(32768, EXPERTS, generator=g, dtype=torch.float64).clamp_min(1e-300)
        return (logp[None, :] - torch.log(-torch.log(u))).topk(2, dim=1).indices.to(torch.int32)
    if name == "5":      # the benchmark's routing, blocking 64
        return torch.randn(TOKENS, EXPERTS, generator=g).argmax(dim=1, keepdim=True).to(torch.int32)
    top = torch.randint(1, EXPERTS, (TOKENS,), generator=g, dtype=torch.int32)   # "5skew": expert 0 takes half of the tokens
    top[torch.randperm(TOKENS, generator=g)[:TOKENS // 2]] = 0
    return top[:, None]


def other_config(name, dev, steps, warmup):
    """Per-product times on another configuration of BASELINE.json ("2", "4", "5", "5skew"): the forward
    products and the four of the backward pass, with the same-problem dense comparator.  dMoE topologies
    come from the library's own routing and topology kernels."""
    import stk_amd as stk
    out = {}

    def timed(fn):
        # one pair of events around `steps` back-to-back calls: launches of tens of microseconds are otherwise
        # timed together with the host's launch latency
        for _ in range(warmup):
            fn()
        # (the better of two batches: a batch now and then contains one call that waits for the allocator to get
        # memory for a large output from the driver)
        best = float("inf")
        for _ in range(2):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            start.record()
            for _ in range(steps):
                fn()
            end.record()
            torch.cuda.synchronize()
            best = min(best, start.elapsed_time(end) / steps)
        return best

    def record(op, fn, flops):
        ms = timed(fn)
        out[op] = {"us": ms * 1e3, "tflops": flops / (ms * 1e-3) / 1e12}

    if name == "2":      # uniform random block sparsity, 4096 x 4096, 25 % of the 128-blocks
        np.random.seed(0)
        s = stk.random.mask(4096, 4096, 0.75, 128).to(dev)
        s = stk.Matrix(s.size(), s.data.bfloat16(), s.row_indices, s.column_indices, s.offsets, s.column_indices_t, s.offsets_t, s.block_offsets_t)
        a = (torch.randn(4096, 4096, device=dev) * 0.02).bfloat16()
        b = (torch.randn(4096, 4096, device=dev) * 0.02).bfloat16()
        flops = s.data.shape[0] * 2.0 * 128 * 128 * 4096
        out["workload"] = f"4096 x 4096, blocking 128, {s.data.shape[0]} of 1024 blocks (numpy seed 0), dense operands 4096 x 4096 bf16"
        record("sdd(a,b)", lambda: stk.ops.sdd(a, b, s), flops)
        record("dsd(s,b)", lambda: stk.ops.dsd(s, b), flops)
        record("dds(a,s)", lambda: stk.ops.dds(a, s), flops)
        record("dsd(s^T,b)", lambda: stk.ops.dsd(s.t(), b), flops)
        record("dds(a,s^T)", lambda: stk.ops.dds(a, s.t()), flops)
        ms = timed(lambda: torch.mm(a, b))
        out["dense 4096^3 scaled by the density"] = {"us": ms * 1e3 * 0.25, "tflops": 2.0 * 4096 ** 3 / (ms * 1e-3) / 1e12}
        return out

    hidden, ffn, blocking, dtype = (2048, 8192, 128, torch.bfloat16) if name == "4" else (HIDDEN, FFN, 64, torch.float16)
    top = _expert_choices(name).to(dev)
    r = stk.ops.route(top, EXPERTS, blocking)
    rows = r.row_slots.numel()
    topo = stk.ops.dmoe_topology(r.padded_bins, blocking, rows // blocking, ffn // blocking, dtype=dtype)
    tokens = (torch.randn(top.shape[0], hidden, device=dev) * 0.02).to(dtype)
    x = stk.ops.padded_gather(tokens, r)        # padding rows are zero, as in a layer
    w1 = (torch.randn(hidden, EXPERTS * ffn, device=dev) * 0.02).to(dtype)
    w2 = (torch.randn(EXPERTS * ffn, hidden, device=dev) * 0.02).to(dtype)
    h = stk.ops.sdd(x, w1, topo)
    nnz = h.data.shape[0]
    flops = nnz * 2.0 * blocking * blocking * hidden
    out["workload"] = (f"{top.shape[0]} tokens top-{top.shape[1]} over {EXPERTS} experts, padded to {blocking}: {rows} rows, {nnz} blocks, "
                       f"hidden {hidden}, ffn {ffn}, {str(dtype).split('.')[-1]}")
    record("sdd(x,W1)", lambda: stk.ops.sdd(x, w1, topo), flops)
    record("dsd(h,W2)", lambda: stk.ops.dsd(h, w2), flops)
    record("dds(x^T,h) dW1", lambda: stk.ops.dds(x.t(), h), flops)
    record("dsd(h^T,x) dW2", lambda: stk.ops.dsd(h.t(), x), flops)
    record("dsd(dh,W1^T) dx", lambda: stk.ops.dsd(h, w1.t()), flops)
    record("sdd(dy,W2^T) dh", lambda: stk.ops.sdd(x, w2.t(), topo), flops)
    te = max(blocking, int(round(rows / EXPERTS / 8)) * 8)
    xe = (torch.randn(EXPERTS, te, hidden, device=dev) * 0.02).to(dtype)
    we = (torch.randn(EXPERTS, hidden, ffn, device=dev) * 0.02).to(dtype)
    record("dense bmm (sdd-like, uniform experts)", lambda: torch.bmm(xe, we), 2.0 * EXPERTS * te * hidden * ffn)
    if name == "5skew":
        # the same problem as two dense launches: the expert with half of the tokens, and the other 63 with their mean
        counts = torch.bincount(top.reshape(-1).long(), minlength=EXPERTS)
        big = int((counts[0].item() + blocking - 1) // blocking * blocking)
        small = max(blocking, int(round((rows - big) / (EXPERTS - 1) / 8)) * 8)
        xb = (torch.randn(1, big, hidden, device=dev) * 0.02).to(dtype)
        xs = (torch.randn(EXPERTS - 1, small, hidden, device=dev) * 0.02).to(dtype)

        def both():
            torch.bmm(xb, we[:1])
            torch.bmm(xs, we[1:])
        record(f"dense bmm (sdd-like, 1 x {big} rows + {EXPERTS - 1} x {small} rows)", both, 2.0 * (big + (EXPERTS - 1) * small) * hidden * ffn)
    return out


# HBM bytes per launch on this workload come from rocprofv3 counters (FETCH_SIZE and WRITE_SIZE, scaled by what the
# same counters read for a plain copy of known size); the tracked summary of that run is read here, so that the
# figure in the JSON line is the one in the repository and names its source.  The summary records the digest of the
# kernel sources it was taken with (`kernel_sources_sha256:`, printed by `bench.py --kernel-sources-digest`) and the
# commit; when the sources in the tree differ, the counters describe other kernels than the ones just timed and the
# line carries no traffic at all rather than a stale one.
HBM_COUNTER_SUMMARY = os.path.join("profiles", "bench_dmoe_fwd_hbm_counters.txt")


def kernel_sources_digest(root=ROOT):
    """sha256 over the device sources of the library (stk_amd/csrc/*.hip and *.h, names and contents, sorted)."""
    import hashlib
    csrc = os.path.join(root, "stk_amd", "csrc")
    digest = hashlib.sha256()
    for name in sorted(n for n in os.listdir(csrc) if n.endswith((".hip", ".h"))):
        digest.update(name.encode() + b"\0")
        with open(os.path.join(csrc, name), "rb") as f:
            digest.update(f.read())
    return digest.hexdigest()


def counter_summary(path=None):
    """{'kernels': {name: bytes per launch}, 'sha256': ..., 'commit': ..., 'stale': bool, 'problem': text or None}."""
    path = path or os.path.join(ROOT, HBM_COUNTER_SUMMARY)
    info = {"kernels": {}, "sha256": None, "commit": None, "stale": True, "problem": None}
    try:
        with open(path) as f:
            for line in f:
                parts = line.split()
                if len(parts) >= 8 and parts[0].endswith("_kernel") and parts[0] not in info["kernels"]:
                    try:
                        info["kernels"][parts[0]] = float(parts[5]) * 1e6      # the 'total MB' column
                    except ValueError:
                        pass
                elif len(parts) == 2 and parts[0] == "kernel_sources_sha256:":
                    info["sha256"] = parts[1]
                elif len(parts) == 2 and parts[0] == "commit:":
                    info["commit"] = parts[1]
    except OSError as err:
        info["problem"] = f"{HBM_COUNTER_SUMMARY}: {err.strerror}"
        return info
    if info["sha256"] is None:
        info["problem"] = f"{HBM_COUNTER_SUMMARY} does not say which kernel sources it was taken with"
    elif info["sha256"] != kernel_sources_digest():
        info["problem"] = (f"{HBM_COUNTER_SUMMARY} was taken at commit {info['commit']} with other kernel sources than the tree holds: "
                           "its traffic figures are not reported (collect the counters again)")
    else:
        info["stale"] = False
    return info


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--preheat-ms", type=float, default=150.0,
                    help="milliseconds of untimed steps before the W warm-up steps: after an idle period the GPU takes about "
                         "40 ms of continuous work to reach its steady clocks (the first steps run up to 25 %% slower)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB -> 1 GiB elementwise kernel (torch.neg), the known-size reference for the HBM counters")
    ap.add_argument("--gradient-pair-only", action="store_true",
                    help="run only the gradient pairs of sdd and of dsd, each as one launch and as two (for the counter profiles)")
    ap.add_argument("--kernel-sources-digest", action="store_true",
                    help="print the digest of the kernel sources that a counter summary under profiles/ records, and exit")
    ap.add_argument("--configs", default="2,4,5,5skew",
                    help="comma-separated other configurations of BASELINE.json to time as well (2, 4, 5, 5skew); 'none' leaves them out")
    args = ap.parse_args()
    if args.kernel_sources_digest:
        print(kernel_sources_digest())
        return
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the block-sparse products have no multi-GPU path in this build (--gpus must be 1)")
    extra = [c for c in args.configs.split(",") if c and c != "none"]
    for name in extra:
        if name not in ("2", "4", "5", "5skew"):
            sys.exit(f"bench.py: unknown configuration {name!r} (2, 4, 5, 5skew, or none)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    import stk_amd as stk
    from stk_amd.backend import _lib
    _lib.load()

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    topo, x, w1, w2, tokens_per_expert, block_rows_e = build_workload(dev)
    nnz = topo.data.shape[0]
    rows = topo.size()[0]
    xt = x.t()
    flops_op = nnz * 2.0 * BLOCK * BLOCK * HIDDEN

    if args.gradient_pair_only:
        with torch.no_grad():
            print(json.dumps({"sdd_gradient_pair": gradient_pair_times(topo, x, w1, max(args.steps, 1)),
                              "dsd_gradient_pair": dsd_gradient_pair_times(topo, x, w1, w2, max(args.steps, 1))}))
        return

    names = ("sdd", "dsd", "dds")
    state = {}

    def run_sdd():
        state["h"] = stk.ops.sdd(x, w1, topo)

    def run_dsd():
        state["y"] = stk.ops.dsd(state["h"], w2)

    def run_dds():
        state["dw1"] = stk.ops.dds(xt, state["h"])

    products = (run_sdd, run_dsd, run_dds)

    def step(events=None):
        if events is not None:
            events[0].record()
        for i, product in enumerate(products):
            product()
            if events is not None:
                events[i + 1].record()

    if args.copy_calibration:
        # one elementwise kernel (torch.neg) that reads 1 GiB and writes 1 GiB in a single dispatch
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        dst = torch.neg(src)
        torch.cuda.synchronize()
        del src, dst

    aux_steps = max(10, args.steps // 2)

    def preheat(ms):
        """Untimed steps for `ms` milliseconds, without a pause at the end."""
        t0, n = time.perf_counter(), 0
        while (time.perf_counter() - t0) * 1e3 < ms:
            for _ in range(5):
                step()
            torch.cuda.synchronize()
            n += 5
        return n

    with torch.no_grad():
        step()
        # the collector of Python objects stays out of the timed passes (a full collection stops the launches
        # for tens of milliseconds, and the idle GPU drops its clocks); nothing in a step creates reference cycles
        gc.collect()
        gc.disable()
        # untimed: the step itself until the clocks have settled; the comparators then run at the same clocks
        preheat_steps = preheat(args.preheat_ms)
        dense = dense_comparators(rows, dev, aux_steps, 5)
        try:
            routing = routing_times(dev, aux_steps, 5)
        except Exception as exc:  # noqa: BLE001  (auxiliary: see other_configs below)
            routing = {"error": f"{type(exc).__name__}: {exc}"[:300]}
        preheat_steps += preheat(args.preheat_ms / 3)
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0

        # the same K steps again with an event between the launches: duration of each kernel inside the step
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
        t0 = time.perf_counter()
        for i in range(args.steps):
            step(evs[i])
        torch.cuda.synchronize()
        wall_with_events = time.perf_counter() - t0
        per_op_ms = {n: float(np.mean([e[i].elapsed_time(e[i + 1]) for e in evs])) for i, n in enumerate(names)}
        # and each product on its own, back to back
        per_op_b2b_ms = {n: time_batch(product, args.steps) for n, product in zip(names, products)}
        try:
            gradient_pair = gradient_pair_times(topo, x, w1, args.steps)
        except Exception as exc:  # noqa: BLE001
            gradient_pair = {"error": f"{type(exc).__name__}: {exc}"[:300]}
        try:
            dsd_gradient_pair = dsd_gradient_pair_times(topo, x, w1, w2, args.steps)
        except Exception as exc:  # noqa: BLE001
            dsd_gradient_pair = {"error": f"{type(exc).__name__}: {exc}"[:300]}
        gc.enable()

        others = {}
        for name in extra:
            # (an auxiliary measurement that fails - out of memory on a busy box, say - must not take the line with it)
            try:
                others[name] = other_config(name, dev, max(5, args.steps // 2), 3)
            except Exception as exc:  # noqa: BLE001
                others[name] = {"error": f"{type(exc).__name__}: {exc}"[:300]}
            torch.cuda.empty_cache()

    ms_per_step = wall * 1e3 / args.steps
    value = 3 * flops_op / (ms_per_step * 1e-3) / 1e12
    per_op_tflops = {n: flops_op / (per_op_ms[n] * 1e-3) / 1e12 for n in names}
    frac_dense = {n: per_op_tflops[n] / dense[n + "_like_tflops"] for n in names}
    frac_dense_b2b = {n: dense[n + "_like_back_to_back_ms"] / per_op_b2b_ms[n] * (flops_op / (2.0 * EXPERTS * dense["tokens_per_expert"] * HIDDEN * FFN))
                      for n in names}
    dense_total_ms = sum(dense[n + "_like_ms"] for n in names)
    dense_flops = 2.0 * EXPERTS * dense["tokens_per_expert"] * HIDDEN * FFN
    dense_step_tflops = 3 * dense_flops / (dense_total_ms * 1e-3) / 1e12

    bytes_op = algorithmic_bytes(nnz, rows, block_rows_e)
    dominant = max(names, key=lambda n: per_op_ms[n])
    ai = flops_op / bytes_op[dominant]
    if ai < PEAK_BF16_TFLOPS * 1e12 / (PEAK_HBM_GBS * 1e9):
        achieved = bytes_op[dominant] / (per_op_ms[dominant] * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": achieved / PEAK_HBM_GBS}
    else:
        achieved = per_op_tflops[dominant]
        roof = {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": achieved / PEAK_BF16_TFLOPS}
    kernel_names = {"sdd": "sdd_fused_kernel", "dsd": "dsd_sliced_kernel", "dds": "dds_fused_kernel"}
    counters = counter_summary()
    if counters["problem"]:
        print("bench.py: " + counters["problem"], file=sys.stderr)

    def traffic_of(n):
        return None if counters["stale"] else counters["kernels"].get(kernel_names[n])

    roof.update({"traffic": traffic_of(dominant), "traffic_source": HBM_COUNTER_SUMMARY, "traffic_commit": counters["commit"],
                 "traffic_stale": counters["stale"], "kernel": kernel_names[dominant], "avg_launch_ms": per_op_ms[dominant],
                 "algorithmic_bytes": bytes_op[dominant], "flops": flops_op,
                 "per_kernel": {kernel_names[n]: {"avg_launch_ms": per_op_ms[n], "algorithmic_bytes": bytes_op[n],
                                                  "frac_of_hbm_peak": bytes_op[n] / (per_op_ms[n] * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                                  "traffic": traffic_of(n)} for n in names}})
    if counters["problem"]:
        roof["traffic_note"] = counters["problem"]

    result = {
        "metric": "nonzero-block TFLOP/s for SDD/DSD/DDS; % of dense bf16 GEMM at dMoE shape",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "dmoe_ffn_fwd_topology: 16384 tokens top-1 over 64 experts (seed 0) padded to 128, hidden 1024, "
                               "ffn 4096, blocking 128; step = sdd(x,W1) + dsd(h,W2) + dds(x^T,h)",
                   "nnz_blocks": int(nnz), "padded_tokens": int(rows), "flops_per_product": flops_op},
        "timing": "value and ms_per_step: wall clock over the K steps between two synchronisations, nothing but the launches inside; "
                  "per_op_ms: a second pass of K steps with a HIP event between the launches (ms_per_step_with_events); "
                  "per_op_back_to_back_ms: each product K times between one pair of events; before the W warm-up steps the "
                  "dense comparators and the routing are timed and the step runs untimed for `preheat.ms` (clock ramp after idle)",
        "preheat": {"ms": args.preheat_ms, "steps": preheat_steps},
        "ms_per_step_with_events": wall_with_events * 1e3 / args.steps,
        "per_op_ms": per_op_ms, "per_op_tflops": per_op_tflops, "per_op_back_to_back_ms": per_op_b2b_ms,
        "frac_of_bf16_peak": value / PEAK_BF16_TFLOPS,
        "dense": dense, "frac_of_dense_per_op": frac_dense, "frac_of_dense_per_op_back_to_back": frac_dense_b2b,
        "frac_of_dense_step": value / dense_step_tflops,
        # against the one plain GEMM of the same FLOPs, which reads 1/64 of the weights (an upper bound, not the same problem)
        "frac_of_single_gemm": {n: per_op_tflops[n] / dense["single_gemm_tflops"] for n in names},
        "frac_of_dense_whole_tiles": {t: {n: per_op_tflops[n] / d[n + "_like_tflops"] for n in names} for t, d in dense["whole_tiles"].items()},
        "roofline": roof,
        "routing": routing,
        "sdd_gradient_pair": gradient_pair,
        "dsd_gradient_pair": dsd_gradient_pair,
    }
    if others:
        result["other_configs"] = others
    if not args.no_cpu_baseline:
        try:
            result["cpu_baseline"] = cpu_baseline(tokens_per_expert)
        except Exception as exc:  # noqa: BLE001  (the line with the GPU figures is worth more than no line)
            result["cpu_baseline"] = {"error": f"{type(exc).__name__}: {exc}"[:300]}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
