"""HIP graphs: the products captured once and replayed.

The launches of sdd / dsd / dds and of their backward passes take their stream from torch, allocate through torch
and keep no host-side state per call (the fusion plan and the dsd workspace exist after the first call on a
topology), so a chain of them can be captured into a graph.  Every replay is checked against the eager result on
the same inputs, with eager work and synchronisations between the replays.
"""
import numpy as np
import pytest
import torch

import stk_amd as stk
from oracle import stk_oracle as O
from tests import _util as U

pytestmark = pytest.mark.gpu
DEV = "cuda"
# enough blocks for the fused eight-wave kernels, the sliced last round of dsd and the joint gradient launches
_TOKENS = np.array([300, 0, 129, 384, 640, 128, 77, 256, 512, 1000, 40, 896, 512, 384, 640, 512])


def _case(hidden, ffn, blocking, dtype, seed):
    topo = O.dmoe_topology(_TOKENS, ffn, blocking)
    g = torch.Generator().manual_seed(seed)
    rows, cols = topo.shape
    x = (torch.randn(rows, hidden, generator=g) * 0.02).to(dtype).to(DEV)
    w1 = (torch.randn(hidden, cols, generator=g) * 0.02).to(dtype).to(DEV)
    w2 = (torch.randn(cols, hidden, generator=g) * 0.02).to(dtype).to(DEV)
    data = torch.empty(len(topo.row_indices), blocking, blocking, dtype=dtype, device=DEV)
    return topo, U.matrix_from_topology(stk, topo, data, DEV), x, w1, w2, g


def _fresh(like, g, scale=0.02):
    return (torch.randn(like.shape, generator=g) * scale).to(like.dtype).to(like.device)


@pytest.mark.parametrize("warm_up_on_capture_stream", [True, False])
@pytest.mark.parametrize("blocking,dtype", [(128, torch.bfloat16), (64, torch.float16)])
def test_forward_chain_replays_from_a_graph(blocking, dtype, warm_up_on_capture_stream):
    topo, tm, x, w1, w2, g = _case(1024, 4096, blocking, dtype, 41)

    def chain():
        h = stk.ops.sdd(x, w1, tm)
        return h.data, stk.ops.dsd(h, w2), stk.ops.dds(x.t(), h), stk.ops.dsd(h.t(), x)

    side = torch.cuda.Stream()
    if warm_up_on_capture_stream:
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            chain()
        torch.cuda.current_stream().wait_stream(side)
    else:
        chain()     # the plan and the workspace come from another stream than the one that captures
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        outs = chain()
    for replay in range(3):
        x.copy_(_fresh(x, g))
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = chain()
        torch.cuda.synchronize()
        for a, b, what in zip(got, want, ("sdd", "dsd", "dds", "dsd t")):
            assert torch.equal(a, b), (what, replay)
    U.assert_close(got[0], O.sdd(U.np32(x), U.np32(w1), topo), dtype, "sdd from the graph")
    U.assert_close(got[1], O.dsd(topo.shape, U.np32(got[0]), topo, False, U.np32(w2)), dtype, "dsd from the graph")


@pytest.mark.parametrize("joint_dsd_gradients", (False, True))
def test_forward_and_backward_replay_from_a_graph(joint_dsd_gradients, monkeypatch):
    from stk_amd.backend import autograd
    monkeypatch.setattr(autograd, "JOINT_DSD_GRADIENTS", joint_dsd_gradients)
    dtype = torch.bfloat16
    topo, tm, x, w1, w2, g = _case(1024, 4096, 128, dtype, 43)
    xs, w1s, w2s = (t.detach().clone().requires_grad_(True) for t in (x, w1, w2))
    a = _fresh(torch.empty(256, topo.shape[0], dtype=dtype, device=DEV), g).requires_grad_(True)
    dy = _fresh(x, g, 0.05)
    dz = _fresh(torch.empty(256, topo.shape[1], dtype=dtype, device=DEV), g, 0.05)
    leaves = (xs, w1s, w2s, a)

    def forward():
        h = stk.ops.sdd(xs, w1s, tm)
        # dsd's gradients are one launch or two launches on two streams, those of the dds (a third product on the same
        # values) run on two streams
        return stk.ops.dsd(h, w2s), stk.ops.dds(a, h)

    def step():
        y, z = forward()
        torch.autograd.backward((y, z), (dy, dz))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
            for t in leaves:
                t.grad = None
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step()
    grads = [t.grad for t in leaves]
    for replay in range(3):
        dy.copy_(_fresh(dy, g, 0.05))
        with torch.no_grad():
            xs.copy_(_fresh(xs, g))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in grads]
        want = torch.autograd.grad(forward(), leaves, (dy, dz))
        torch.cuda.synchronize()
        for p, q, what in zip(got, want, ("dx", "dW1", "dW2", "da")):
            assert torch.equal(p, q), (what, replay)
    assert all(torch.isfinite(t.float()).all() and t.float().abs().sum() > 0 for t in got)


def test_a_plan_built_inside_a_capture_serves_that_capture_only(monkeypatch):
    # no call on this topology before the capture: its plan is built by the captured launches and exists only in the
    # graph's replays; the captured dsd cuts its last round with a workspace of the graph's own
    from stk_amd.backend import hip_kernels
    dtype = torch.bfloat16
    topo, tm, x, w1, w2, g = _case(1024, 4096, 128, dtype, 45)
    other = U.matrix_from_topology(stk, topo, torch.empty_like(tm.data), DEV)     # the same pattern in tensors of its own
    stk.ops.dsd(stk.ops.sdd(x, w1, other), w2)                                    # the library is loaded and warm
    hip_kernels.release_workspaces()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        h = stk.ops.sdd(x, w1, tm)
        y = stk.ops.dsd(h, w2)
    assert not hip_kernels._dsd_workspaces
    # eager launches on the captured topology before any replay: the captured plan has never been computed
    h_eager = stk.ops.sdd(x, w1, tm)
    y_eager = stk.ops.dsd(h_eager, w2)
    h_other = stk.ops.sdd(x, w1, other)
    assert torch.equal(h_eager.data, h_other.data) and torch.equal(y_eager, stk.ops.dsd(h_other, w2))
    eager_workspaces = dict(hip_kernels._dsd_workspaces)
    for replay in range(2):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(h.data, h_eager.data) and torch.equal(y, y_eager), replay
    assert hip_kernels._dsd_workspaces == eager_workspaces          # the graph's workspace is not the device's
    with pytest.raises(RuntimeError, match="cannot be captured"):
        with torch.cuda.graph(torch.cuda.CUDAGraph(), stream=side):
            stk.ops.to_sparse(y, 128)


def test_replays_beside_eager_launches_and_other_graphs_share_no_workspace():
    # a captured dsd with a sliced last round owns its counters and partial-tile slots: replays on one stream next to
    # eager launches and to the replays of a second graph on other streams all give the eager result
    dtype = torch.bfloat16
    topo, tm, x, w1, w2, g = _case(1024, 4096, 128, dtype, 49)
    h = stk.ops.sdd(x, w1, tm)
    want = stk.ops.dsd(h, w2)
    want_t = stk.ops.dsd(h.t(), x)
    torch.cuda.synchronize()
    graphs, outs = [], []
    for product in (lambda: stk.ops.dsd(h, w2), lambda: stk.ops.dsd(h.t(), x)):
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            outs.append(product())
        graphs.append(graph)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for round_ in range(3):
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        for graph, stream in zip(graphs, streams):
            with torch.cuda.stream(stream):
                graph.replay()
        eager = stk.ops.dsd(h, w2)                      # on the default stream, with the device's workspace
        torch.cuda.synchronize()
        assert torch.equal(outs[0], want) and torch.equal(outs[1], want_t) and torch.equal(eager, want), round_


def test_a_routed_layer_replays_from_a_graph_with_new_expert_choices():
    # route -> gather -> topology -> sdd -> dsd -> weighted scatter and its backward pass in one graph: with the rows of the
    # padded layout fixed at their upper bound nothing is read back to the host, and the topology, its transpose
    # metadata and its fusion plan are rebuilt by every replay from the expert choices of that replay
    tokens, experts, blocking, hidden, ffn, top_k = 4096, 16, 128, 1024, 4096, 2
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(47)
    capacity = stk.ops.route_capacity(tokens * top_k, experts, blocking)
    top = torch.zeros(tokens, top_k, dtype=torch.int32, device=DEV)
    x = _fresh(torch.empty(tokens, hidden, dtype=dtype, device=DEV), g, 0.5).requires_grad_(True)
    w1 = _fresh(torch.empty(hidden, experts * ffn, dtype=dtype, device=DEV), g, 0.05).requires_grad_(True)
    w2 = _fresh(torch.empty(experts * ffn, hidden, dtype=dtype, device=DEV), g, 0.05).requires_grad_(True)
    weights = torch.rand(tokens, top_k, generator=g).to(DEV).requires_grad_(True)
    grad = _fresh(torch.empty(tokens, hidden, dtype=dtype, device=DEV), g, 1.0)
    leaves = (x, w1, w2, weights)

    def layer(padded_rows):
        r = stk.ops.route(top, experts, blocking, padded_rows)
        padded = stk.ops.padded_gather(x, r)
        topo = stk.ops.dmoe_topology(r.padded_bins, blocking, padded.shape[0] // blocking, ffn // blocking, dtype=dtype)
        return stk.ops.padded_scatter(stk.ops.dsd(stk.ops.sdd(padded, w1, topo), w2), r, weights)

    def choices(seed, skew):
        p = torch.arange(1, experts + 1, dtype=torch.float64).pow(-skew)
        picks = torch.multinomial(p.expand(tokens, experts), top_k, generator=torch.Generator().manual_seed(seed))
        return picks.to(torch.int32).to(DEV)

    top.copy_(choices(1, 0.0))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            layer(capacity).backward(grad)
            for t in leaves:
                t.grad = None
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out = layer(capacity)
        out.backward(grad)
    grads = [t.grad for t in leaves]
    for replay, skew in enumerate((0.0, 1.2, 3.0)):
        top.copy_(choices(10 + replay, skew))      # uniform, skewed, and nearly everything on two experts
        graph.replay()
        torch.cuda.synchronize()
        got = [out.clone()] + [t.clone() for t in grads]
        eager = layer(capacity)
        want = [eager] + list(torch.autograd.grad(eager, leaves, grad))
        exact = layer(None)                        # rows read back from the device: no surplus rows behind the last expert
        torch.cuda.synchronize()
        for p, q, what in zip(got, want, ("out", "dx", "dW1", "dW2", "dweights")):
            assert torch.equal(p, q), (what, replay)
        U.assert_close(got[0], U.np32(exact), dtype, "surplus rows change nothing")
        assert got[0].float().abs().sum() > 0
