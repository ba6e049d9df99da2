"""CPU tier: the C ABI library, the host-side mirror of the reference interface
and the host format path.  No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import stk_amd as stk
from oracle import stk_oracle as O
from stk_amd.backend import _lib
from tests.test_oracle import FORMAT_CASES, KAT

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "stk_amd.h")).read()
    declared = set(re.findall(r"\b(stk_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    assert os.path.exists(_lib.LIB_PATH), "build the library first: make -C stk_amd/csrc"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert _lib.load().stk_abi_version() == _lib.ABI_VERSION
    assert _lib.load().stk_transpose_meta_workspace_bytes(1000) >= 4 * 4 * 1000


def test_status_codes_without_touching_the_gpu():
    lib = _lib.load()
    # argument validation happens before any HIP call
    rc = lib.stk_sdd(None, 1, 1, None, 1, 1, 100, 64, 128, None, None, None, None, None, 1, 128, _lib.STK_BF16, _lib.STK_I16, None, None)
    assert rc == _lib.STK_ERR_DIMS and b"incompatible dimensions" in lib.stk_last_error()
    rc = lib.stk_sdd(None, 1, 1, None, 1, 1, 128, 64, 128, None, None, None, None, None, 1, 32, _lib.STK_BF16, _lib.STK_I16, None, None)
    assert rc == _lib.STK_ERR_UNSUPPORTED
    with pytest.raises(AssertionError):
        _lib.check(_lib.STK_ERR_DIMS)
    with pytest.raises(NotImplementedError):
        _lib.check(_lib.STK_ERR_UNSUPPORTED)
    rc = lib.stk_transpose_meta(None, None, 10, 4, _lib.STK_I16, None, None, None, None, 0, None)
    assert rc == _lib.STK_ERR_WORKSPACE


def _simulated_launch(tiles, length, units, k):
    """Order-of-dispatch model behind stk_dsd_tail_slices, item by item: workgroups start in order, each on
    the compute unit that is free first; the tiles of the last round are cut into k slices."""
    import heapq
    kinds = [length, 0.75 * length, 0.58 * length]
    start, seam = 4.0, 2.0
    items = [d for d, n in zip(kinds, tiles) for _ in range(n)]
    whole = (len(items) - 1) // units * units
    work = [d + start for d in items[:whole]]
    tail = items[whole:]
    for _ in range(k):
        work += [d + start if k == 1 else d / k + start + seam for d in tail]
    free = [0.0] * units
    end = 0.0
    for d in work:
        t = heapq.heappop(free) + d
        end = max(end, t)
        heapq.heappush(free, t)
    return end


@pytest.mark.parametrize("tiles,length", [((140, 232, 0), 32), ((256, 0, 0), 32), ((128, 0, 0), 32), ((300, 0, 0), 32),
                                          ((0, 0, 104), 71), ((0, 0, 208), 71), ((64, 48, 12), 32), ((32, 0, 0), 256),
                                          ((1000, 2000, 0), 32), ((600, 300, 0), 32), ((140, 232, 0), 4), ((0, 0, 0), 8), ((7, 5, 3), 1)])
def test_dsd_tail_slice_rule_matches_an_item_by_item_simulation(tiles, length):
    # the library groups compute units with equal free times; a plain event simulation must pick the same k
    units = 256
    got = _lib.load().stk_dsd_tail_slices(*tiles, float(length), units)
    considered = 0 < sum(tiles) <= 4 * units      # more rounds than that: never cut
    ends = {k: _simulated_launch(tiles, float(length), units, k) for k in (1, 2, 3, 4)} if considered else {1: 0.0}
    want = 1
    for k in (2, 3, 4):
        if considered and ends[k] < ends[want] - 1e-4 and ends[k] < 0.98 * ends[1]:
            want = k
    assert got == want, (got, want, ends)


def test_host_tensors_go_to_the_host_library_and_gpu_only_operations_refuse_them():
    m = stk.ops.to_sparse(torch.ones(128, 128, dtype=torch.float16), 128)
    ones = torch.ones(128, 128, dtype=torch.float16)
    assert torch.equal(stk.ops.dsd(m, ones), torch.full((128, 128), 128.0, dtype=torch.float16))
    assert torch.equal(stk.ops.dds(ones, m), torch.full((128, 128), 128.0, dtype=torch.float16))
    assert torch.equal(stk.ops.sdd(ones, ones, m).data, torch.full((1, 128, 128), 128.0, dtype=torch.float16))
    # what exists on the GPU only says so
    from stk_amd.backend import hip_kernels as hk
    meta = (m.offsets, m.row_indices, m.column_indices, m.offsets_t, m.column_indices_t, m.block_offsets_t)
    with pytest.raises(RuntimeError, match="GPU"):
        hk.dsd_dds((128, 128), m.data, *meta, ones, torch.empty_like(ones), ones, torch.empty_like(ones))
    with pytest.raises(RuntimeError, match="GPU"):
        stk.ops.route(torch.zeros(4, 1, dtype=torch.int32), 2, 128)
    with pytest.raises(RuntimeError, match="GPU"):
        stk.ops.dmoe_topology(torch.tensor([128], dtype=torch.int32), 128, 1, 1)


def test_config1_known_answer_host_path():
    np.random.seed(0)
    m = stk.random.mask(1024, 1024, 0.5, 128)
    m.validate()
    for k, want in KAT.items():
        assert getattr(m, k).tolist() == want, k
    assert m.offsets_t.dtype == torch.int32 and m.block_offsets_t.dtype == torch.int32 and m.column_indices_t.dtype == torch.int16
    assert stk.ops.row_indices(m.size(), m.data, m.offsets, m.column_indices).tolist() == KAT["row_indices"]


@pytest.mark.parametrize("rows,cols,sparsity,blocking", FORMAT_CASES)
def test_host_format_matches_oracle(rows, cols, sparsity, blocking):
    np.random.seed(rows + 7 * cols)
    torch.manual_seed(0)
    mask = stk.random.dense_mask(rows, cols, sparsity, blocking)
    assert mask.shape == (rows, cols) and mask.dtype == torch.float32
    nnz = round(rows // blocking * cols // blocking * (1 - sparsity)) * blocking ** 2
    assert torch.count_nonzero(mask).item() == nnz
    x = (torch.randn(rows, cols) * mask).half()
    m = stk.ops.to_sparse(x, blocking)
    m.validate()
    assert m.nnz == nnz and m.dim() == 2 and tuple(m.size()) == (rows, cols)
    data, topo = O.to_sparse(x.numpy(), blocking)
    assert np.array_equal(m.data.numpy(), data)
    for k in KAT:
        assert np.array_equal(getattr(m, k).numpy(), getattr(topo, k)), k
        assert getattr(m, k).numpy().dtype == getattr(topo, k).dtype, k
    assert torch.equal(stk.ops.to_dense(m), x)
    sm = stk.random.mask(rows, cols, sparsity, blocking)
    sm.validate()
    assert sm.nnz == nnz and bool(torch.logical_or(sm.data == 0, sm.data == 1).all())


def test_matrix_surface():
    np.random.seed(3)
    m = stk.random.mask(64, 96, 0.5, 16)
    t = m.t()
    assert tuple(t.size()) == (96, 64) and not t.is_contiguous() and m.is_contiguous()
    assert t.data.data_ptr() == m.data.data_ptr() and t.t().is_contiguous()
    assert m.blocking == 16 and m.nnz == m.data.numel() and m.dtype == torch.float16 and not m.is_cuda
    c = m.clone()
    assert c.data.data_ptr() != m.data.data_ptr() and torch.equal(c.block_offsets_t, m.block_offsets_t)
    v = m.view(2, 32, 96)
    assert tuple(v.size()) == (2, 32, 96) and tuple(stk.ops.to_dense(v).shape) == (2, 32, 96)
    with pytest.raises(ValueError):
        m.view(96, 64)
    with pytest.raises(ValueError):
        v.t()
    with pytest.raises(ValueError):
        m.contiguous()
    assert len(m.state_dict()) == 0
    m.requires_grad_(True)
    assert m.requires_grad
    stk.ops.sum(stk.ops.mul(m, m)).backward()
    assert torch.equal(m.grad.data, 2 * m.data) and tuple(m.t().grad.size()) == (96, 64)
    o = stk.ops.ones_like(m)
    assert bool((o.data == 1).all()) and torch.equal(o.column_indices_t, m.column_indices_t)
    r = stk.random.randn((2, 32, 96), 0.5, 16)
    assert tuple(r.size()) == (2, 32, 96)


def test_index_overflow_guard_and_validation_errors():
    data = torch.zeros(1, 2, 2, dtype=torch.float16)
    idx = torch.zeros(1, dtype=torch.int16)
    big = 2 * 32768
    with pytest.raises(ValueError, match="16-bit"):
        stk.Matrix((big, 2), data, idx, idx, torch.zeros(big // 2 + 1, dtype=torch.int32))
    ok = stk.Matrix((2, 2), data, idx, idx, torch.tensor([0, 1], dtype=torch.int32))
    ok.validate()
    for bad in (stk.Matrix((2, 2), data.float(), idx, idx, torch.tensor([0, 1], dtype=torch.int32)),
                stk.Matrix((2, 2), data, idx.int(), idx.int(), torch.tensor([0, 1], dtype=torch.int32)),
                stk.Matrix((2, 2), data, idx, idx, torch.tensor([0, 1], dtype=torch.int64)),
                stk.Matrix((3, 2), data, idx, idx, torch.tensor([0, 1], dtype=torch.int32)),
                stk.Matrix((2, 2), data, idx, idx, torch.tensor([0, 1, 1], dtype=torch.int32))):
        with pytest.raises(ValueError):
            bad.validate()


def test_autocast_wrappers_cast_only_eligible_tensors():
    from stk_amd.backend import autocast
    seen = {}

    @autocast.custom_fwd
    def fwd(a, b, c):
        seen["dtypes"] = (a.dtype, b.dtype, c)
        seen["inside"] = torch.is_autocast_enabled()
        return a

    x = torch.ones(2)
    fwd(x, x.double(), 3)
    assert seen["dtypes"] == (torch.float32, torch.float64, 3)      # autocast off: untouched
    with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
        fwd(x, x.double(), 3)
    assert seen["dtypes"] == (torch.float32, torch.float64, 3)      # host tensors are never cast
    assert seen["inside"] is False


def test_bench_rejects_what_it_does_not_measure():
    """bench.py is a one-GPU measurement: more GPUs and unknown configurations end with a message, before any GPU work."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for flags, text in ((["--gpus", "2"], "one GPU"), (["--configs", "2,9"], "unknown configuration '9'")):
        run = subprocess.run([sys.executable, os.path.join(root, "bench.py")] + flags, capture_output=True, text=True, timeout=300)
        assert run.returncode != 0
        assert text in run.stderr, run.stderr


def test_bench_reports_no_traffic_from_counters_taken_with_other_kernel_sources(tmp_path):
    # roofline.traffic comes from a tracked counter summary; it is only reported while the kernel sources are the ones
    # the counters were taken with
    import bench
    digest = bench.kernel_sources_digest()
    assert len(digest) == 64 and digest == bench.kernel_sources_digest()
    row = "  dds_fused_kernel       100779.6     524670.4     206.4      537.3      743.7            742.7    1.00\n"
    fresh = tmp_path / "fresh.txt"
    fresh.write_text("commit: abc1234\nkernel_sources_sha256: " + digest + "\n" + row)
    info = bench.counter_summary(str(fresh))
    assert not info["stale"] and info["problem"] is None and info["commit"] == "abc1234"
    assert info["kernels"]["dds_fused_kernel"] == pytest.approx(743.7e6)
    stale = tmp_path / "stale.txt"
    stale.write_text("commit: abc1234\nkernel_sources_sha256: " + "0" * 64 + "\n" + row)
    info = bench.counter_summary(str(stale))
    assert info["stale"] and "other kernel sources" in info["problem"]
    unmarked = tmp_path / "unmarked.txt"
    unmarked.write_text(row)
    assert bench.counter_summary(str(unmarked))["stale"]
    assert bench.counter_summary(str(tmp_path / "missing.txt"))["stale"]


def test_dsd_workspace_choice():
    # captured launches never touch the device's shared workspace; eager launches share it and serialise across streams
    from stk_amd.backend.hip_kernels import _workspace_choice
    assert _workspace_choice(True, None, 5) == "private"
    assert _workspace_choice(True, 5, 5) == "private"       # even on the stream that owns the shared one: replays may run elsewhere
    assert _workspace_choice(True, 7, 5) == "private"
    assert _workspace_choice(False, None, 5) == "create"
    assert _workspace_choice(False, 5, 5) == "shared"
    assert _workspace_choice(False, 7, 5) == "wait"


def test_fusion_plan_cache_is_tied_to_the_index_tensors_it_was_built_from():
    # the plan of a topology is cached on its offsets tensor; the entry holds the other index tensors, so that
    # a new tensor at a recycled address, an in-place change or a tensor without a version counter miss
    from stk_amd.backend import hip_kernels as hk
    offsets = torch.arange(0, 20, 4, dtype=torch.int32)
    ci = torch.tensor([0, 1, 2, 3] * 4, dtype=torch.int16)
    ot, cit = torch.arange(0, 20, 4, dtype=torch.int32), torch.tensor([0, 1, 2, 3] * 4, dtype=torch.int16)
    plan = object()
    assert hk._plan_cache_get((offsets, ci), 128) is None
    assert hk._plan_cache_put((offsets, ci, ot, cit), 128, plan, 7, None, 0)
    assert hk._plan_cache_get((offsets, ci, ot, cit), 128)[1] is plan
    assert hk._plan_cache_get((offsets, ci), 128)[1] is plan               # a request without the transpose metadata
    assert hk._plan_cache_get((offsets, ci, ot, cit), 64) is None          # another blocking
    # the column indices replaced by an equal-sized tensor: a miss, and the old tensor is still alive in the entry
    held = offsets._stk_plan[0][0]
    assert held is ci
    address = ci.data_ptr()
    del ci
    other = torch.tensor([3, 2, 1, 0] * 4, dtype=torch.int16)
    assert held.data_ptr() == address and other.data_ptr() != address
    assert hk._plan_cache_get((offsets, other, ot, cit), 128) is None
    # modified in place: the version counter moves
    assert hk._plan_cache_get((offsets, held, ot, cit), 128)[1] is plan
    held[0] = 5
    assert hk._plan_cache_get((offsets, held, ot, cit), 128) is None
    # a plan built without the transpose metadata does not serve a request with it
    assert hk._plan_cache_put((offsets, held), 128, plan, 7, None, 0)
    assert hk._plan_cache_get((offsets, held, ot, cit), 128) is None
    # tensors made under inference mode keep no version counter: never cached, and asking does not raise
    with torch.inference_mode():
        frozen = torch.arange(0, 20, 4, dtype=torch.int32)
        fci = torch.zeros(16, dtype=torch.int16)
    assert not hk._plan_cache_put((frozen, fci), 128, plan, 7, None, 0)
    assert hk._plan_cache_get((frozen, fci), 128) is None
