"""stk_route_static: the routing entry point that allocates nothing (its per-tile table lives in a device array
owned by the library) against stk_route with a caller-supplied workspace, through the C ABI.

Both run the same three launches, so every output must agree bit for bit.  Two calls in a row, the second
with a smaller input, show that nothing read by a call is left over from the call before it; both are also
checked against the CPU oracle.  Sizes beyond the built-in table are refused with STK_ERR_WORKSPACE.
"""
import numpy as np
import pytest
import torch

from oracle import stk_oracle as O
from stk_amd.backend import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda"
_OUTPUTS = ("indices", "bin_ids", "bins", "padded_bins", "slot_rows", "row_slots")


def _outputs(slots, experts, padded_rows, fill):
    """Output arrays pre-filled with a value that no routing writes, so that an element left untouched shows."""
    sizes = dict(indices=slots, bin_ids=slots, bins=experts, padded_bins=experts, slot_rows=slots, row_slots=padded_rows)
    return {name: torch.full((max(sizes[name], 1),), fill, dtype=torch.int32, device=DEV)[:sizes[name]] for name in _OUTPUTS}


def _route_both(top, experts, blocking):
    """(outputs of stk_route, outputs of stk_route_static) for the same choices, launched on torch's current stream."""
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    slots = top.numel()
    padded_rows = (slots + experts * (blocking - 1)) // blocking * blocking
    ws_bytes = lib.stk_route_workspace_bytes(slots, experts)
    ws = torch.full((max(ws_bytes, 4) // 4,), -7, dtype=torch.int32, device=DEV)
    a, b = _outputs(slots, experts, padded_rows, -3), _outputs(slots, experts, padded_rows, -5)
    ptr = lambda t: t.data_ptr() if t.numel() else None
    _lib.check(lib.stk_route(ptr(top), slots, experts, blocking, padded_rows, *(ptr(a[n]) for n in _OUTPUTS), ws.data_ptr(), ws_bytes, stream))
    before = torch.cuda.memory_allocated()
    _lib.check(lib.stk_route_static(ptr(top), slots, experts, blocking, padded_rows, *(ptr(b[n]) for n in _OUTPUTS), stream))
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    return a, b, padded_rows


def _check(top_host, experts, blocking, what):
    top = top_host.to(torch.int32).reshape(-1).to(DEV)
    a, b, padded_rows = _route_both(top, experts, blocking)
    want = O.route(top_host.numpy().reshape(-1, 1), experts, blocking, padded_rows=padded_rows)
    for name in _OUTPUTS:
        assert torch.equal(a[name], b[name]), f"{what}: {name} differs between stk_route and stk_route_static"
        assert np.array_equal(b[name].cpu().numpy(), getattr(want, name)), f"{what}: {name} differs from the oracle"


def test_route_static_matches_route_on_two_calls_in_a_row():
    g = torch.Generator().manual_seed(11)
    # config 4's size (65536 slots over 64 experts, 256 tiles), then a much smaller input on fewer experts:
    # the second call reads a part of the table the first one filled
    logp = -1.2 * torch.log(torch.arange(1, 65, dtype=torch.float64))
    u = torch.rand(32768, 64, generator=g, dtype=torch.float64).clamp_min(1e-300)
    first = (logp[None, :] - torch.log(-torch.log(u))).topk(2, dim=1).indices
    _check(first, 64, 128, "first call")
    second = torch.randint(0, 5, (777,), generator=g)
    _check(second, 5, 64, "second, smaller call")
    # and again larger, with more experts than before and an empty one
    third = torch.randint(0, 200, (20000,), generator=g)
    third[third == 17] = 18
    _check(third, 200, 128, "third call")
    _check(torch.zeros(0, dtype=torch.int64), 3, 128, "no slots")


def test_route_static_refuses_what_its_table_cannot_hold():
    lib = _lib.load()
    slots, experts = 1 << 20, 1024          # 4096 tiles x 1024 experts = 4 Mi entries > the built-in 1 Mi
    assert lib.stk_route_workspace_bytes(slots, experts) > 4 * (1 << 20)
    top = torch.zeros(8, dtype=torch.int32, device=DEV)
    rc = lib.stk_route_static(top.data_ptr(), slots, experts, 128, slots + experts * 128, top.data_ptr(), top.data_ptr(), top.data_ptr(),
                              top.data_ptr(), top.data_ptr(), top.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.STK_ERR_WORKSPACE and b"stk_route_static" in lib.stk_last_error()
    torch.cuda.synchronize()
    # the largest size of the routing tests that fits: 2^20 slots over 256 experts fill the table exactly
    g = torch.Generator().manual_seed(12)
    _check(torch.randint(0, 256, (1 << 20,), generator=g), 256, 128, "table filled exactly")
