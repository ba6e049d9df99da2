"""Shared helpers for the GPU parity tests: seeded inputs, oracle bridges, tolerances."""
import zlib

import numpy as np
import torch

from oracle import stk_oracle as O

# north-star tolerances against the fp32 oracle
TOL = {torch.bfloat16: dict(rtol=1e-2, atol=1e-2), torch.float16: dict(rtol=1e-2, atol=5e-3),
       # float32 values (not part of the north-star statement): sums of up to 2048 fp32 products, two summation orders
       torch.float32: dict(rtol=1e-4, atol=1e-5)}


# Scale-free bounds beside them.  The absolute tolerances above exceed the size of the outputs when the
# operands are ~N(0, 0.02), so a result can lose a whole K-tile and still pass them; these cannot be passed
# that way.  A result rounded once to 16 bits from an exact sum is off by at most half an ulp, i.e. 2^-8
# (bfloat16) or 2^-11 (float16) of its own size:
#   max |got - want|  <=  MAX_REL * max |want|       (2x / 4x half an ulp of the largest element)
#   ||got - want||_F  <=  RMS_REL * ||want||_F       (rounding noise is about 0.4 x 2^-8 resp. 2^-11 of the norm)
MAX_REL = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -9, torch.float32: 2.0 ** -16}
RMS_REL = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -10, torch.float32: 2.0 ** -18}


def stable_seed(*args):
    """Seed derived from the arguments that is the same in every process (Python's hash() of strings is not)."""
    return zlib.crc32(repr(tuple(str(a) for a in args)).encode()) % (2 ** 31)


def np32(t):
    return t.detach().float().cpu().numpy()


def topo_of(m):
    """stk_amd.Matrix -> oracle Topology (numpy copies of the metadata)."""
    f = lambda t: t.detach().cpu().numpy()
    return O.Topology(tuple(m._size) if not m._transposed else (m._size[1], m._size[0]), m.blocking,
                      f(m.row_indices), f(m.column_indices), f(m.offsets),
                      f(m.column_indices_t), f(m.offsets_t), f(m.block_offsets_t))


def assert_close(got, want, dtype, what=""):
    got = np32(got) if isinstance(got, torch.Tensor) else np.asarray(got, dtype=np.float32)
    want = np.asarray(want, dtype=np.float32)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    tol = TOL[dtype]
    bad = ~np.isclose(got, want, **tol)
    if bad.any():
        idx = np.argwhere(bad)[0]
        raise AssertionError(f"{what}: {bad.sum()} of {bad.size} elements outside rtol={tol['rtol']} atol={tol['atol']}; "
                             f"first at {tuple(idx)}: got {got[tuple(idx)]} want {want[tuple(idx)]}")


def assert_close_scaled(got, want, dtype, what="", tol=None):
    """The north-star tolerance (or `tol`) and the two scale-free bounds, for tensors on any device (computed
    there, so that full-size results need not travel to the host).  `want` is the fp32 reference."""
    got = got.detach().float() if isinstance(got, torch.Tensor) else torch.as_tensor(np.asarray(got, dtype=np.float32))
    want = want.detach().float() if isinstance(want, torch.Tensor) else torch.as_tensor(np.asarray(want, dtype=np.float32))
    want = want.to(got.device)
    assert got.shape == want.shape, (what, tuple(got.shape), tuple(want.shape))
    if got.numel() == 0:
        return
    tol = tol or TOL[dtype]
    bad = ~torch.isclose(got, want, **tol)
    if bool(bad.any()):
        idx = tuple(int(i) for i in bad.nonzero()[0])
        raise AssertionError(f"{what}: {int(bad.sum())} of {bad.numel()} elements outside rtol={tol['rtol']} atol={tol['atol']}; "
                             f"first at {idx}: got {float(got[idx])} want {float(want[idx])}")
    err = got - want
    scale = float(want.abs().max())
    worst = float(err.abs().max())
    assert worst <= MAX_REL[dtype] * scale, f"{what}: max |got - want| = {worst:.3e} exceeds {MAX_REL[dtype]:.2e} x max |want| = {scale:.3e}"
    rel = float(torch.linalg.vector_norm(err.double()) / torch.linalg.vector_norm(want.double()).clamp_min(1e-300))
    assert rel <= RMS_REL[dtype], f"{what}: ||got - want|| / ||want|| = {rel:.3e} exceeds {RMS_REL[dtype]:.2e}"


def assert_topology_equal(m, topo, what=""):
    """Bit-exact comparison of every metadata array (values and dtypes)."""
    for name in ("row_indices", "column_indices", "offsets", "column_indices_t", "offsets_t", "block_offsets_t"):
        got = getattr(m, name).detach().cpu().numpy()
        want = getattr(topo, name)
        assert got.dtype == want.dtype, (what, name, got.dtype, want.dtype)
        assert np.array_equal(got, want), (what, name)


def sparse_from_dense(stk, dense_cpu, blocking, device):
    """Builds the Matrix on the host like the reference's tests, then moves it."""
    return stk.ops.to_sparse(dense_cpu, blocking).to(device)


def dmoe_tokens_top1(tokens, experts, seed):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(tokens, experts, generator=g)
    return torch.bincount(logits.argmax(dim=1), minlength=experts).numpy()


def dmoe_tokens_zipf_top2(tokens, experts, seed, s=1.2):
    g = torch.Generator().manual_seed(seed)
    logp = -s * torch.log(torch.arange(1, experts + 1, dtype=torch.float64))
    u = torch.rand(tokens, experts, generator=g, dtype=torch.float64).clamp_min(1e-300)
    gumbel = -torch.log(-torch.log(u))
    top2 = (logp[None, :] + gumbel).topk(2, dim=1).indices
    return torch.bincount(top2.reshape(-1), minlength=experts).numpy()


def dmoe_tokens_skewed(tokens, experts, seed):
    """Expert 0 takes half of the tokens, the rest spread uniformly over the others."""
    g = torch.Generator().manual_seed(seed)
    rest = torch.randint(1, experts, (tokens - tokens // 2,), generator=g)
    counts = torch.bincount(rest, minlength=experts)
    counts[0] = tokens // 2
    return counts.numpy()


def matrix_from_topology(stk, topo, data, device):
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    return stk.Matrix(torch.Size(topo.shape), data, t(topo.row_indices), t(topo.column_indices), t(topo.offsets),
                      t(topo.column_indices_t), t(topo.offsets_t), t(topo.block_offsets_t))
