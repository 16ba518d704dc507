"""GPU check of ``opmx_moe_select_static``: MoeSelect for callers that cannot allocate.

It is ``opmx_moe_select`` with the library's own scratch array in place of a caller's
workspace, so both are called through the C ABI on the same inputs and every output must match
bit for bit (integers, weights and row copies alike: the kernels are the same).  Two calls in a
row share the array, the second one smaller than the first, so stale contents of the first
call sit behind the part the second one uses; the oracle checks the second call as well.
Further down: the two calls enqueued back to back with no synchronisation between them, the
allocator's byte count across a call, and the call captured into a HIP graph and replayed.
"""
import pytest
import torch

from _util import dev, tie_heavy_scores
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu

# T, H, E, k, dtype: all beyond 256 tokens, where the kernels use the scratch memory
CALLS = [
    (5000, 256, 64, 8, torch.bfloat16),    # 2.6 KB of chunk histograms + 160 KB of ids
    (700, 512, 8, 2, torch.float16),       # smaller: re-uses the front of the array
]


def _outputs(X, s, E, k, with_ids):
    T, H = X.shape
    d = X.device
    xe = torch.full((T * k, H), float("nan"), dtype=X.dtype, device=d)
    w = torch.full((T, k), float("nan"), dtype=s.dtype, device=d)
    inv = torch.full((T * k,), -7, dtype=torch.int64, device=d)
    off = torch.full((E + 1,), -7, dtype=torch.int64, device=d)
    ids = torch.full((T, k), -7, dtype=torch.int32, device=d) if with_ids else None
    return xe, w, inv, off, ids


def _enqueue_static(X, s, E, k, outs):
    """opmx_moe_select_static on torch's current stream into preallocated outputs; no synchronisation."""
    from torch_function import _lib
    L = _lib.lib()
    T, H = X.shape
    xe, w, inv, off, ids = outs
    rc = L.opmx_moe_select_static(_lib.ptr(X), _lib.ptr(s), T, H, E, k, _lib.dtype_id(X, "select_static"), _lib.ptr(xe),
                                  _lib.ptr(w), _lib.ptr(inv), _lib.ptr(off), _lib.ptr(ids), _lib.stream_ptr(X.device))
    assert rc == 0, rc


def _call(fn_name, X, s, E, k, with_ids):
    from torch_function import _lib
    L = _lib.lib()
    T, H = X.shape
    outs = _outputs(X, s, E, k, with_ids)
    if fn_name == "opmx_moe_select":
        xe, w, inv, off, ids = outs
        ws = _lib.workspace(L.opmx_moe_select_workspace_bytes(T, E, k), X.device)
        rc = L.opmx_moe_select(_lib.ptr(X), _lib.ptr(s), T, H, E, k, _lib.dtype_id(X, fn_name), _lib.ptr(xe), _lib.ptr(w),
                               _lib.ptr(inv), _lib.ptr(off), _lib.ptr(ids), _lib.ptr(ws), ws.numel(),
                               _lib.stream_ptr(X.device))
        assert rc == 0, (fn_name, rc)
    else:
        _enqueue_static(X, s, E, k, outs)
    torch.cuda.synchronize()
    return outs


def _inputs(n):
    T, H, E, k, dtype = CALLS[n]
    g = torch.Generator().manual_seed(100 + n)
    X = torch.randn(T, H, generator=g).to(dtype)
    s = tie_heavy_scores(T, E, dtype, seed=n) if n == 0 else torch.randn(T, E, generator=g).to(dtype)
    return X.to(dev()), s.to(dev()), E, k


def _same_bits(a, b):
    return torch.equal(a.contiguous().view(torch.uint8), b.contiguous().view(torch.uint8))


@pytest.mark.parametrize("with_ids", [False, True])
def test_static_scratch_select_matches_workspace_select(with_ids):
    for n, (T, H, E, k, dtype) in enumerate(CALLS):
        g = torch.Generator().manual_seed(100 + n)
        X = torch.randn(T, H, generator=g).to(dtype)
        s = tie_heavy_scores(T, E, dtype, seed=n) if n == 0 else torch.randn(T, E, generator=g).to(dtype)
        Xd, sd = X.to(dev()), s.to(dev())
        print("select_static call", n, (T, H, E, k, dtype), "ids" if with_ids else "no ids", flush=True)
        got = _call("opmx_moe_select_static", Xd, sd, E, k, with_ids)
        ref = _call("opmx_moe_select", Xd, sd, E, k, with_ids)
        for name, a, b in zip(("X_expand_permute", "expert_weights", "invert_permutation", "expert_offset", "ids"),
                              got, ref):
            if a is None:
                continue
            assert _same_bits(a, b), "call {}: {} differs from opmx_moe_select".format(n, name)
        # and against the oracle (integers and row copies bit-exact)
        rxe, _, rinv, roff = O.moe_select(X, s, E, k)
        assert torch.equal(got[2].cpu().view(T, k), rinv) and torch.equal(got[3].cpu(), roff)
        assert _same_bits(got[0].cpu(), rxe.reshape(T * k, H))


def test_static_scratch_select_few_tokens_and_empty():
    """Sizes that never touch the scratch memory go through the same entry point."""
    for T, H, E, k, dtype in [(32, 4096, 8, 2, torch.float16), (0, 64, 8, 2, torch.float16)]:
        g = torch.Generator().manual_seed(T)
        X = torch.randn(T, H, generator=g).to(dtype).to(dev())
        s = torch.randn(T, E, generator=g).to(dtype).to(dev())
        got = _call("opmx_moe_select_static", X, s, E, k, False)
        ref = _call("opmx_moe_select", X, s, E, k, False)
        for a, b in zip(got[:4], ref[:4]):
            assert _same_bits(a, b)


def test_static_scratch_select_back_to_back_without_sync_and_without_allocation():
    """The larger and the smaller call enqueued one behind the other on one stream with nothing
    between them (the second overwrites the front of the scratch array as soon as the first is done
    with it: stream order is the only protection, and it is enough), and the allocator's byte
    count does not move across the two calls."""
    a, b = _inputs(0), _inputs(1)
    _call("opmx_moe_select_static", *a, True)               # first use on this GPU: symbol lookup, kernel attributes
    outs_a, outs_b = _outputs(*a, True), _outputs(*b, True)
    torch.cuda.synchronize()
    before = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
    _enqueue_static(*a, outs_a)
    _enqueue_static(*b, outs_b)
    after = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
    torch.cuda.synchronize()
    assert before == after
    for args, outs in ((a, outs_a), (b, outs_b)):
        for got, ref in zip(outs, _call("opmx_moe_select", *args, True)):
            assert _same_bits(got, ref)


def test_static_scratch_select_captured_in_a_hip_graph():
    """After one call outside capture (kernel attributes, the scratch address) the entry point only
    enqueues kernels, so it records into a HIP graph; every replay, with eager calls of another size
    and synchronisation in between, gives the eager bits."""
    X, s, E, k = _inputs(0)
    ref = _call("opmx_moe_select_static", X, s, E, k, True)
    outs = _outputs(X, s, E, k, True)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _enqueue_static(X, s, E, k, outs)
    for replay in range(3):
        for t in outs:
            t.fill_(-3)
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, ref):
            assert _same_bits(got, want), "replay {}".format(replay)
        _call("opmx_moe_select_static", *_inputs(1), False)     # eager work on the same scratch array in between
