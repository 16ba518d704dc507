"""GPU check of ``opmx_moe_select_static``: MoeSelect for callers that cannot allocate.

It is ``opmx_moe_select`` with the library's own scratch array in place of a caller's
workspace, so both are called through the C ABI on the same inputs and every output must match
bit for bit (integers, weights and row copies alike: the kernels are the same).  Two calls in a
row share the array, the second one smaller than the first, so stale contents of the first
call sit behind the part the second one uses; the oracle checks the second call as well.
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


def _call(fn_name, X, s, E, k, with_ids):
    from torch_function import _lib
    L = _lib.lib()
    T, H = X.shape
    d = X.device
    xe = torch.full((T * k, H), float("nan"), dtype=X.dtype, device=d)
    w = torch.full((T, k), float("nan"), dtype=s.dtype, device=d)
    inv = torch.full((T * k,), -7, dtype=torch.int64, device=d)
    off = torch.full((E + 1,), -7, dtype=torch.int64, device=d)
    ids = torch.full((T, k), -7, dtype=torch.int32, device=d) if with_ids else None
    dt = _lib.dtype_id(X, fn_name)
    stream = _lib.stream_ptr(d)
    if fn_name == "opmx_moe_select":
        ws = _lib.workspace(L.opmx_moe_select_workspace_bytes(T, E, k), d)
        rc = L.opmx_moe_select(_lib.ptr(X), _lib.ptr(s), T, H, E, k, dt, _lib.ptr(xe), _lib.ptr(w), _lib.ptr(inv),
                               _lib.ptr(off), _lib.ptr(ids), _lib.ptr(ws), ws.numel(), stream)
    else:
        rc = L.opmx_moe_select_static(_lib.ptr(X), _lib.ptr(s), T, H, E, k, dt, _lib.ptr(xe), _lib.ptr(w),
                                      _lib.ptr(inv), _lib.ptr(off), _lib.ptr(ids), stream)
    assert rc == 0, (fn_name, rc)
    torch.cuda.synchronize()
    return xe, w, inv, off, ids


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
