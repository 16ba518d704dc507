"""Pins the routing half of the oracle (MoeSelect / MoeReduce restatements)
without the reference: brute force, closed forms, invariants, hand-made tie
cases, and agreement of the two independent restatements (Python and C)."""
import itertools
import json
import math
import os

import pytest
import torch

from oracle import c_oracle
from oracle import moe_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))


def brute_topk(row, k):
    """Pure-Python definition of the tie rule: order ids by (value desc, id asc)."""
    def key(e):
        v = row[e]
        if math.isnan(v):
            return (0, 0.0, e)
        return (1, -v, e)          # -(-0.0) == 0.0 compares equal to 0.0
    return sorted(range(len(row)), key=key)[:k]


def brute_select(idx_rows, E):
    """inv/off by the literal loops of MoeSelect.py:44-60 on Python lists."""
    flat = [e for r in idx_rows for e in r]
    perm = sorted(range(len(flat)), key=lambda j: (flat[j], j))     # stable sort
    inv = [-1] * len(flat)
    for i, j in enumerate(perm):
        inv[j] = i
    srt = [flat[j] for j in perm]
    off, ptr = [], 0
    for e in range(E):
        while ptr < len(srt) and srt[ptr] < e:
            ptr += 1
        off.append(ptr)
    off.append(len(flat))
    return perm, inv, off


@pytest.mark.parametrize("E,k", [(3, 1), (4, 2), (5, 3), (4, 4)])
def test_topk_bruteforce_all_tie_patterns(E, k):
    # every assignment of E scores from a 3-letter alphabet: all tie patterns
    vals = [-1.0, 0.5, 2.0]
    rows = list(itertools.product(vals, repeat=E))
    s = torch.tensor(rows, dtype=torch.float32)
    _, idx = O.topk_lower_id(s, k)
    for r, row in enumerate(rows):
        assert idx[r].tolist() == brute_topk(list(row), k), row
    _, _, _, _, cidx = c_oracle.moe_select(torch.zeros(len(rows), 2), s, E, k)
    assert torch.equal(cidx, idx)


def test_topk_special_values():
    nan, inf = float("nan"), float("inf")
    rows = [[0.0, -0.0, 0.0, -0.0], [-0.0, 0.0, -1.0, 0.0], [1.0, nan, 1.0, nan],
            [inf, inf, -inf, 3.0], [-inf, -inf, -inf, -inf], [nan, nan, nan, nan]]
    s = torch.tensor(rows)
    for k in (1, 2, 3):
        _, idx = O.topk_lower_id(s, k)
        _, _, _, _, cidx = c_oracle.moe_select(torch.zeros(len(rows), 2), s, 4, k)
        for r, row in enumerate(rows):
            assert idx[r].tolist() == brute_topk(row, k), (row, k)
        assert torch.equal(cidx, idx)
    # hand-written expectations, independent of brute_topk
    _, idx = O.topk_lower_id(s, 2)
    assert idx.tolist() == [[0, 1], [0, 1], [1, 3], [0, 1], [0, 1], [0, 1]]


def test_hand_made_tie_cases_file():
    """tests/golden/tie_cases.json was written by hand (expected values worked
    out on paper from the operator definition, not produced by any code)."""
    cases = json.load(open(os.path.join(HERE, "golden", "tie_cases.json")))
    for c in cases:
        E, k = c["E"], c["k"]
        s = torch.tensor(c["scores"], dtype=torch.float32)
        T = s.shape[0]
        X = torch.arange(T * 2, dtype=torch.float32).view(T, 2)
        for impl in ("py", "c"):
            if impl == "py":
                xe, w, inv, off, idx = O.moe_select(X, s, E, k, return_indices=True)
                xe = xe.reshape(-1, 2)
            else:
                xe, w, inv, off, idx = c_oracle.moe_select(X, s, E, k)
            assert idx.tolist() == c["idx"], (c["name"], impl)
            assert inv.tolist() == c["inv"], (c["name"], impl)
            assert off.tolist() == c["off"], (c["name"], impl)
            src = [int(v) // 2 for v in xe[:, 0].tolist()]
            assert src == c["row_source_token"], (c["name"], impl)
            if "weights" in c:
                assert torch.allclose(w.float(), torch.tensor(c["weights"]), atol=1e-6), c["name"]


@pytest.mark.parametrize("T,E,k,dtype", [(1, 8, 2, torch.float16), (7, 8, 2, torch.float32),
                                         (33, 64, 8, torch.bfloat16), (64, 8, 2, torch.float16),
                                         (50, 5, 5, torch.float32), (19, 16, 1, torch.float16)])
def test_select_matches_literal_loops_and_invariants(T, E, k, dtype):
    g = torch.Generator().manual_seed(T * 131 + E)
    H = 6
    X = torch.randn(T, H, generator=g).to(dtype)
    # coarse grid => many exact ties in every dtype
    s = (torch.randint(-3, 4, (T, E), generator=g).float() * 0.25).to(dtype)
    xe, w, inv, off, idx = O.moe_select(X, s, E, k, return_indices=True)
    R = T * k
    perm, binv, boff = brute_select(idx.tolist(), E)
    assert inv.reshape(-1).tolist() == binv and off.tolist() == boff
    for t in range(T):
        assert idx[t].tolist() == brute_topk(s[t].float().tolist(), k)
    # invariants
    assert inv.dtype == torch.int64 and off.dtype == torch.int64
    assert off[0] == 0 and off[E] == R and bool((off[1:] >= off[:-1]).all())
    assert sorted(inv.reshape(-1).tolist()) == list(range(R))
    xe2 = xe.reshape(R, H)
    assert torch.equal(xe2[inv.reshape(-1)], X.repeat_interleave(k, 0))   # bit-for-bit rows
    expert_of_row = torch.searchsorted(off[1:], torch.arange(R), right=True)
    assert torch.equal(expert_of_row[inv.reshape(-1)], idx.reshape(-1))
    for e in range(E):                          # stability: source tokens ascend inside a segment
        seg = [perm[r] for r in range(boff[e], boff[e + 1])]
        assert seg == sorted(seg)
    # closed forms for off
    srt = torch.sort(idx.reshape(-1)).values
    assert torch.equal(off, torch.searchsorted(srt, torch.arange(E + 1)))
    # weights: descending, sum to 1, equal softmax over ALL scores renormalised on the picks
    wf = w.float()
    assert bool((wf[:, :-1] >= wf[:, 1:]).all()) if k > 1 else True
    tol = {torch.float32: 1e-6, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}[dtype]
    assert torch.allclose(wf.sum(-1), torch.ones(T), atol=tol * k)
    full = torch.softmax(s.double(), -1)
    ref = torch.gather(full, 1, idx)
    ref = ref / ref.sum(-1, keepdim=True)
    assert torch.allclose(wf.double(), ref, atol=tol)
    # C restatement agrees on every integer and (to fp32 rounding) on weights
    cxe, cw, cinv, coff, cidx = c_oracle.moe_select(X, s, E, k)
    assert torch.equal(cidx, idx) and torch.equal(cinv, inv) and torch.equal(coff, off)
    assert torch.equal(cxe, xe2.float())
    assert torch.allclose(cw, ref.float(), atol=1e-6)


def test_select_leading_dims_and_empty():
    X = torch.randn(2, 3, 4)
    s = torch.randn(2, 3, 8)
    xe, w, inv, off = O.moe_select(X, s, 8, 2)
    assert xe.shape == (2, 3, 2, 4) and w.shape == (2, 3, 2) and inv.shape == (2, 3, 2) and off.shape == (9,)
    xe, w, inv, off = O.moe_select(torch.zeros(0, 4), torch.zeros(0, 8), 8, 2)
    assert xe.shape == (0, 2, 4) and off.tolist() == [0] * 9


def test_reduce_closed_forms():
    g = torch.Generator().manual_seed(5)
    T, k, N = 9, 4, 16
    Y = torch.randn(T, k, N, generator=g)
    # inv = identity and w = 1/k  => mean over the k slots
    inv = torch.arange(T * k).view(T, k)
    w = torch.full((T, k), 1.0 / k)
    out = O.moe_reduce(Y, w, inv, k)
    assert torch.allclose(out, Y.mean(1), atol=1e-6)
    # random permutation: equals index_add formulation
    perm = torch.randperm(T * k, generator=g)
    w = torch.rand(T, k, generator=g)
    out = O.moe_reduce(Y, w, perm.view(T, k), k)
    ref = torch.zeros(T, N, dtype=torch.float64)
    for t in range(T):
        for s_ in range(k):
            ref[t] += w[t, s_].double() * Y.view(-1, N)[perm[t * k + s_]].double()
    assert torch.allclose(out.double(), ref, atol=1e-6)
    cout = c_oracle.moe_reduce(Y, w, perm.view(T, k), k)
    assert torch.allclose(cout.double(), ref, atol=1e-6)
    # one-hot weights pick exactly one row, bit-for-bit
    w1 = torch.zeros(T, k)
    w1[:, 2] = 1.0
    out = O.moe_reduce(Y.half(), w1.half(), perm.view(T, k), k)
    assert torch.equal(out, Y.half().view(-1, N)[perm.view(T, k)[:, 2]])


def test_as_written_bookkeeping_equals_vectorised():
    g = torch.Generator().manual_seed(9)
    for T, E, k in ((1, 8, 2), (37, 8, 2), (20, 64, 8)):
        X = torch.randn(T, 5, generator=g)
        s = (torch.randint(-3, 4, (T, E), generator=g).float() * 0.25)
        a = O.moe_select(X, s, E, k)
        b = O.moe_select_as_written(X, s, E, k)
        assert all(torch.equal(p, q) for p, q in zip(a, b))
