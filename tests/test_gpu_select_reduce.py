"""GPU parity: MoeSelect / MoeReduce / SwiGLU / SiLU / router Linear against the
CPU oracle on identical inputs.  Integer outputs and row copies bit-exact."""
import json
import os

import pytest
import torch

from _util import assert_close_ulp, dev, tie_heavy_scores
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
W_TOL = {torch.float32: 2e-6, torch.float16: 1e-3, torch.bfloat16: 8e-3}


def opmx():
    import torch_function as OPMX
    return OPMX


def check_select(X, s, E, k):
    OPMX = opmx()
    xe, w, inv, off = OPMX.moe_select(X.to(dev()), s.to(dev()), E, k)
    rxe, rw, rinv, roff = O.moe_select(X, s, E, k)
    assert inv.dtype == torch.int64 and off.dtype == torch.int64 and xe.dtype == X.dtype and w.dtype == s.dtype
    assert xe.shape == rxe.shape and w.shape == rw.shape and inv.shape == rinv.shape and off.shape == roff.shape
    assert torch.equal(off.cpu(), roff), "expert_offset"
    assert torch.equal(inv.cpu(), rinv), "invert_permutation"
    assert torch.equal(xe.cpu().view(torch.uint8), rxe.contiguous().view(torch.uint8)), "X_expand_permute bits"
    wd = (w.cpu().double() - rw.double()).abs()
    finite = torch.isfinite(rw.double())
    assert torch.equal(torch.isfinite(w.cpu().double()), finite)
    assert float(wd[finite].max() if finite.any() else 0.0) <= W_TOL[s.dtype], "expert_weights"
    return xe, w, inv, off


SELECT_CASES = [
    # T, H, E, k, dtype                      path
    (1, 64, 8, 2, torch.float16),          # single token, one launch
    (32, 4096, 8, 2, torch.float16),       # Mixtral decode
    (64, 512, 8, 2, torch.float16),        # largest one-launch size for E=8
    (65, 512, 8, 2, torch.float16),        # picks by the top-k kernel, bookkeeping + rows by the small kernel
    (128, 4096, 8, 2, torch.float16),
    (256, 128, 8, 2, torch.float16),       # largest size of that two-launch form
    (8, 2048, 64, 8, torch.bfloat16),      # 64 experts: one launch up to 8 tokens
    (16, 256, 32, 4, torch.bfloat16),      # 32 experts: one launch up to 16
    (17, 256, 32, 4, torch.bfloat16),
    (32, 2048, 64, 8, torch.bfloat16),     # fine-grained decode, two launches
    (200, 64, 256, 32, torch.float16),     # two launches at the limits E = 256, k = 32
    (7, 6, 5, 3, torch.float32),           # rows not 16-byte multiples: scalar copy
    (33, 40, 5, 5, torch.float32),         # k == E
    (257, 64, 8, 2, torch.float16),        # first general-path size
    (300, 72, 16, 1, torch.bfloat16),      # k == 1
    (2048, 512, 8, 2, torch.float16),
    (4096, 2048, 64, 8, torch.bfloat16),   # fine-grained prefill
    (1000, 48, 100, 5, torch.float32),     # E > 64: several experts per lane
    (513, 16, 256, 32, torch.float16),     # limits: E = 256, k = 32
    (40, 16, 200, 9, torch.float32),       # E > 64 on the small path
]


@pytest.mark.parametrize("T,H,E,k,dtype", SELECT_CASES)
def test_select_random_scores(T, H, E, k, dtype):
    g = torch.Generator().manual_seed(T * 7 + E)
    X = torch.randn(T, H, generator=g).to(dtype)
    s = torch.randn(T, E, generator=g).to(dtype)
    check_select(X, s, E, k)


@pytest.mark.parametrize("T,H,E,k,dtype", SELECT_CASES)
def test_select_tie_heavy_scores(T, H, E, k, dtype):
    g = torch.Generator().manual_seed(T + 3)
    X = torch.randn(T, H, generator=g).to(dtype)
    check_select(X, tie_heavy_scores(T, E, dtype, seed=T * 13 + E), E, k)


def test_select_golden_tie_cases():
    for c in json.load(open(os.path.join(HERE, "golden", "tie_cases.json"))):
        E, k = c["E"], c["k"]
        for dtype in (torch.float32, torch.float16, torch.bfloat16):
            s = torch.tensor(c["scores"]).to(dtype)
            T = s.shape[0]
            X = torch.arange(T * 8, dtype=torch.float32).view(T, 8).to(dtype)
            xe, w, inv, off = opmx().moe_select(X.to(dev()), s.to(dev()), E, k)
            assert inv.cpu().tolist() == c["inv"], c["name"]
            assert off.cpu().tolist() == c["off"], c["name"]
            src = [int(v) // 8 for v in xe.cpu().float().view(-1, 8)[:, 0].tolist()]
            assert src == c["row_source_token"], c["name"]
            if "weights" in c:
                assert torch.allclose(w.cpu().float(), torch.tensor(c["weights"]), atol=W_TOL[dtype])


def test_select_special_values():
    nan, inf = float("nan"), float("inf")
    rows = [[0.0, -0.0, 0.0, -0.0, 1.0, 1.0, -1.0, -0.0], [nan, 1.0, nan, 2.0, 2.0, -inf, inf, 0.0],
            [-inf] * 8, [inf, 3.0, inf, 3.0, 3.0, 1.0, 0.0, nan], [5.0, 5.0, 5.0, 5.0, 5.0, 5.0, 5.0, 5.0]]
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        s = torch.tensor(rows).to(dtype)
        X = torch.randn(len(rows), 16).to(dtype)
        for k in (1, 2, 3):
            OPMX = opmx()
            xe, w, inv, off = OPMX.moe_select(X.to(dev()), s.to(dev()), 8, k)
            rxe, rw, rinv, roff = O.moe_select(X, s, 8, k)
            assert torch.equal(inv.cpu(), rinv) and torch.equal(off.cpu(), roff)
            assert torch.equal(torch.isnan(w.cpu()), torch.isnan(rw))


def test_select_leading_dims_empty_and_errors():
    OPMX = opmx()
    X = torch.randn(2, 3, 32).half()
    s = torch.randn(2, 3, 8).half()
    xe, w, inv, off = OPMX.moe_select(X.to(dev()), s.to(dev()), 8, 2)
    rxe, rw, rinv, roff = O.moe_select(X, s, 8, 2)
    assert xe.shape == (2, 3, 2, 32) and w.shape == (2, 3, 2) and inv.shape == (2, 3, 2)
    assert torch.equal(inv.cpu(), rinv) and torch.equal(xe.cpu(), rxe)
    xe, w, inv, off = OPMX.moe_select(torch.zeros(0, 32, device=dev()), torch.zeros(0, 8, device=dev()), 8, 2)
    assert xe.shape == (0, 2, 32) and off.cpu().tolist() == [0] * 9
    with pytest.raises(RuntimeError):
        OPMX.moe_select(X, s, 8, 2)                                   # CPU tensors: no fallback
    with pytest.raises(RuntimeError):
        OPMX.moe_select(torch.zeros(4, 8, device=dev()), torch.zeros(4, 300, device=dev()), 300, 2)
    with pytest.raises(ValueError):
        OPMX.moe_select(X.to(dev()), s.to(dev()), 8, 9)


def test_select_full_size_properties():
    """Mixtral prefill size (T=8192): size-independent invariants + oracle integers."""
    T, H, E, k = 8192, 4096, 8, 2
    g = torch.Generator().manual_seed(0)
    X = torch.randn(T, H, generator=g).half()
    s = (torch.randn(T, E, generator=g) + O.zipf_router_bias(E, 4.0)).half()
    xe, w, inv, off = check_select(X, s, E, k)
    R = T * k
    invf = inv.view(-1)
    assert int(off[0]) == 0 and int(off[E]) == R and bool((off[1:] >= off[:-1]).all())
    assert torch.equal(torch.sort(invf).values, torch.arange(R, device=dev()))
    assert torch.equal(xe.view(R, H)[invf], X.to(dev()).repeat_interleave(k, 0))
    assert float((off[1:] - off[:-1]).max()) / R > 0.40            # the skew the config asks for


@pytest.mark.parametrize("T,k,N,dtype", [(1, 2, 4096, torch.float16), (32, 2, 4096, torch.float16),
                                         (8192, 2, 4096, torch.float16), (4096, 8, 2048, torch.bfloat16),
                                         (64, 2, 1024, torch.float32), (5, 3, 10, torch.float32),
                                         (9, 32, 24, torch.float16)])
def test_reduce(T, k, N, dtype):
    g = torch.Generator().manual_seed(T + k)
    Y = torch.randn(T, k, N, generator=g).to(dtype)
    w = torch.softmax(torch.randn(T, k, generator=g), -1).to(dtype)
    inv = torch.randperm(T * k, generator=g).view(T, k)
    out = opmx().moe_reduce(Y.to(dev()), w.to(dev()), inv.to(dev()), k)
    ref = O.moe_reduce(Y, w, inv, k, acc=torch.float64)
    assert out.shape == (T, N) and out.dtype == dtype
    assert_close_ulp(out, ref, dtype, ulps=1.5 if dtype != torch.float32 else 8, what="moe_reduce",
                     floor=0.01 if dtype != torch.float32 else 0.25)
    # one-hot weights select one row bit-for-bit
    w1 = torch.zeros(T, k)
    w1[:, k - 1] = 1.0
    out = opmx().moe_reduce(Y.to(dev()), w1.to(dtype).to(dev()), inv.to(dev()), k)
    assert torch.equal(out.cpu(), Y.view(-1, N)[inv[:, k - 1]])


@pytest.mark.parametrize("R,D,dtype", [(64, 14336, torch.float16), (16384, 1408, torch.bfloat16),
                                       (128, 2816, torch.float32), (3, 7, torch.float16), (5, 12, torch.float32)])
def test_swiglu_and_silu(R, D, dtype):
    g = torch.Generator().manual_seed(R + D)
    X = (torch.randn(R, 2 * D, generator=g) * 2).to(dtype)
    OPMX = opmx()
    tol = dict(ulps=1.5 if dtype != torch.float32 else 16)
    assert_close_ulp(OPMX.swiglu(X.to(dev())), O.swiglu(X, acc=torch.float64), dtype, what="swiglu", **tol)
    assert_close_ulp(OPMX.swiglu(X.to(dev()), 1.7), O.swiglu(X, beta=1.7, acc=torch.float64), dtype,
                     what="swiglu beta", **tol)
    x, gt = X[:, :D].contiguous(), X[:, D:].contiguous()
    assert_close_ulp(OPMX.silu(x.to(dev()), gt.to(dev())), O.silu(x, gt, acc=torch.float64), dtype, what="silu gate",
                     **tol)
    assert_close_ulp(OPMX.silu(x.to(dev())), O.silu(x, acc=torch.float64), dtype, what="silu", **tol)


@pytest.mark.parametrize("T,K,N,dtype,bias", [(32, 4096, 8, torch.float16, False), (1, 4096, 8, torch.float16, True),
                                              (8192, 4096, 8, torch.float16, False),
                                              (4096, 2048, 64, torch.bfloat16, False),
                                              (64, 1024, 8, torch.float32, True), (5, 30, 3, torch.float32, True),
                                              (1030, 72, 20, torch.float16, True),
                                              # many tokens, few outputs: the kernel that splits K over waves
                                              (4097, 4096, 5, torch.float16, True),     # ragged last token tile
                                              (600, 96, 33, torch.bfloat16, True),      # 3 k-steps for 8 waves, 3 output tiles
                                              (513, 1024, 16, torch.float16, False),
                                              (700, 32, 24, torch.float16, True),       # a single k-step
                                              (2048, 4096 + 32 * 37, 48, torch.bfloat16, False),   # odd number of k-steps
                                              (8192, 2048, 64, torch.bfloat16, True),   # back on the tile kernel
                                              (1000, 1024, 256, torch.bfloat16, True),  # 256 outputs: four blocks of 64 per token tile
                                              (600, 512, 100, torch.float16, False),    # last block of outputs ragged
                                              (130, 256, 256, torch.bfloat16, True),    # 256 outputs from 128 tokens on
                                              (3000, 512, 200, torch.float16, True)])   # too many tokens for that: tile kernel
def test_router_linear(T, K, N, dtype, bias):
    g = torch.Generator().manual_seed(K + N)
    X = torch.randn(T, K, generator=g).to(dtype)
    W = (torch.randn(N, K, generator=g) * 0.02).to(dtype)
    B = torch.randn(N, generator=g).to(dtype) if bias else None
    out = opmx().linear(X.to(dev()), W.to(dev()), None if B is None else B.to(dev()), K, N)
    ref = O.linear(X, W, B, acc=torch.float64, out_dtype=torch.float64)
    assert out.shape == (T, N) and out.dtype == dtype
    assert_close_ulp(out, ref, dtype, ulps=1.5 if dtype != torch.float32 else 32, what="linear",
                     floor=0.01 if dtype != torch.float32 else 0.25)


# Router gate and MoeSelect in one call.  Up to 8 tokens and 16 experts in fp16/bf16 with
# H % 32 == 0 it is a single launch whose logits come from the MFMA units; every other case runs
# the two operators inside the library.  The bar is the same either way: the returned logits
# within rounding of the fp32 oracle, and the routing bit-exact given those logits.
ROUTE_SELECT_CASES = [
    # T, H, E, k, dtype, bias
    (1, 4096, 8, 2, torch.float16, False),      # Mixtral, one token
    (8, 4096, 8, 2, torch.float16, True),       # largest single-launch size
    (5, 1024, 16, 4, torch.bfloat16, True),     # 16 experts
    (7, 96, 5, 2, torch.bfloat16, False),       # three k-steps for sixteen waves, E not a multiple of 4
    (8, 32, 3, 3, torch.float16, True),         # one k-step: all waves but one add nothing
    (8, 4096 + 32 * 67, 8, 2, torch.float16, True),    # k-steps not a multiple of the waves or of the unrolling
    (9, 4096, 8, 2, torch.float16, True),       # one token too many: two launches
    (32, 4096, 8, 2, torch.float16, True),      # Mixtral decode
    (8, 2048, 64, 8, torch.bfloat16, False),    # too many experts
    (8, 100, 8, 2, torch.float16, True),        # H not a multiple of 32
    (8, 64, 8, 2, torch.float32, True),         # fp32
    (600, 512, 16, 2, torch.float16, False),    # long prompt, 16 experts: the router kernel routes in its epilogue
    (4096, 512, 8, 2, torch.float16, True),     # 8 experts from 4096 tokens on: router kernel with routing epilogue
    (4100, 256, 8, 2, torch.bfloat16, False),   # ... a last block with 4 tokens
    (1000, 2048, 64, 8, torch.bfloat16, False), # 64 experts, top-8: one key per lane of a whole wave
    (700, 256, 33, 5, torch.float16, True),     # 33 experts: three 16-output tiles, the last one ragged
    (520, 256, 64, 32, torch.float16, False),   # limits of the routing epilogue: 64 experts, 32 picks
    (300, 512, 16, 2, torch.float16, False),    # below 512 tokens: the two operators one after the other
]


@pytest.mark.parametrize("T,H,E,k,dtype,bias", ROUTE_SELECT_CASES)
def test_route_select_matches_oracle(T, H, E, k, dtype, bias):
    g = torch.Generator().manual_seed(T * 31 + H + E)
    X = torch.randn(T, H, generator=g).to(dtype)
    Wg = (torch.randn(E, H, generator=g) * (H ** -0.5)).to(dtype)
    b = torch.randn(E, generator=g).to(dtype) if bias else None
    d = dev()
    xe, w, inv, off, scores = opmx().moe_route_select(X.to(d), Wg.to(d), None if b is None else b.to(d), E, k)
    assert scores.shape == (T, E) and scores.dtype == dtype
    ref = O.linear(X, Wg, b, out_dtype=torch.float32)
    # one rounding of an fp32 sum; in fp32 the sum itself is only as good as its summation order
    assert_close_ulp(scores, ref, dtype, ulps=2.0 if dtype != torch.float32 else 64.0, what="router logits")
    rxe, rw, rinv, roff = O.moe_select(X, scores.cpu(), E, k)
    assert torch.equal(off.cpu(), roff) and torch.equal(inv.cpu(), rinv)
    assert torch.equal(xe.cpu().view(torch.uint8), rxe.contiguous().view(torch.uint8))
    assert float((w.cpu().double() - rw.double()).abs().max()) <= W_TOL[dtype]
    # the separate operators on the same inputs: same routing whenever the logits agree bit for bit
    s2 = opmx().linear(X.to(d), Wg.to(d), None if b is None else b.to(d), H, E)
    if torch.equal(s2, scores):
        xe2, w2, inv2, off2 = opmx().moe_select(X.to(d), s2, E, k)
        assert torch.equal(inv2, inv) and torch.equal(off2, off) and torch.equal(xe2, xe) and torch.equal(w2, w)


def test_route_select_ties_go_to_the_lower_expert():
    """Identical gate rows give identical logits for every token: all picks are ties."""
    T, H, E, k = 8, 64, 8, 3
    g = torch.Generator().manual_seed(5)
    X = torch.randn(T, H, generator=g).half()
    Wg = torch.randn(1, H, generator=g).half().repeat(E, 1)
    d = dev()
    xe, w, inv, off, scores = opmx().moe_route_select(X.to(d), Wg.to(d), None, E, k)
    assert torch.equal(scores[:, :1].expand(T, E), scores)
    assert off.cpu().tolist() == [0, T, 2 * T, 3 * T] + [3 * T] * (E - 3)
    rxe, rw, rinv, roff = O.moe_select(X, scores.cpu(), E, k)
    assert torch.equal(inv.cpu(), rinv) and torch.equal(xe.cpu(), rxe)
