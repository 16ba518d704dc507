"""Pins the arithmetic half of the oracle: grouped linears, activations and the
whole layer, through special cases that reduce to library routines, the
permutation-free float64 formulation, and the independent C restatement."""
import pytest
import torch
import torch.nn.functional as F

from oracle import c_oracle
from oracle import moe_oracle as O


def test_grouped_linear_special_cases():
    g = torch.Generator().manual_seed(1)
    E, N, K, R = 4, 12, 10, 9
    W = torch.randn(E, N, K, generator=g)
    B = torch.randn(E, N, generator=g)
    X = torch.randn(R, K, generator=g)
    # all rows to one expert => one dense linear
    off = torch.tensor([0, 0, R, R, R])
    Y = O.moe_column_parallel_linear(X, off, W, B)
    assert torch.allclose(Y, F.linear(X, W[1], B[1]), atol=1e-5)
    # off = arange(E+1): the reference's own demo input
    # (MoeColumnParallelLinear.py:135-136) => row e uses expert e; rows >= E stay zero
    off = torch.arange(E + 1)
    Y = O.moe_row_parallel_linear(X, off, W, None)
    for e in range(E):
        assert torch.allclose(Y[e], W[e] @ X[e], atol=1e-5)
    assert torch.count_nonzero(Y[E:]) == 0
    # empty experts in the middle, ragged sizes
    off = torch.tensor([0, 3, 3, 3, 9])
    Y = O.moe_column_parallel_linear(X, off, W, B)
    assert torch.allclose(Y[:3], F.linear(X[:3], W[0], B[0]), atol=1e-5)
    assert torch.allclose(Y[3:], F.linear(X[3:], W[3], B[3]), atol=1e-5)
    Yc = c_oracle.grouped_linear(X, off, W, B)
    assert torch.allclose(Yc, Y, atol=1e-5)
    # in_features check, as MoeColumnParallelLinear.py:40
    with pytest.raises(AssertionError):
        O.moe_column_parallel_linear(X[:, :-1], off, W, B)
    # leading dims are preserved ([*, k, K] -> [*, k, N])
    Y3 = O.moe_column_parallel_linear(X[:8].view(4, 2, K), torch.tensor([0, 2, 4, 6, 8]), W, None)
    assert Y3.shape == (4, 2, N)


def test_linear_with_bias_pins():
    """O.linear (Linear.py:32) against the library routine and against an explicit double loop,
    with a bias whose sign, index and transposition mistakes would all show."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(11)
    X, W, B = torch.randn(5, 7, generator=g), torch.randn(3, 7, generator=g), torch.tensor([10.0, -20.0, 30.0])
    got = O.linear(X, W, B)
    assert got.shape == (5, 3)
    assert torch.allclose(got, F.linear(X, W, B), rtol=0, atol=1e-5)
    for t in range(5):
        for n in range(3):
            want = sum(float(X[t, c]) * float(W[n, c]) for c in range(7)) + float(B[n])
            assert abs(float(got[t, n]) - want) < 1e-4
    assert torch.allclose(O.linear(X, W), F.linear(X, W), rtol=0, atol=1e-5)       # no bias
    # known answer: ones . arange + bias
    assert torch.equal(O.linear(torch.ones(1, 4), torch.arange(8.0).view(2, 4), torch.tensor([0.5, -0.5])),
                       torch.tensor([[6.5, 21.5]]))
    # low precision: fp32 accumulation, rounded once, in the weight's dtype; leading dims kept
    Xh, Wh, Bh = torch.randn(2, 3, 64, generator=g).half(), torch.randn(9, 64, generator=g).half(), torch.randn(9, generator=g).half()
    got = O.linear(Xh, Wh, Bh)
    assert got.dtype == torch.float16 and got.shape == (2, 3, 9)
    assert torch.equal(got, F.linear(Xh.float(), Wh.float(), Bh.float()).half())


def test_grouped_linear_low_precision_rounds_once():
    g = torch.Generator().manual_seed(2)
    E, N, K, R = 2, 8, 512, 6
    W = (torch.randn(E, N, K, generator=g) * 0.05).half()
    X = torch.randn(R, K, generator=g).half()
    off = torch.tensor([0, 2, 6])
    Y = O.moe_column_parallel_linear(X, off, W)
    assert Y.dtype == torch.float16
    ref = torch.cat([X[:2].double() @ W[0].double().t(), X[2:].double() @ W[1].double().t()])
    assert torch.equal(Y, ref.half()) or (Y.float() - ref.float()).abs().max() < 1e-3
    Yc = c_oracle.grouped_linear(X, off, W).half()
    # fp32-accumulated vs double-accumulated: at most one fp16 ulp apart
    assert (Yc.float() - Y.float()).abs().max() <= 2 ** -9 * max(1.0, ref.abs().max().item())


def test_activations():
    g = torch.Generator().manual_seed(3)
    X = torch.randn(5, 14, generator=g)
    x, gt = X[:, :7], X[:, 7:]
    assert torch.allclose(O.swiglu(X), F.silu(x) * gt, atol=1e-6)          # SwiGLU.py:15-16
    assert torch.allclose(O.swiglu(X, beta=1.7), gt * x * torch.sigmoid(1.7 * x), atol=1e-6)
    assert torch.allclose(O.silu(x, gt), F.silu(x) * gt, atol=1e-6)        # SiLU.py:18-21
    assert torch.allclose(O.silu(x), F.silu(x), atol=1e-6)
    assert torch.allclose(c_oracle.swiglu(X, 1.7), O.swiglu(X, beta=1.7), atol=1e-6)
    assert torch.allclose(c_oracle.silu(x.contiguous(), gt.contiguous()), O.silu(x, gt), atol=1e-6)
    # the halves are not interchangeable: swapping them must change the result
    assert not torch.allclose(O.swiglu(torch.cat([gt, x], -1)), O.swiglu(X), atol=1e-3)
    # known values: x=0 -> 0 ; large x -> g*x
    assert O.swiglu(torch.tensor([[0.0, 3.0]])).item() == 0.0
    assert abs(O.swiglu(torch.tensor([[30.0, 2.0]])).item() - 60.0) < 1e-4


@pytest.mark.parametrize("T,H,E,k,I,dtype", [(16, 64, 8, 2, 96, torch.float32),
                                             (8, 128, 64, 8, 64, torch.float32),
                                             (24, 64, 8, 2, 96, torch.float16),
                                             (5, 32, 4, 4, 16, torch.bfloat16)])
def test_layer_equals_dense_fp64(T, H, E, k, I, dtype):
    x, Wg, wu, w2 = O.make_inputs(T, H, E, I, dtype=dtype, seed=7)
    Wg = (Wg.float() * 10).to(dtype)        # spread the routing
    scores = O.linear(x, Wg)
    full = O.moe_layer(x, Wg, wu, w2, E, k, scores=scores, round_between_ops=False, acc=torch.float64)
    dense = O.moe_layer_dense_fp64(x, Wg, wu, w2, E, k, scores=scores)
    scale = dense.abs().max().item()
    eps = {torch.float32: 2e-6, torch.float16: 1e-3, torch.bfloat16: 8e-3}[dtype]
    assert (full.double() - dense).abs().max().item() <= eps * max(scale, 1e-3)
    # fp32 accumulation with rounding between operators stays within the parity bar
    rounded = O.moe_layer(x, Wg, wu, w2, E, k, scores=scores, round_between_ops=True)
    err = (rounded.double() - dense).abs()
    assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3


def test_layer_c_restatement_agrees():
    T, H, E, k, I = 16, 64, 8, 2, 96
    x, Wg, wu, w2 = O.make_inputs(T, H, E, I, dtype=torch.float32, seed=11)
    Wg = Wg * 10
    r = O.moe_layer(x, Wg, wu, w2, E, k, return_all=True)
    sc = c_oracle.linear(x, Wg)
    assert torch.allclose(sc, r["scores"], atol=1e-5)
    xe, w, inv, off, idx = c_oracle.moe_select(x, r["scores"], E, k)
    assert torch.equal(inv, r["inv"]) and torch.equal(off, r["off"]) and torch.equal(idx, r["idx"])
    h = c_oracle.grouped_linear(xe, off, wu)
    a = c_oracle.swiglu(h)
    y = c_oracle.grouped_linear(a, off, w2)
    out = c_oracle.moe_reduce(y, w, inv, k)
    assert torch.allclose(out, r["out"], atol=1e-5)
    assert torch.allclose(h, r["x13"].view(-1, 2 * I), atol=1e-5)


def test_zipf_bias_skews_routing():
    T, H, E, k = 2048, 64, 8, 2
    x, Wg = O.make_inputs(T, H, E, 0, dtype=torch.float16, seed=0, with_w=False)
    for alpha in (2.0, 4.0):
        b = O.zipf_router_bias(E, alpha)
        s = O.linear(x, Wg, b.half())
        _, _, _, off = O.moe_select(x, s, E, k)
        share = (off[1:] - off[:-1]).max().item() / (T * k)
        assert 0.25 < share <= 0.5
    assert share > 0.40        # alpha=4: the benchmark's skew requirement


def test_make_inputs_is_deterministic():
    a = O.make_inputs(4, 8, 2, 6, seed=0)
    b = O.make_inputs(4, 8, 2, 6, seed=0)
    assert all(torch.equal(p, q) for p, q in zip(a, b))
    assert a[2].shape == (2, 12, 8) and a[3].shape == (2, 8, 6)


def test_rms_norm_pins():
    """skip_rms_norm / rms_norm (RMSNorm.py:16-24, 44-56) against a library routine, closed
    forms and the properties the definition fixes."""
    g = torch.Generator().manual_seed(5)
    X = torch.randn(6, 96, generator=g)
    S = torch.randn(6, 96, generator=g)
    w = torch.rand(96, generator=g) + 0.5
    # library routine (independent implementation)
    assert torch.allclose(O.rms_norm(X, w, 1e-5), F.rms_norm(X, (96,), w, 1e-5), atol=1e-6)
    Y, so = O.skip_rms_norm(X, w, S, 1e-6)
    assert torch.equal(so, X + S)                                        # skip output is the plain sum
    assert torch.allclose(Y, F.rms_norm(X + S, (96,), w, 1e-6), atol=1e-6)
    # closed forms: a constant row c normalises to sign(c) * weight; weights of one give unit RMS
    c = torch.full((1, 32), -3.0)
    assert torch.allclose(O.rms_norm(c, torch.arange(32.0), 0.0), -torch.arange(32.0).view(1, 32))
    assert torch.allclose(O.rms_norm(X, torch.ones(96), 0.0).pow(2).mean(-1), torch.ones(6), atol=1e-5)
    # scale invariance without eps, and eps really sits under the root: a zero row stays zero
    assert torch.allclose(O.rms_norm(7.5 * X, w, 0.0), O.rms_norm(X, w, 0.0), atol=1e-5)
    assert torch.equal(O.rms_norm(torch.zeros(2, 8), torch.ones(8), 1e-5), torch.zeros(2, 8))
    row = torch.tensor([[3.0, 4.0]])                                     # mean square 12.5
    assert torch.allclose(O.rms_norm(row, torch.ones(2), 3.5), row / 4.0)  # sqrt(12.5 + 3.5) = 4
    # without a skip input the skip output is X itself
    assert O.skip_rms_norm(X, w)[1] is X
    # low precision: the sum is rounded to the input dtype before the norm, the normalised value
    # is rounded before the multiply by the weight (two roundings, as the reference's type_as)
    Xh, Sh, wh = X.half(), S.half(), w.half()
    Yh, soh = O.skip_rms_norm(Xh, wh, Sh, 1e-5)
    assert soh.dtype == torch.float16 and torch.equal(soh, Xh + Sh)
    x32 = soh.float()
    y16 = (x32 * torch.rsqrt((x32 * x32).mean(-1, keepdim=True) + 1e-5)).half()
    assert torch.equal(Yh, (y16.float() * wh.float()).half())
