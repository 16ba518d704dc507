"""GPU parity of the index form of MoeSelect and of the gate/up GEMM that reads its rows through it.

The reference materialises ``X_expand_permute = X.repeat_interleave(k)[perm]``
(torch_function/MoeSelect.py:45-47) and multiplies it (MoeColumnParallelLinear.py:58-67).
``moe_select_index`` returns ``row_token`` (= perm // k) instead of the copy and
``moe_column_parallel_linear_indexed`` reads ``X[row_token]`` inside the GEMM.  Bar: the routing
outputs equal the oracle's bit for bit, ``X[row_token]`` is the oracle's ``X_expand_permute`` bit
for bit, and the indexed GEMM equals the GEMM on the expanded copy bit for bit in every kernel
family (it does the same arithmetic on the same operands, only fetched differently); the
expanded GEMM itself is checked against the float64 oracle in test_gpu_gemm.py."""
import pytest
import torch

from _util import assert_close_ulp, dev, gpu_inputs, tie_heavy_scores
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def opmx():
    import torch_function as OPMX
    return OPMX


INDEX_CASES = [
    (1, 64, 8, 2, torch.float16), (32, 4096, 8, 2, torch.float16), (65, 512, 8, 2, torch.float16),
    (256, 128, 8, 2, torch.float16), (8, 2048, 64, 8, torch.bfloat16), (32, 2048, 64, 8, torch.bfloat16),
    (200, 64, 256, 32, torch.float16), (33, 40, 5, 5, torch.float32), (257, 64, 8, 2, torch.float16),
    (2048, 512, 8, 2, torch.float16), (4096, 256, 64, 8, torch.bfloat16), (1000, 48, 100, 5, torch.float32),
]


@pytest.mark.parametrize("T,H,E,k,dtype", INDEX_CASES)
@pytest.mark.parametrize("ties", [False, True])
def test_select_index_matches_oracle_and_select(T, H, E, k, dtype, ties):
    OPMX = opmx()
    g = torch.Generator().manual_seed(T * 3 + E)
    X = torch.randn(T, H, generator=g).to(dtype)
    s = tie_heavy_scores(T, E, dtype, seed=T + E) if ties else torch.randn(T, E, generator=g).to(dtype)
    w, inv, off, row_token = OPMX.moe_select_index(s.to(dev()), E, k)
    assert row_token.dtype == torch.int32 and row_token.shape == (T * k,)
    rxe, rw, rinv, roff = O.moe_select(X, s, E, k)
    assert torch.equal(inv.cpu(), rinv) and torch.equal(off.cpu(), roff)
    # the index stands for X_expand_permute: X[row_token] is the oracle's copy, bit for bit
    assert torch.equal(X[row_token.cpu().long()].view(torch.uint8), rxe.reshape(T * k, H).contiguous().view(torch.uint8))
    # ... and is the inverse of invert_permutation on the token axis
    assert torch.equal(row_token[inv.view(-1)].cpu().long(), torch.arange(T).repeat_interleave(k))
    # same weights, bit for bit, as the operator with the copy
    xe2, w2, inv2, off2 = OPMX.moe_select(X.to(dev()), s.to(dev()), E, k)
    assert torch.equal(w.view(torch.uint8), w2.view(torch.uint8)) and torch.equal(inv, inv2) and torch.equal(off, off2)


ROUTE_INDEX_CASES = [
    # one launch of one block (fp16 / bf16; by default up to 8 tokens and 16 experts, with the knob up to 64 and
    # 64): one, two token tiles; 1, 2, 4 expert tiles
    (1, 4096, 8, 2, torch.float16), (8, 4096, 8, 2, torch.float16), (16, 4096, 8, 2, torch.float16),
    (17, 4096, 8, 2, torch.float16), (32, 4096, 8, 2, torch.float16), (8, 2048, 16, 4, torch.bfloat16),
    (32, 2048, 64, 8, torch.bfloat16), (5, 2048, 64, 8, torch.bfloat16), (31, 96, 33, 5, torch.float16),
    (32, 6144, 24, 24, torch.float16), (3, 32, 3, 1, torch.bfloat16), (20, 64, 64, 32, torch.float16),
    # beyond: the router kernel and the select kernels one after the other
    (33, 4096, 8, 2, torch.float16), (64, 2048, 64, 8, torch.bfloat16), (600, 512, 16, 2, torch.float16),
    (5, 96, 8, 2, torch.float32), (16, 40, 8, 2, torch.float16), (12, 512, 100, 4, torch.bfloat16),
]


def check_route_select_index(T, H, E, k, dtype, bias=True, wscale=0.05, seed=None):
    """moe_route_select_index against the oracle: logits within one rounding of the fp32 sum, and the
    routing bit-exact on the logits the call itself returns."""
    OPMX = opmx()
    g = torch.Generator().manual_seed(T + H if seed is None else seed)
    Xc = torch.randn(T, H, generator=g).to(dtype)
    Wgc = (torch.randn(E, H, generator=g) * wscale).to(dtype)
    Bgc = torch.randn(E, generator=g).to(dtype) if bias else None
    X, Wg, Bg = Xc.to(dev()), Wgc.to(dev()), None if Bgc is None else Bgc.to(dev())
    w, inv, off, row_token, scores = OPMX.moe_route_select_index(X, Wg, Bg, E, k)
    assert scores.shape == (T, E) and scores.dtype == dtype and row_token.dtype == torch.int32
    ref = O.linear(Xc, Wgc, Bgc, out_dtype=torch.float32)
    assert_close_ulp(scores, ref, dtype, ulps=2.0 if dtype != torch.float32 else 64.0, what="router logits")
    rxe, rw, rinv, roff = O.moe_select(Xc, scores.cpu(), E, k)
    assert torch.equal(inv.cpu(), rinv) and torch.equal(off.cpu(), roff)
    assert torch.equal(Xc[row_token.cpu().long()].view(torch.uint8), rxe.reshape(T * k, H).contiguous().view(torch.uint8))
    assert float((w.cpu().double() - rw.double()).abs().max()) <= {torch.float32: 1e-6, torch.float16: 1e-3,
                                                                   torch.bfloat16: 8e-3}[dtype]
    # the same routing, bit for bit, as moe_select_index fed those logits
    w2, inv2, off2, rt2 = OPMX.moe_select_index(scores, E, k)
    assert torch.equal(w.view(torch.uint8), w2.view(torch.uint8)) and torch.equal(inv, inv2)
    assert torch.equal(off, off2) and torch.equal(row_token, rt2)
    return scores


@pytest.mark.parametrize("T,H,E,k,dtype", ROUTE_INDEX_CASES)
@pytest.mark.parametrize("one_launch_up_to", [None, 64])
def test_route_select_index_matches_oracle(T, H, E, k, dtype, one_launch_up_to):
    from torch_function import _lib
    _lib.set_option("OPMX_MOE_ROUTE_INDEX_TOKENS", one_launch_up_to)
    try:
        check_route_select_index(T, H, E, k, dtype, bias=True)
        check_route_select_index(T, H, E, k, dtype, bias=False, wscale=H ** -0.5, seed=7 * T + E)
    finally:
        _lib.set_option("OPMX_MOE_ROUTE_INDEX_TOKENS", None)


def test_route_select_index_one_launch_up_to_64_tokens():
    """The one-launch kernel's four-token-tile form (33 ... 64 tokens), switched on through its knob."""
    from torch_function import _lib
    _lib.set_option("OPMX_MOE_ROUTE_INDEX_TOKENS", 64)
    try:
        for T, H, E, k, dtype in [(33, 4096, 8, 2, torch.float16), (64, 2048, 64, 8, torch.bfloat16),
                                  (49, 512, 40, 6, torch.float16)]:
            check_route_select_index(T, H, E, k, dtype)
        _lib.set_option("OPMX_MOE_ROUTE_INDEX_TOKENS", 0)       # never: the separate kernels
        check_route_select_index(8, 4096, 8, 2, torch.float16)
    finally:
        _lib.set_option("OPMX_MOE_ROUTE_INDEX_TOKENS", None)


def test_route_select_index_ties_go_to_the_lower_expert():
    """Identical gate rows give identical logits for every token: all picks are ties."""
    T, H, E, k = 24, 64, 8, 3
    g = torch.Generator().manual_seed(5)
    X = torch.randn(T, H, generator=g).half()
    Wg = torch.randn(1, H, generator=g).half().repeat(E, 1)
    w, inv, off, row_token, scores = opmx().moe_route_select_index(X.to(dev()), Wg.to(dev()), None, E, k)
    assert torch.equal(scores[:, :1].expand(T, E), scores)
    assert off.cpu().tolist() == [0, T, 2 * T, 3 * T] + [3 * T] * (E - 3)
    assert row_token.cpu().tolist() == list(range(T)) * 3
    rxe, rw, rinv, roff = O.moe_select(X, scores.cpu(), E, k)
    assert torch.equal(inv.cpu(), rinv)


def offsets(sizes, lo=0):
    return torch.tensor([lo] + [lo + int(v) for v in torch.tensor(sizes).cumsum(0)], dtype=torch.int64)


def indexed_case(sizes, T, K, N, dtype, bias, env=None, swiglu=False, lo=0, tail=0, seed=0):
    """The indexed GEMM against the GEMM on the gathered copy, bit for bit; both against the oracle."""
    from torch_function import _lib
    OPMX = opmx()
    E = len(sizes)
    off = offsets(sizes, lo)
    R = lo + int(sum(sizes)) + tail                     # rows in front of / behind every expert: set to zero
    g = torch.Generator().manual_seed(seed + K + N + R)
    Xtok = torch.randn(T, K, generator=g).to(dtype)
    row_token = torch.randint(0, T, (R,), generator=g, dtype=torch.int32)
    W = (torch.randn(E, N, K, generator=g) * 0.05).to(dtype)
    B = torch.randn(E, N, generator=g).to(dtype) if bias else None
    for key, val in (env or {}).items():
        _lib.set_option(key, val)
    try:
        d = dev()
        Wd, Bd, offd = W.to(d), None if B is None else B.to(d), off.to(d)
        Xe = Xtok[row_token.long()].to(d)
        if swiglu:
            want = OPMX.moe_column_parallel_linear_swiglu(Xe, offd, Wd, Bd, E, K, N)
        else:
            want = OPMX.moe_column_parallel_linear(Xe, offd, Wd, Bd, None, E, K, N, False)
        got = OPMX.moe_column_parallel_linear_indexed(Xtok.to(d), row_token.to(d), offd, Wd, Bd, E, K, N, swiglu=swiglu)
        torch.cuda.synchronize()
    finally:
        for key in (env or {}):
            _lib.set_option(key, None)
    assert got.shape == (T, R // T, want.shape[-1]) if R % T == 0 else True
    assert torch.equal(got.reshape(want.shape).view(torch.uint8), want.view(torch.uint8)), \
        "indexed GEMM differs from the GEMM on the gathered rows: {} K{} N{} {} {}".format(sizes, K, N, dtype, env)
    ref = O.moe_column_parallel_linear(Xtok[row_token.long()], off, W, B, acc=torch.float64, out_dtype=torch.float64)
    if swiglu:
        ref = O.swiglu(ref, acc=torch.float64)
    f32 = dtype == torch.float32
    assert_close_ulp(got.reshape(ref.shape), ref, dtype, ulps=64 if f32 else 2, floor=0.25 if f32 else 0.02,
                     what="indexed {} K{} N{} {} {}".format(sizes, K, N, dtype, env))


RAGGED8 = [5, 0, 17, 1, 0, 64, 3, 38]            # 128 rows
BIG8 = [1500, 0, 700, 33, 1281, 256, 5, 1345]    # 5120 rows, ragged row tiles


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("swiglu", [False, True])
def test_indexed_generic_kernel(dtype, swiglu):
    env = {"OPMX_MOE_GEMM": "generic"}
    indexed_case(RAGGED8, 64, 72, 96, dtype, True, env, swiglu=swiglu)
    indexed_case([3, 200, 0, 7], 105, 50, 34, dtype, False, env, swiglu=swiglu)     # odd K and N; R = 2 T


@pytest.mark.parametrize("swiglu", [False, True])
def test_indexed_fp32_matrix_unit_kernel(swiglu):
    indexed_case(RAGGED8, 64, 128, 96, torch.float32, True, swiglu=swiglu)         # 32-row tiles
    indexed_case(RAGGED8, 64, 512, 96, torch.float32, True, {"OPMX_MOE_GEMM_F32_VARIANT": "0"}, swiglu=swiglu)
    indexed_case(RAGGED8, 64, 512, 96, torch.float32, True, {"OPMX_MOE_GEMM_F32_VARIANT": "1"}, swiglu=swiglu)   # waves split K
    indexed_case(BIG8, 2560, 100, 256, torch.float32, False, swiglu=swiglu)        # 128-row tiles, ragged K tile


@pytest.mark.parametrize("variant", ["0", "1", "2", "3"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_indexed_tiled_kernels(variant, dtype):
    env = {"OPMX_MOE_GEMM": "tiled", "OPMX_MOE_GEMM_TILED_VARIANT": variant, "OPMX_MOE_GEMM_STREAMK": "0"}
    indexed_case(BIG8, 2560, 128, 4096, dtype, True, env)                      # 16 column tiles: expert-major order
    indexed_case(BIG8, 2560, 256, 4096, dtype, False, env, swiglu=True)        # persistent form when variant 0
    indexed_case(BIG8, 640, 64, 2816, dtype, False, env)                       # 11 column tiles: row partition
    indexed_case([300, 77, 129], 256, 192, 512, dtype, True, env, lo=3, tail=3)   # rows no expert owns
    if variant == "0":
        indexed_case(BIG8, 2560, 512, 4096, dtype, False, dict(env, OPMX_MOE_GEMM_PERSIST="0"))
        indexed_case([300, 77, 129], 253, 2048, 4096, dtype, False, dict(env, OPMX_MOE_GEMM_STREAMK="2"))  # tail split over K


@pytest.mark.parametrize("variant", ["0", "2", "4"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_indexed_stream_kernels(variant, dtype):
    env = {"OPMX_MOE_GEMM": "stream", "OPMX_MOE_GEMM_STREAM_VARIANT": variant}
    for sizes, T in (([1, 0, 1, 0, 0, 0, 0, 0], 1), ([8, 9, 7, 11, 0, 16, 5, 8], 32), ([30, 2, 17, 0, 32, 1, 25, 21], 64),
                     ([64, 40, 0, 3, 50, 33, 1, 65], 128), ([128, 0, 0, 100, 7, 0, 0, 21], 128)):
        indexed_case(sizes, T, 512, 192, dtype, True, env)
        indexed_case(sizes, T, 4096, 2 * 128, dtype, False, env, swiglu=True)
    indexed_case([30, 2, 17, 0, 32, 1, 25, 21], 64, 4096, 2 * 4168, dtype, True, env, swiglu=True)   # SwiGLU by wave pairs
    indexed_case([64, 40, 0, 3, 50, 33, 1, 65], 128, 4104, 192, dtype, False, env)                  # K a multiple of 8 only


def test_indexed_rejects_bad_arguments():
    OPMX = opmx()
    d = dev()
    X = torch.randn(8, 64, device=d).half()
    W = torch.randn(2, 32, 64, device=d).half()
    off = torch.tensor([0, 8, 16], device=d)
    with pytest.raises(ValueError):      # int64 index
        OPMX.moe_column_parallel_linear_indexed(X, torch.zeros(16, dtype=torch.int64, device=d), off, W, None, 2, 64, 32)
    with pytest.raises(ValueError):      # not a whole number of picks per token
        OPMX.moe_column_parallel_linear_indexed(X, torch.zeros(15, dtype=torch.int32, device=d), off, W, None, 2, 64, 32)
    with pytest.raises(AssertionError):  # the reference's in_features assert
        OPMX.moe_column_parallel_linear_indexed(X, torch.zeros(16, dtype=torch.int32, device=d), off, W, None, 2, 63, 32)
    # indices outside X are clamped into it on the device, never read out of bounds
    bad = torch.tensor([0, 7, 100, -5] * 4, dtype=torch.int32, device=d)
    y = OPMX.moe_column_parallel_linear_indexed(X, bad, off, W, None, 2, 64, 32)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y.float()).all())
    # ... in every kernel family, to the same rows: an index below 0 reads row 0, one past the end the last row
    from torch_function import _lib
    T, K, N, R = 96, 128, 256, 672          # seven rows per token
    g = torch.Generator().manual_seed(3)
    Xb = torch.randn(T, K, generator=g).half().to(d)
    Wb = (torch.randn(2, N, K, generator=g) * 0.05).half().to(d)
    offb = torch.tensor([0, 300, R], device=d)
    idx = torch.randint(-50, T + 50, (R,), generator=g, dtype=torch.int32).to(d)
    want = None
    for env in ({"OPMX_MOE_GEMM": "generic"}, {"OPMX_MOE_GEMM": "stream"},
                {"OPMX_MOE_GEMM": "tiled", "OPMX_MOE_GEMM_TILED_VARIANT": "0"},
                {"OPMX_MOE_GEMM": "tiled", "OPMX_MOE_GEMM_TILED_VARIANT": "0", "OPMX_MOE_GEMM_PERSIST": "0"},
                {"OPMX_MOE_GEMM": "tiled", "OPMX_MOE_GEMM_TILED_VARIANT": "2"},
                {"OPMX_MOE_GEMM": "tiled", "OPMX_MOE_GEMM_TILED_VARIANT": "3"}):
        for key, val in env.items():
            _lib.set_option(key, val)
        try:
            got = OPMX.moe_column_parallel_linear_indexed(Xb, idx, offb, Wb, None, 2, K, N)
            if want is None:
                want = OPMX.moe_column_parallel_linear_indexed(Xb, idx.clamp(0, T - 1), offb, Wb, None, 2, K, N)
            torch.cuda.synchronize()
        finally:
            for key in env:
                _lib.set_option(key, None)
        assert float((got.float() - want.float()).abs().max()) <= 2e-2, env


def test_indexed_gemm_on_an_empty_batch():
    import torch_function as OPMX
    W = torch.zeros(4, 32, 64, dtype=torch.float16, device=dev())
    X = torch.zeros(0, 64, dtype=torch.float16, device=dev())
    rt = torch.zeros(0, dtype=torch.int32, device=dev())
    off = torch.zeros(5, dtype=torch.int64, device=dev())
    assert OPMX.moe_column_parallel_linear_indexed(X, rt, off, W, None, 4, 64, 32, num_experts_per_token=2).shape == (0, 2, 32)
    assert OPMX.moe_column_parallel_linear_indexed(X, rt, off, W, None, 4, 64, 32, swiglu=True,
                                                   num_experts_per_token=2).shape == (0, 2, 16)
    with pytest.raises(ValueError):      # rows that name tokens of an empty X
        OPMX.moe_column_parallel_linear_indexed(X, torch.zeros(2, dtype=torch.int32, device=dev()), off, W, None, 4, 64, 32)


@pytest.mark.parametrize("T,H,E,k,I,dtype,skew", [
    (32, 4096, 8, 2, 14336, torch.float16, 0.0), (128, 4096, 8, 2, 14336, torch.float16, 0.0),
    (2048, 4096, 8, 2, 14336, torch.float16, 1.5), (4096, 2048, 64, 8, 1408, torch.bfloat16, 0.0),
    (16, 6144, 8, 2, 16384, torch.float16, 0.0)])
def test_layer_with_the_gather_folded_into_the_gemm(T, H, E, k, I, dtype, skew):
    """Benchmark-shaped blocks: with the gather folded into the gate/up GEMM the block gives the bits
    of the operator-by-operator block, alone and together with the other fused forms (those
    against the oracle, routed by the logits the block's own router call returned)."""
    from test_gpu_layer import build_layer, check_fused_against_oracle, run_ops
    (x, Wg, wu, w2), host = gpu_inputs(T, H, E, I, dtype, seed=7)
    bias = O.zipf_router_bias(E, skew).to(dtype) if skew else None
    g = run_ops(x, Wg, wu, w2, E, k, bias=None if bias is None else bias.to(dev()))

    def layer(**kw):
        m = build_layer(H, I, E, k, dtype, Wg, wu, w2, **kw)
        if bias is not None:
            m.gate.bias = torch.nn.Parameter(bias.to(dev()), requires_grad=False)
        return m
    m = layer()
    m.fuse_x_gather = True
    assert torch.equal(m(x), g["out"]), "gather folded into the GEMM changes the block's output bits"
    for route in (False, True):
        mf = layer(fuse=True, route=route)
        mf.fuse_x_gather = True
        check_fused_against_oracle(mf, x, host, E, k, bias=bias, full=T <= 2048)
