"""GPU parity on seeded random shapes: many expert counts, ragged / empty segments, odd widths.

The fixed cases elsewhere sit on the boundaries the kernels were written around; these draw
shapes nobody chose (expert counts from 1 to 256, segments from empty to several row tiles, K any
multiple of 8 or 64, N anything) and send each through every grouped-GEMM family it admits, and
through MoeSelect / MoeReduce, against the CPU oracle.  Seeds are fixed: a failure names its case."""
import random

import pytest
import torch

from _util import assert_close_ulp, dev
from oracle import moe_oracle as O
from test_gpu_gemm import run_case
from test_gpu_layer import build_layer, check_against_oracle, run_ops
from test_gpu_select_reduce import check_select

pytestmark = pytest.mark.gpu


def draw_sizes(rng, E, style):
    if style == "sparse":          # most experts empty
        return [rng.choice([0, 0, 0, rng.randint(1, 40)]) for _ in range(E)]
    if style == "even":
        base = rng.randint(1, 300)
        return [max(0, base + rng.randint(-3, 3)) for _ in range(E)]
    if style == "skewed":          # a few big segments, many small
        return [rng.randint(200, 900) if rng.random() < 0.15 else rng.randint(0, 12) for _ in range(E)]
    return [rng.randint(0, 70) for _ in range(E)]


@pytest.mark.parametrize("seed", range(40))
def test_grouped_gemm_random(seed):
    rng = random.Random(1000 + seed)
    E = rng.choice([1, 2, 3, 8, 8, 16, 31, 64, 64, 100, 128, 256])
    style = rng.choice(["sparse", "even", "skewed", "ragged"])
    sizes = draw_sizes(rng, E, style)
    if E >= 64 and style == "even":
        sizes = [min(s, 40) for s in sizes]          # keep the case small
    if sum(sizes) == 0:
        sizes[rng.randrange(E)] = 5
    dtype = rng.choice([torch.float16, torch.bfloat16])
    K = rng.choice([64, 128, 192, 256, 512, 1024, 1408]) if rng.random() < 0.7 else 8 * rng.randint(1, 60)
    N = rng.choice([64, 128, 256, 320, 512]) if rng.random() < 0.6 else rng.randint(1, 400)
    bias = rng.random() < 0.5
    kind = rng.choice(["column", "row"])
    families = ["generic", "stream"] + (["tiled"] if K % 64 == 0 else [])
    for fam in families:
        run_case(kind, sizes, K, N, dtype, bias, {"OPMX_MOE_GEMM": fam}, seed=seed)
    if N % 2 == 0:
        for fam in families:
            run_case("column", sizes, K, N, dtype, bias, {"OPMX_MOE_GEMM": fam}, swiglu=True, seed=seed)
    run_case(kind, sizes, K, N, dtype, bias, None, seed=seed)      # automatic selection


@pytest.mark.parametrize("seed", range(24))
def test_grouped_gemm_random_fp32(seed):
    """float32 tensors: the library's own choice among the fp32 matrix-unit kernels, each of their forms forced
    (128-column tiles; 32-row tiles whose waves split K), and the shape-agnostic kernel, K any multiple of 4."""
    rng = random.Random(3000 + seed)
    E = rng.choice([1, 2, 3, 8, 8, 16, 31, 64, 100])
    style = rng.choice(["sparse", "even", "skewed", "ragged"])
    sizes = draw_sizes(rng, E, style)
    if E >= 16:
        sizes = [min(s, 150) for s in sizes]          # keep the float64 oracle quick
    if sum(sizes) == 0:
        sizes[rng.randrange(E)] = 5
    K = rng.choice([32, 64, 128, 256, 1024]) if rng.random() < 0.5 else 4 * rng.randint(1, 200)
    N = rng.choice([32, 64, 128, 256]) if rng.random() < 0.5 else rng.randint(1, 300)
    bias = rng.random() < 0.5
    kind = rng.choice(["column", "row"])
    for env in (None, {"OPMX_MOE_GEMM_F32_VARIANT": "0"}, {"OPMX_MOE_GEMM_F32_VARIANT": "1"}, {"OPMX_MOE_GEMM": "generic"}):
        run_case(kind, sizes, K, N, torch.float32, bias, env, seed=seed)
        if N % 2 == 0:
            run_case("column", sizes, K, N, torch.float32, bias, env, swiglu=True, seed=seed)


@pytest.mark.parametrize("seed", range(40))
def test_select_reduce_random(seed):
    rng = random.Random(5000 + seed)
    E = rng.choice([2, 5, 8, 8, 16, 32, 33, 64, 64, 128, 200, 256])
    k = rng.randint(1, min(E, 32))
    T = rng.choice([1, 2, 7, 16, 17, 31, 64, 65, 130, 256, 257, 700, 1500])
    H = rng.choice([8, 24, 64, 72, 256, 1000])
    dtype = rng.choice([torch.float16, torch.bfloat16, torch.float32])
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(T, H, generator=g).to(dtype)
    if rng.random() < 0.4:                           # many exact ties
        s = (torch.randint(-2, 3, (T, E), generator=g).float() * 0.5).to(dtype)
    else:
        s = torch.randn(T, E, generator=g).to(dtype)
    xe, w, inv, off = check_select(X, s, E, k)
    # MoeReduce on the same routing: gather, weight, sum
    import torch_function as OPMX
    Y = torch.randn(T * k, H, generator=g).to(dtype).view(T, k, H)
    out = OPMX.moe_reduce(Y.to(dev()), w, inv, k)
    ref = O.moe_reduce(Y, w.cpu(), inv.cpu(), k, acc=torch.float64, out_dtype=torch.float64)
    # a sum of k products: relative to the largest output where the terms cancel
    f32 = dtype == torch.float32
    assert_close_ulp(out, ref, dtype, ulps=16.0 if f32 else 2.0, what="moe_reduce", floor=0.25 if f32 else 0.02)


@pytest.mark.parametrize("seed", range(16))
def test_layer_random(seed):
    """The whole layer at random small sizes, operator by operator and through the block with its
    fused forms, against the oracle (routing bit-exact on the logits the path produced)."""
    from _util import gpu_inputs
    rng = random.Random(9000 + seed)
    E = rng.choice([2, 4, 8, 8, 16, 64, 128])
    k = rng.randint(1, min(E, 8))
    T = rng.choice([1, 3, 8, 9, 33, 100, 257, 600])
    H = rng.choice([64, 128, 256, 512])
    I = rng.choice([64, 192, 256, 704])
    dtype = rng.choice([torch.float16, torch.bfloat16])
    (x, Wg, wu, w2), host = gpu_inputs(T, H, E, I, dtype, seed=seed)
    g = run_ops(x, Wg, wu, w2, E, k)
    check_against_oracle(g, host, E, k)
    gr = run_ops(x, Wg, wu, w2, E, k, route=True)
    check_against_oracle(gr, host, E, k)
    for fuse, route, gather in ((True, False, False), (True, True, False), (False, False, True), (True, True, True)):
        m = build_layer(H, I, E, k, dtype, Wg, wu, w2, fuse=fuse, route=route, gather=gather)
        want = gr["out"] if route else g["out"]
        if not fuse:           # the gather alone changes no bit
            assert torch.equal(m(x), want)
            continue
        err = (m(x).double() - want.double()).abs()
        assert float(err.max()) <= 2e-2 and float(err.mean()) <= 2e-3, (fuse, route, gather, float(err.max()))
