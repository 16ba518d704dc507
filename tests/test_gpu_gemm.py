"""GPU parity: grouped expert GEMMs (generic, MFMA-tiled and weight-streaming
kernels, bias, SwiGLU epilogue, ragged / empty / partial offsets) against the CPU
oracle on identical inputs.  Tolerance: 2 ulp of the output dtype (one rounding
plus fp32 accumulation order), relative to max(|ref|, 2% of max|ref|)."""
import os

import pytest
import torch

from _util import assert_close_ulp, dev
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def opmx():
    import torch_function as OPMX
    return OPMX


def offsets(sizes):
    return torch.tensor([0] + list(torch.tensor(sizes).cumsum(0).tolist()), dtype=torch.int64)


def run_case(kind, sizes, K, N, dtype, bias, env=None, swiglu=False, lead3=False, off=None, R=None, seed=0):
    """kind: 'column' | 'row'.  sizes: rows per expert."""
    OPMX = opmx()
    E = len(sizes)
    off = offsets(sizes) if off is None else off
    R = int(sum(sizes)) if R is None else R
    g = torch.Generator().manual_seed(seed + K + N + R)
    X = torch.randn(R, K, generator=g).to(dtype)
    W = (torch.randn(E, N, K, generator=g) * 0.05).to(dtype)
    B = torch.randn(E, N, generator=g).to(dtype) if bias else None
    if lead3 == "batch":                       # [1, R, K]: leading dimensions say nothing about the routing
        X = X.view(1, R, K)
    elif lead3:                                # [T, k, K] as MoeSelect returns it
        X = X.view(R // 2, 2, K)
    from torch_function import _lib
    for key, val in (env or {}).items():      # tuning knobs: force a kernel family / variant
        _lib.set_option(key, val)
    try:
        args = (X.to(dev()), off.to(dev()), W.to(dev()), None if B is None else B.to(dev()))
        if swiglu:
            Y = OPMX.moe_column_parallel_linear_swiglu(*args, E, K, N)
        elif kind == "column":
            Y = OPMX.moe_column_parallel_linear(*args, None, E, K, N, False)
        else:
            Y = OPMX.moe_row_parallel_linear(*args, None, E, K, N, True)
        torch.cuda.synchronize()
    finally:
        for key in (env or {}):
            _lib.set_option(key, None)         # back to automatic
    ref = O.moe_column_parallel_linear(X, off, W, B, acc=torch.float64, out_dtype=torch.float64)
    if swiglu:
        ref = O.swiglu(ref, acc=torch.float64)
    assert Y.dtype == dtype and Y.shape == ref.shape
    f32 = dtype == torch.float32
    assert_close_ulp(Y, ref, dtype, ulps=64 if f32 else 2, floor=0.25 if f32 else 0.02,
                     what="{} {} K{} N{} {} {}".format(kind, sizes, K, N, dtype, env))
    return Y


RAGGED8 = [5, 0, 17, 1, 0, 64, 3, 38]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("swiglu", [False, True])
def test_generic_kernel(dtype, swiglu):
    env = {"OPMX_MOE_GEMM": "generic"}
    run_case("column", RAGGED8, 72, 100, dtype, True, env, swiglu=swiglu)
    run_case("row", [3, 130, 0, 70], 50, 66, dtype, False, env, swiglu=swiglu)
    run_case("column", [1], 8, 2, dtype, True, env, swiglu=swiglu)


def test_tiny_config_fp32_shapes():
    """The CPU-runnable reference config: H=1024, I=2816, E=8, fp32."""
    sizes = [20, 9, 31, 0, 16, 25, 12, 15]
    run_case("column", sizes, 1024, 5632, torch.float32, False)
    run_case("row", sizes, 2816, 1024, torch.float32, False)
    run_case("column", sizes, 1024, 5632, torch.float32, True, swiglu=True)


@pytest.mark.parametrize("swiglu", [False, True])
def test_fp32_matrix_unit_kernel(swiglu):
    """fp32 tensors with K a multiple of 4 go to the fp32 MFMA kernels: 32-row tiles whose waves split K
    (few rows per expert, or few tiles), 32- and 128-row tiles of 128 columns; ragged / empty / one-row
    experts, K that is no multiple of the 32-wide k-tile, N that is no multiple of the W tile, bias;
    against the float64 oracle, and close to the shape-agnostic kernel (both accumulate in fp32, in
    different orders)."""
    few = [5, 0, 17, 1, 0, 31, 3, 38]
    many = [300, 0, 129, 1, 256, 77, 0, 513]
    # the library's own choice, the 128-column tile forms (32- or 128-row tiles) and the form whose waves split K
    for variant in (None, "0", "1"):
        env = {} if variant is None else {"OPMX_MOE_GEMM_F32_VARIANT": variant}
        for sizes in (few, many):
            for kind, K, N, bias in (("column", 128, 512, False), ("row", 100, 72, True), ("column", 36, 200, True),
                                     ("row", 1024, 130, False), ("column", 4, 8, True), ("row", 2816, 96, True)):
                if swiglu and (kind == "row" or N % 2):
                    continue
                a = run_case(kind, sizes, K, N, torch.float32, bias, env, swiglu=swiglu)
                if variant is None:
                    b = run_case(kind, sizes, K, N, torch.float32, bias, {"OPMX_MOE_GEMM": "generic"}, swiglu=swiglu)
                    assert float((a - b).abs().max()) <= 1e-4 * max(1.0, float(b.abs().max()))
        y = run_case("column", [9, 0, 20], 256, 64, torch.float32, True, env, off=torch.tensor([2, 11, 11, 31]), R=40, swiglu=swiglu)
        assert float(y[:2].abs().max()) == 0.0 and float(y[31:].abs().max()) == 0.0
    # rows that belong to no expert stay zero; K % 4 != 0 falls back to the shape-agnostic kernel
    off = torch.tensor([3, 40, 40, 100], dtype=torch.int64)
    y = run_case("column", [37, 0, 60], 64, 96, torch.float32, True, off=off, R=110, swiglu=swiglu)
    assert float(y[:3].abs().max()) == 0.0 and float(y[100:].abs().max()) == 0.0
    run_case("column", few, 50, 64, torch.float32, True, swiglu=swiglu)


@pytest.mark.parametrize("variant", ["0", "1", "2", "3"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_tiled_kernel_variants(variant, dtype):
    env = {"OPMX_MOE_GEMM": "tiled", "OPMX_MOE_GEMM_TILED_VARIANT": variant}
    sizes = [300, 0, 129, 1, 256, 77, 0, 513]
    run_case("column", sizes, 256, 512, dtype, False, env)
    run_case("row", sizes, 448, 384, dtype, True, env)
    run_case("column", sizes, 128, 200, dtype, True, env)                 # N not a tile multiple
    run_case("column", sizes, 192, 512, dtype, True, env, swiglu=True)
    run_case("column", sizes, 64, 1000, dtype, False, env, swiglu=True)   # D=500: ragged epilogue tile


@pytest.mark.parametrize("variant", ["0", "1", "2", "3"])
def test_tile_order_with_partial_last_round(variant):
    """16 column tiles and 24 row tiles: one full 16 x 16 round in the XCD-grouped order plus
    eight row tiles dealt out by the remainder rule; SwiGLU case: 16 column tiles of 128."""
    env = {"OPMX_MOE_GEMM": "tiled", "OPMX_MOE_GEMM_TILED_VARIANT": variant}
    sizes = [1500, 0, 700, 33, 1281, 256, 5, 1300]
    run_case("column", sizes, 128, 4096, torch.float16, True, env)
    run_case("column", sizes, 128, 4096, torch.bfloat16, False, env, swiglu=True)
    run_case("row", [4096], 192, 4096, torch.float16, False, env)          # exactly one full round


@pytest.mark.parametrize("variant", ["0", "1", "3"])
def test_expert_major_and_row_partition_tile_orders(variant):
    """Tile orders of the 256-row kernels.  Expert-major (column tiles divisible by 8): experts
    with 16-row-tile bands plus leftovers (4200 rows = 17 tiles, 5000 = 20), empty and one-row
    experts, 8 and 24 column tiles.  Row partition (any other column-tile count): 3 and 11 column
    tiles, more and fewer row tiles than XCDs.  Every tile must be computed exactly once: the
    output starts out uninitialised."""
    env = {"OPMX_MOE_GEMM": "tiled", "OPMX_MOE_GEMM_TILED_VARIANT": variant}
    big = [4200, 0, 300, 5000, 17, 256, 1, 2100]
    run_case("column", big, 128, 2048, torch.float16, True, env)
    run_case("row", big, 64, 6144, torch.bfloat16, False, env)
    run_case("column", big, 128, 4096, torch.float16, False, env, swiglu=True)    # 16 column tiles of 128
    run_case("column", big, 64, 768, torch.float16, True, env)                   # 3 column tiles
    run_case("row", [300, 0, 129], 128, 2816, torch.bfloat16, False, env)         # 11 column tiles, 4 row tiles
    run_case("column", [70] * 19, 64, 2816, torch.float16, False, env, swiglu=True)   # 19 row tiles, 11 column tiles of 128


@pytest.mark.parametrize("variant", ["0", "3"])
def test_expert_grouped_tile_order(variant):
    """The order for many small experts (each XCD owns a contiguous eighth of the tiles strung
    together expert by expert): chosen by itself up to four row tiles per expert on average,
    forced here for experts with more than one row group of 8 as well.  Tile counts that are and
    are not multiples of 8, fewer tiles than XCDs, empty experts, 11 and 8 column tiles, the
    persistent form walking several tiles per workgroup; same bits as the expert-major order."""
    env = {"OPMX_MOE_GEMM": "tiled", "OPMX_MOE_GEMM_TILED_VARIANT": variant, "OPMX_MOE_GEMM_GNX": "32"}
    g = torch.Generator().manual_seed(7)
    small = [int(v) for v in torch.randint(480, 545, (64,), generator=g)]      # two or three row tiles of 256 each
    small[5] = small[40] = 0
    a = run_case("column", small, 128, 2816, torch.bfloat16, False, env)          # 11 column tiles
    b = run_case("column", small, 128, 2816, torch.bfloat16, False, dict(env, OPMX_MOE_GEMM_GNX="16"))
    assert torch.equal(a, b)
    a = run_case("row", small, 192, 2048, torch.float16, True, env)               # 8 column tiles
    b = run_case("row", small, 192, 2048, torch.float16, True, dict(env, OPMX_MOE_GEMM_GNX="8"))
    assert torch.equal(a, b)
    run_case("column", small, 64, 4096, torch.float16, True, env, swiglu=True)
    run_case("column", [4200, 0, 300, 5000, 17, 256, 1, 2100], 128, 2048, torch.float16, True, env)   # row groups of 8 + rest
    run_case("row", [3], 64, 256, torch.float16, False, env)                      # one tile
    run_case("row", [300, 0, 129], 128, 768, torch.bfloat16, False, env)          # 9 (variant 3: 15) tiles
    # what the library picks by itself for this shape
    run_case("column", small, 128, 2816, torch.bfloat16, False, {"OPMX_MOE_GEMM": "tiled", "OPMX_MOE_GEMM_TILED_VARIANT": variant})


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("variant", ["0", "3"])
def test_persistent_kernel_streams_tiles(dtype, variant):
    """The persistent form of the 256x256 and of the 128x256 kernel (16 column tiles, K >= 256): fewer
    tiles than workgroups, then 27 (128-row tiles: 50) row tiles x 16 so that workgroups walk on to a
    second tile (ragged row tiles, bias, SwiGLU with 16 column tiles of 128), K = 256 being the
    shortest stream it takes; the one-tile-per-workgroup form must give the same bits."""
    env = {"OPMX_MOE_GEMM": "tiled", "OPMX_MOE_GEMM_TILED_VARIANT": variant, "OPMX_MOE_GEMM_STREAMK": "0"}
    sizes = [1500, 0, 700, 33, 1281, 256, 5, 1300, 1024, 300]
    run_case("column", [300, 77, 129], 256, 4096, dtype, True, env)
    for K, bias, swiglu in ((256, False, False), (320, True, False), (512, True, True), (1024, False, True)):
        a = run_case("column", sizes, K, 4096, dtype, bias, env, swiglu=swiglu)
        b = run_case("column", sizes, K, 4096, dtype, bias, dict(env, OPMX_MOE_GEMM_PERSIST="0"), swiglu=swiglu)
        assert torch.equal(a, b)
    # row-partition order (11 column tiles), several tiles per workgroup, uneven XCD shares (27 row tiles)
    a = run_case("column", sizes, 256, 2816, dtype, True, env)
    b = run_case("column", sizes, 256, 2816, dtype, True, dict(env, OPMX_MOE_GEMM_PERSIST="0"))
    assert torch.equal(a, b)
    # a long K, where the persistent form is taken only on request
    a = run_case("row", sizes, 8192, 512, dtype, False, dict(env, OPMX_MOE_GEMM_PERSIST="1"))
    b = run_case("row", sizes, 8192, 512, dtype, False, dict(env, OPMX_MOE_GEMM_PERSIST="0"))
    assert torch.equal(a, b)
    # with the tail of the last round split over k by the second launch
    run_case("row", sizes, 1024, 4096, dtype, True, dict(env, OPMX_MOE_GEMM_STREAMK="2"))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_tail_tiles_split_over_k(dtype):
    """Few tiles (4 row tiles x 16 column tiles, 2-D tile order) and a long K: the tail launch of
    the 256x256 kernel cuts every tile into k-ranges whose fp32 partial sums meet in the workspace
    (K=2048: 4 ranges, K=1024: 2)."""
    env = {"OPMX_MOE_GEMM": "tiled", "OPMX_MOE_GEMM_TILED_VARIANT": "0", "OPMX_MOE_GEMM_STREAMK": "2"}   # 2: always split
    sizes = [300, 77, 129]
    a = run_case("row", sizes, 2048, 4096, dtype, True, env)
    run_case("column", sizes, 1024, 4096, dtype, False, env, swiglu=True)     # 16 column tiles of 128
    run_case("column", [700, 300, 1], 1024, 4096, dtype, False, env)          # 6 x 16 tiles
    # same result bit for bit on a second call (summation order is fixed); close to the unsplit one
    b = run_case("row", sizes, 2048, 4096, dtype, True, env)
    assert torch.equal(a, b)
    c = run_case("row", sizes, 2048, 4096, dtype, True, dict(env, OPMX_MOE_GEMM_STREAMK="0"))
    assert (a.float() - c.float()).abs().max() <= 2e-2 * max(1.0, float(c.float().abs().max()))
    # the 128 x 256 tile form of the kernel (half-size partial tiles)
    run_case("row", sizes, 2048, 4096, dtype, True, dict(env, OPMX_MOE_GEMM_TILED_VARIANT="3"))
    # a K long enough for the default policy to split (144 k-tiles, 8 ranges)
    if dtype == torch.float16:
        run_case("row", [200, 60], 9216, 4096, dtype, False, {"OPMX_MOE_GEMM": "tiled", "OPMX_MOE_GEMM_TILED_VARIANT": "0"})


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_stream_two_row_tiles(dtype):
    """Calls with at most two rows in all and K >= 4096 stage two X rows per tile instead of sixteen:
    one token with two experts, two rows of one expert, a single row; one-wave and four-wave blocks
    (few and many weight rows), a ragged last K chunk, bias, and the SwiGLU form by wave pairs
    (N/2 >= 8192 columns for two active experts)."""
    env = {"OPMX_MOE_GEMM": "stream"}
    for sizes in ([1, 0, 1, 0, 0, 0, 0, 0], [0, 0, 0, 2, 0, 0, 0, 0], [0, 1], [1]):
        run_case("column", sizes, 4096, 192, dtype, True, env)              # one-wave blocks
        run_case("row", sizes, 4096 + 72, 320, dtype, False, env)           # ragged last chunk
        run_case("column", sizes, 4096, 33000, dtype, True, env)            # four-wave blocks, N not a multiple of 64
        run_case("column", sizes, 4096, 2 * 8256, dtype, True, env, swiglu=True)
    run_case("column", [1, 0, 1, 0], 8192, 2 * 192, dtype, False, env, swiglu=True)   # few columns: the narrow SwiGLU form


@pytest.mark.parametrize("variant", ["0", "1", "2", "3", "4", "5"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_stream_kernel_variants(variant, dtype):
    env = {"OPMX_MOE_GEMM": "stream", "OPMX_MOE_GEMM_STREAM_VARIANT": variant}
    for sizes in ([1, 0, 1, 0, 0, 0, 0, 0],               # T=1 decode: two active experts
                  [8, 9, 7, 11, 0, 16, 5, 8],             # <= 16 rows per expert
                  [30, 2, 17, 0, 32, 1, 25, 21],          # <= 32
                  [64, 40, 0, 3, 50, 33, 1, 65],          # <= 64 (+ one expert with a second tile)
                  [128, 0, 0, 100, 7, 0, 0, 21]):
        run_case("column", sizes, 512, 192, dtype, False, env, lead3=False)
        run_case("row", sizes, 1408, 128, dtype, True, env)           # K not a multiple of the K-chunk
    run_case("column", [8, 9, 7, 11, 0, 16, 5, 8], 256, 100, dtype, True, env)      # N not a multiple of 64
    run_case("column", [8, 9, 7, 11, 0, 16, 5, 8], 264, 128, dtype, True, env)      # K % 8 == 0 only
    run_case("column", [8, 9, 7, 11, 0, 16, 5, 8], 512, 256, dtype, True, env, swiglu=True)
    run_case("column", [4] * 64, 256, 128, dtype, False, env)                       # 64 experts
    # many weight rows: 4-wave blocks (the small cases above run the 1-wave blocks), ragged last slab
    run_case("column", [8, 9, 7, 11, 0, 16, 5, 8], 256, 4200, dtype, True, env)
    run_case("row", [30, 2, 17, 0, 32, 1, 25, 21], 512, 4160, dtype, False, env)
    # 16 and more K chunks: every block starts its walk over K somewhere else and wraps around,
    # also through a ragged last chunk and in the SwiGLU form
    run_case("row", [8, 9, 7, 11, 0, 16, 5, 8], 8192 + 72, 320, dtype, True, env)
    run_case("column", [30, 2, 17, 0, 32, 1, 25, 21], 4096, 2 * 192, dtype, False, env, swiglu=True)
    # K below 4096 takes narrower K chunks (all the cases above but the last two): the wide-chunk
    # kernels for single rows and for 64-row tiles, and the narrow SwiGLU one for single rows
    run_case("column", [1, 0, 1, 0, 0, 0, 0, 0], 4096, 192, dtype, True, env)
    run_case("row", [64, 40, 0, 3, 50, 33, 1, 65], 4096 + 64, 192, dtype, False, env)
    run_case("column", [1, 0, 1, 0, 0, 0, 1, 0], 1408, 2 * 128, dtype, True, env, swiglu=True)
    run_case("column", [1, 0, 1, 0, 0, 0, 1, 0], 4096, 2 * 128, dtype, False, env, swiglu=True)
    # SwiGLU form with a long K and many weight rows: gate and up rows streamed by pairs of waves
    run_case("column", [30, 2, 17, 0, 32, 1, 25, 21], 4096, 2 * 4168, dtype, True, env, swiglu=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_automatic_selection_and_hint(dtype):
    # [T, k, K] input, as MoeSelect returns it
    run_case("column", [10, 6, 0, 16, 8, 8, 9, 7], 512, 256, dtype, False, lead3=True)
    run_case("column", [700, 6, 0, 16, 800, 8, 90, 428], 512, 256, dtype, False, lead3=True)
    # a 3-D input that is not [T, k, K]: experts with thousands of rows behind a leading 1
    run_case("column", [1500, 6, 0, 1600, 800, 8, 90, 428], 512, 256, dtype, False, lead3="batch")
    run_case("row", [40, 6, 0, 16, 80, 8, 90, 16], 512, 256, dtype, False, lead3="batch")
    run_case("row", [700, 6, 0, 16, 800, 8, 90, 428], 512, 256, dtype, True)
    if dtype != torch.float32:
        # K a multiple of 8 but not of 64 with many rows: the stream kernel's 128-row tiles, not the FMA fallback
        run_case("column", [700, 6, 0, 16, 800, 8, 90, 428], 520, 256, dtype, True)
        run_case("row", [700, 6, 0, 16, 800, 8, 90, 428], 1000, 192, dtype, False)


@pytest.mark.parametrize("force", ["generic", "tiled", "stream"])
def test_rows_owned_by_no_expert_are_zero(force):
    """off = arange(E+1) with more rows than experts is the reference's own demo
    input (MoeColumnParallelLinear.py:135-136): row e uses expert e, the rest stay 0.
    Also offsets that start after row 0."""
    E, K, N = 8, 128, 192
    env = {"OPMX_MOE_GEMM": force}
    Y = run_case("column", [1] * E, K, N, torch.float16, True, env, off=torch.arange(E + 1), R=80)
    assert torch.count_nonzero(Y[E:]) == 0
    off = torch.tensor([5, 5, 9, 20, 20, 31, 40, 41, 60])
    Y = run_case("row", [0] * E, K, N, torch.float16, False, env, off=off, R=64)
    assert torch.count_nonzero(Y[:5]) == 0 and torch.count_nonzero(Y[60:]) == 0


def test_argument_errors():
    OPMX = opmx()
    d = dev()
    X = torch.zeros(4, 2, 64, device=d, dtype=torch.float16)
    off = torch.tensor([0, 8], device=d)
    W = torch.zeros(1, 32, 64, device=d, dtype=torch.float16)
    with pytest.raises(AssertionError):                       # MoeColumnParallelLinear.py:40
        OPMX.moe_column_parallel_linear(X, off, W, None, None, 1, 63, 32, False)
    with pytest.raises(TypeError):
        OPMX.moe_column_parallel_linear(X.float(), off, W, None, None, 1, 64, 32, False)
    with pytest.raises(RuntimeError):
        OPMX.moe_row_parallel_linear(X.cpu(), off.cpu(), W.cpu(), None, None, 1, 64, 32, True)
    Y = OPMX.moe_row_parallel_linear(X[:0], torch.zeros(2, dtype=torch.int64, device=d), W, None, None, 1, 64, 32)
    assert Y.shape == (0, 2, 32)


@pytest.mark.parametrize("force", ["generic", "tiled", "stream"])
def test_fewer_rows_than_experts(force):
    """One token routed to 8 of 64 experts: 8 rows, each its own expert's only row.  The launch
    is sized by the row count (every tile holds at least one row), not by the expert count."""
    env = {"OPMX_MOE_GEMM": force}
    sizes = [0] * 64
    for e in (3, 4, 17, 30, 31, 40, 62, 63):
        sizes[e] = 1
    run_case("column", sizes, 256, 192, torch.bfloat16, True, env)
    run_case("row", sizes, 128, 320, torch.float16, False, env)
    run_case("column", sizes, 256, 2 * 96, torch.float16, True, env, swiglu=True)
    one = [0] * 64
    one[63] = 1                                   # a single row, for the last expert
    run_case("row", one, 128, 64, torch.float16, True, env)
    two = [0] * 64
    two[0], two[63] = 2, 1                        # three rows in two tiles
    run_case("column", two, 256, 128, torch.float16, False, env)
