"""CPU checks of the drop-in boundary: the C-ABI library loads, exports every
symbol the header declares (and nothing undeclared), and rejects bad arguments
before touching a device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "opmx_moe.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(opmx_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from torch_function import _lib
    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    return _lib.lib()


def test_header_and_library_agree(lib):
    from torch_function import _lib
    names = declared_functions()
    assert len(names) >= 11
    for n in names:
        assert hasattr(lib, n), "library does not export " + n
    assert sorted(_lib.EXPORTED_SYMBOLS) == names, "python binding and header list different entry points"
    assert lib.opmx_moe_abi_version() == 1


def test_status_strings(lib):
    assert lib.opmx_status_string(0) == b"ok"
    for code in (-1, -2, -3, -4, -5):
        assert lib.opmx_status_string(code) not in (b"ok", b"unknown status")
    assert lib.opmx_status_string(-99) == b"unknown status"


def test_argument_validation_needs_no_device(lib):
    """Every rejection below happens on the host; nothing is enqueued."""
    P = ctypes.c_void_p
    one = P(256)          # never dereferenced on these paths
    assert lib.opmx_moe_select(one, one, 4, 8, 8, 9, 1, one, one, one, one, None, one, 1 << 20, None) == -1  # k > E
    assert lib.opmx_moe_select(one, one, 4, 8, 300, 2, 1, one, one, one, one, None, one, 1 << 20, None) == -2  # E
    assert lib.opmx_moe_select(one, one, 4, 8, 64, 33, 1, one, one, one, one, None, one, 1 << 20, None) == -2  # k
    assert lib.opmx_moe_select(one, one, 4, 8, 8, 2, 7, one, one, one, one, None, one, 1 << 20, None) == -2   # dtype
    assert lib.opmx_moe_select(one, one, 4, 8, 8, 2, 1, one, one, one, one, None, None, 0, None) == -3      # workspace
    assert lib.opmx_moe_select(one, one, 4, 8, 8, 2, 1, one, one, one, one, None, P(8), 1 << 20, None) == -4  # align
    assert lib.opmx_moe_select(None, one, 4, 8, 8, 2, 1, one, one, one, one, None, one, 1 << 20, None) == -1
    # the variant with the library's own scratch array: same checks, and sizes beyond the array
    from torch_function import _lib
    st = lambda *a: lib.opmx_moe_select_static(*a)
    assert st(one, one, 4, 8, 8, 9, 1, one, one, one, one, None, None) == -1    # k > E
    assert st(one, one, 4, 8, 300, 2, 1, one, one, one, one, None, None) == -2  # E
    assert st(one, one, 4, 8, 8, 2, 7, one, one, one, one, None, None) == -2    # dtype
    assert st(None, one, 4, 8, 8, 2, 1, one, one, one, one, None, None) == -1
    assert lib.opmx_moe_select_workspace_bytes(1 << 20, 8, 2) > _lib.SELECT_STATIC_SCRATCH_BYTES
    assert st(one, one, 1 << 20, 64, 8, 2, 1, one, one, one, one, None, None) == -3   # 8 MB of ids alone
    assert lib.opmx_moe_select_workspace_bytes(1 << 18, 64, 8) > _lib.SELECT_STATIC_SCRATCH_BYTES
    assert st(one, one, 1 << 18, 64, 64, 8, 2, one, one, one, one, None, None) == -3
    # router gate + select in one call: the argument checks of opmx_moe_select
    rs = lambda *a: lib.opmx_moe_route_select(*a)
    assert rs(one, one, None, 4, 8, 8, 9, 1, one, one, one, one, one, None, one, 1 << 20, None) == -1   # k > E
    assert rs(one, one, None, 4, 8, 300, 2, 1, one, one, one, one, one, None, one, 1 << 20, None) == -2  # E
    assert rs(one, one, None, 4, 8, 8, 2, 7, one, one, one, one, one, None, one, 1 << 20, None) == -2   # dtype
    assert rs(one, one, None, 4, 8, 8, 2, 1, one, one, one, one, one, None, None, 0, None) == -3        # workspace
    assert rs(one, None, None, 4, 8, 8, 2, 1, one, one, one, one, one, None, one, 1 << 20, None) == -1  # gate weight
    assert rs(one, one, None, 4, 8, 8, 2, 1, None, one, one, one, one, None, one, 1 << 20, None) == -1  # scores
    # MoeSelect as an index, and the GEMM that reads its rows through it
    si = lambda *a: lib.opmx_moe_select_index(*a)
    assert si(one, 4, 8, 9, 1, one, one, one, one, None, one, 1 << 20, None) == -1      # k > E
    assert si(one, 4, 300, 2, 1, one, one, one, one, None, one, 1 << 20, None) == -2    # E
    assert si(one, 4, 8, 2, 1, one, one, one, None, None, one, 1 << 20, None) == -1     # no row_token
    assert si(one, 4, 8, 2, 1, one, one, one, one, None, None, 0, None) == -3           # workspace
    rsi = lambda *a: lib.opmx_moe_route_select_index(*a)
    assert rsi(one, None, None, 4, 8, 8, 2, 1, one, one, one, one, one, None, one, 1 << 20, None) == -1   # gate weight
    assert rsi(one, one, None, 4, 8, 8, 2, 1, one, one, one, one, None, None, one, 1 << 20, None) == -1   # no row_token
    gi = lambda *a: lib.opmx_moe_column_parallel_linear_indexed(*a)
    assert gi(one, 4, None, one, one, None, 8, 8, 64, 32, 1, 0, 0, one, None, 0, None) == -1    # no index
    assert gi(one, 0, one, one, one, None, 8, 8, 64, 32, 1, 0, 0, one, None, 0, None) == -1     # X without rows
    assert gi(one, 4, one, one, one, None, 8, 8, 64, 33, 1, 1, 0, one, None, 0, None) == -1     # SwiGLU needs an even N
    assert gi(None, 0, None, None, None, None, 8, 0, 64, 32, 1, 0, 0, None, None, 0, None) == 0  # empty
    assert lib.opmx_moe_column_parallel_linear(one, one, one, None, 8, 4, 64, 33, 1, 1, 0, one, None, 0, None) == -1
    assert lib.opmx_moe_column_parallel_linear(one, None, one, None, 8, 4, 64, 32, 1, 0, 0, one, None, 0, None) == -1
    assert lib.opmx_moe_row_parallel_linear(one, one, one, None, 999, 4, 64, 32, 1, 0, one, None, 0, None) == -2
    assert lib.opmx_moe_reduce(one, one, one, 4, 40, 8, 1, one, None) == -2
    assert lib.opmx_moe_reduce(one, one, one, -1, 2, 8, 1, one, None) == -1
    assert lib.opmx_swiglu(None, 4, 8, 1.0, 1, one, None) == -1
    assert lib.opmx_silu(one, None, 8, 9, one, None) == -2
    assert lib.opmx_linear(one, one, None, 4, 0, 8, 1, one, None) == -1
    assert lib.opmx_rms_norm(one, None, None, 4, 8, 1e-5, 1, one, None, None) == -1      # no weight
    assert lib.opmx_rms_norm(one, one, None, 4, 8, -1.0, 1, one, None, None) == -1       # eps < 0
    assert lib.opmx_rms_norm(one, one, None, 4, 8, 1e-5, 5, one, None, None) == -2       # dtype
    assert lib.opmx_rms_norm(None, None, None, 0, 8, 1e-5, 1, None, None, None) == 0     # empty
    # empty problems are no-ops that succeed
    assert lib.opmx_moe_reduce(None, None, None, 0, 2, 8, 1, None, None) == 0
    assert lib.opmx_swiglu(None, 0, 8, 1.0, 1, None, None) == 0
    assert lib.opmx_moe_row_parallel_linear(None, None, None, None, 8, 0, 64, 32, 1, 0, None, None, 0, None) == 0


def test_tuning_knobs(lib):
    assert lib.opmx_moe_set_option(b"OPMX_MOE_GEMM", 2) == 0
    assert lib.opmx_moe_set_option(b"OPMX_MOE_GEMM", -1) == 0          # back to automatic
    for name in (b"OPMX_MOE_GEMM_TILED_VARIANT", b"OPMX_MOE_GEMM_STREAM_VARIANT", b"OPMX_MOE_GEMM_GNX",
                 b"OPMX_MOE_GEMM_STREAMK", b"OPMX_MOE_GEMM_PERSIST", b"OPMX_MOE_ROUTE_INDEX_TOKENS", b"OPMX_MOE_GEMM_F32_VARIANT"):
        assert lib.opmx_moe_set_option(name, -1) == 0
    assert lib.opmx_moe_set_option(b"OPMX_NO_SUCH_KNOB", 1) == -1
    assert lib.opmx_moe_set_option(None, 1) == -1


def test_workspace_sizes(lib):
    assert lib.opmx_moe_select_workspace_bytes(0, 8, 2) >= 256
    small = lib.opmx_moe_select_workspace_bytes(32, 8, 2)
    big = lib.opmx_moe_select_workspace_bytes(8192, 8, 2)
    assert small % 256 == 0 and big % 256 == 0 and big >= 8192 * 2 * 4 + 32 * 8 * 4 > small
    g = lib.opmx_moe_grouped_gemm_workspace_bytes(8, 64, 4096, 28672, 1)
    assert g >= 256 and g % 256 == 0      # epilogues run in registers: a token workspace is enough
