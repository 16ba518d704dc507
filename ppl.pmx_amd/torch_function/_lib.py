"""Loader and call glue for ``libopmx_moe.so`` (the C ABI in ``include/opmx_moe.h``).

PyTorch only supplies device memory and the current HIP stream here; every
number on the path is produced by the HIP kernels in the library.  There is no
CPU or eager-PyTorch fallback: if the library is missing, or a tensor is not on
a GPU, the operators raise.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_PKG_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG_ROOT, "lib", "libopmx_moe.so")
ABI_VERSION = 1

F32, F16, BF16 = 0, 1, 2
EPILOGUE_NONE, EPILOGUE_SWIGLU = 0, 1
MAX_EXPERTS, MAX_EXPERTS_PER_TOKEN = 256, 32
SELECT_STATIC_SCRATCH_BYTES = 4 << 20

_DTYPES = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}
_lib = None

_i64, _int, _vp, _sz, _f = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float
_SIGNATURES = {
    "opmx_moe_abi_version": (_int, []),
    "opmx_status_string": (ctypes.c_char_p, [_int]),
    "opmx_moe_set_option": (_int, [ctypes.c_char_p, _int]),
    "opmx_linear": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _vp, _vp]),
    "opmx_moe_select_workspace_bytes": (_sz, [_i64, _int, _int]),
    "opmx_moe_select": (_int, [_vp, _vp, _i64, _i64, _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "opmx_moe_select_static": (_int, [_vp, _vp, _i64, _i64, _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp]),
    "opmx_moe_route_select": (_int, [_vp, _vp, _vp, _i64, _i64, _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                     _sz, _vp]),
    "opmx_moe_select_index": (_int, [_vp, _i64, _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "opmx_moe_route_select_index": (_int, [_vp, _vp, _vp, _i64, _i64, _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp,
                                           _vp, _sz, _vp]),
    "opmx_moe_grouped_gemm_workspace_bytes": (_sz, [_int, _i64, _i64, _i64, _int]),
    "opmx_moe_column_parallel_linear_indexed": (_int, [_vp, _i64, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _int, _int,
                                                       _i64, _vp, _vp, _sz, _vp]),
    "opmx_moe_column_parallel_linear": (_int, [_vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _int, _int, _i64,
                                               _vp, _vp, _sz, _vp]),
    "opmx_moe_row_parallel_linear": (_int, [_vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _int, _i64,
                                            _vp, _vp, _sz, _vp]),
    "opmx_swiglu": (_int, [_vp, _i64, _i64, _f, _int, _vp, _vp]),
    "opmx_silu": (_int, [_vp, _vp, _i64, _int, _vp, _vp]),
    "opmx_rms_norm": (_int, [_vp, _vp, _vp, _i64, _i64, _f, _int, _vp, _vp, _vp]),
    "opmx_moe_reduce": (_int, [_vp, _vp, _vp, _i64, _int, _i64, _int, _vp, _vp]),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libopmx_moe.so not found at {}: build it with `make -C {}` (or "
                "__graft_entry__.build()). The OPMX MoE operators have no fallback path."
                .format(LIB_PATH, os.path.join(_PKG_ROOT, "csrc")))
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        if handle.opmx_moe_abi_version() != ABI_VERSION:
            raise RuntimeError("libopmx_moe.so ABI version mismatch")
        _lib = handle
    return _lib


def set_option(name: str, value) -> None:
    """Sets a tuning knob of the grouped GEMMs (``opmx_moe_set_option``); ``None`` = automatic.
    ``OPMX_MOE_GEMM`` also takes the words generic / tiled / stream."""
    if name == "OPMX_MOE_GEMM" and isinstance(value, str) and not value.isdigit():
        value = {"generic": 1, "tiled": 2, "stream": 3}[value]
    check(lib().opmx_moe_set_option(name.encode(), -1 if value is None else int(value)), "opmx_moe_set_option")


def check(status: int, what: str) -> None:
    if status != 0:
        raise RuntimeError("{} failed: {} ({})".format(what, lib().opmx_status_string(status).decode(), status))


def dtype_id(t: torch.Tensor, what: str) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError("{}: dtype {} is not supported (float32, float16, bfloat16)".format(what, t.dtype))


def require_gpu(what: str, *tensors: Optional[torch.Tensor]) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("{}: tensors must live on an MI355X device; this operator set has no CPU "
                               "path (got a {} tensor)".format(what, t.device))
        if dev is not None and t.device != dev:
            raise RuntimeError("{}: tensors are on different devices".format(what))
        dev = t.device
    return dev


def ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def stream_ptr(dev: torch.device):
    return torch.cuda.current_stream(dev).cuda_stream


def workspace(nbytes: int, dev: torch.device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=dev)


def world_size(proc_group) -> int:
    return 1 if proc_group is None else torch.distributed.get_world_size(group=proc_group)
