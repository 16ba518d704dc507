"""ctypes binding of the plain-C oracle (``moe_oracle.c``).  TEST INFRASTRUCTURE ONLY.

Inputs are torch CPU tensors of any float dtype; they are up-cast exactly to
float32 for the C code, which accumulates in double.  Outputs are float32 /
int64 tensors; callers round to the dtype they compare against.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmoe_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
            os.path.join(_HERE, "moe_oracle.c")):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libmoe_oracle.so"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.oracle_moe_select.restype = ctypes.c_int
    return _lib


def _f32(t):
    return t.detach().to(torch.float32).contiguous()


def _p(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def moe_select(X, scores, E, k):
    """-> (X_expand [R,H] f32, weights [T,k] f32, inv [T,k] i64, off [E+1] i64, idx [T,k] i64)"""
    Xf, sf = _f32(X.reshape(-1, X.shape[-1])), _f32(scores.reshape(-1, E))
    T, H = Xf.shape
    idx = torch.empty(T, k, dtype=torch.int64)
    w = torch.empty(T, k, dtype=torch.float32)
    inv = torch.empty(T, k, dtype=torch.int64)
    off = torch.empty(E + 1, dtype=torch.int64)
    rc = lib().oracle_moe_select(_p(sf), ctypes.c_int64(T), E, k, _p(idx), _p(w), _p(inv), _p(off))
    assert rc == 0, rc
    Xp = torch.empty(T * k, H, dtype=torch.float32)
    lib().oracle_expand_rows(_p(Xf), ctypes.c_int64(T), ctypes.c_int64(H), k, _p(inv), _p(Xp))
    return Xp, w, inv, off, idx


def grouped_linear(X, off, W, B=None):
    E, N, K = W.shape
    Xf = _f32(X.reshape(-1, K))
    R = Xf.shape[0]
    Wf = _f32(W)
    Bf = _f32(B) if B is not None else None
    Y = torch.empty(R, N, dtype=torch.float32)
    lib().oracle_grouped_linear(_p(Xf), _p(off.to(torch.int64).contiguous()), _p(Wf), _p(Bf), E,
                                ctypes.c_int64(R), ctypes.c_int64(K), ctypes.c_int64(N), _p(Y))
    return Y


def linear(X, W, B=None):
    N, K = W.shape
    Xf = _f32(X.reshape(-1, K))
    Y = torch.empty(Xf.shape[0], N, dtype=torch.float32)
    lib().oracle_linear(_p(Xf), _p(_f32(W)), _p(_f32(B) if B is not None else None),
                        ctypes.c_int64(Xf.shape[0]), ctypes.c_int64(K), ctypes.c_int64(N), _p(Y))
    return Y


def swiglu(X, beta=1.0):
    D = X.shape[-1] // 2
    Xf = _f32(X.reshape(-1, 2 * D))
    Y = torch.empty(Xf.shape[0], D, dtype=torch.float32)
    lib().oracle_swiglu(_p(Xf), ctypes.c_int64(Xf.shape[0]), ctypes.c_int64(D), ctypes.c_float(beta), _p(Y))
    return Y


def silu(X, gate=None):
    Xf = _f32(X)
    Gf = _f32(gate) if gate is not None else None
    Y = torch.empty_like(Xf)
    lib().oracle_silu(_p(Xf), _p(Gf), ctypes.c_int64(Xf.numel()), _p(Y))
    return Y


def moe_reduce(Y, w, inv, k):
    N = Y.shape[-1]
    Yf, wf = _f32(Y.reshape(-1, N)), _f32(w.reshape(-1, k))
    T = wf.shape[0]
    out = torch.empty(T, N, dtype=torch.float32)
    lib().oracle_moe_reduce(_p(Yf), _p(wf), _p(inv.to(torch.int64).contiguous()), ctypes.c_int64(T), k,
                            ctypes.c_int64(N), _p(out))
    return out
