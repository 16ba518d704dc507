"""``opmx::SiLU`` on MI355X.  Drop-in for ``torch_function/SiLU.py``
(``gate * silu(X)``, or ``silu(X)`` without a gate, ``SiLU.py:18-21``); used by the
unfused gate/up form of the Mixtral expert FFN."""
import torch

from . import _lib


class SiLU(torch.autograd.Function):
    @staticmethod
    def symbolic(g, X, gate=None):
        node = g.op("opmx::SiLU", X) if gate is None else g.op("opmx::SiLU", X, gate)
        return node.setTypeAs(X)

    @staticmethod
    def forward(ctx, X, gate=None):
        if torch.onnx.is_in_onnx_export():
            return X
        dev = _lib.require_gpu("silu", X, gate)
        if gate is not None and (gate.shape != X.shape or gate.dtype != X.dtype):
            raise ValueError("silu: gate must match X in shape and dtype")
        dt = _lib.dtype_id(X, "silu")
        Xc = X.contiguous()
        Gc = None if gate is None else gate.contiguous()
        Y = torch.empty_like(Xc)
        _lib.check(_lib.lib().opmx_silu(_lib.ptr(Xc), _lib.ptr(Gc), Xc.numel(), dt, _lib.ptr(Y),
                                        _lib.stream_ptr(dev)), "silu")
        return Y


def silu(X: torch.Tensor, gate: torch.Tensor = None):
    return SiLU.apply(X, gate)
