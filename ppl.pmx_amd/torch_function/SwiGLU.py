"""``opmx::SwiGLU`` on MI355X.  Drop-in for ``torch_function/SwiGLU.py``
(``Y = g * x * sigmoid(beta * x)`` with x the first and g the second half of the
last dimension, ``SwiGLU.py:15-16``)."""
import torch

from . import _lib


class SwiGLU(torch.autograd.Function):
    @staticmethod
    def symbolic(g, X, beta=1.0):
        return g.op("opmx::SwiGLU", X, beta_f=beta)

    @staticmethod
    def forward(ctx, X, beta=1.0):
        D = X.shape[-1] // 2
        if torch.onnx.is_in_onnx_export():
            return torch.zeros(*X.shape[:-1], D, dtype=X.dtype, device=X.device)
        dev = _lib.require_gpu("swiglu", X)
        if X.shape[-1] != 2 * D:
            raise ValueError("swiglu: last dimension must be even")
        dt = _lib.dtype_id(X, "swiglu")
        Xf = X.reshape(-1, 2 * D).contiguous()
        Y = torch.empty(Xf.shape[0], D, dtype=X.dtype, device=dev)
        _lib.check(_lib.lib().opmx_swiglu(_lib.ptr(Xf), Xf.shape[0], D, float(beta), dt, _lib.ptr(Y),
                                          _lib.stream_ptr(dev)), "swiglu")
        return Y.view(*X.shape[:-1], D)


def swiglu(X: torch.Tensor, beta: float = 1.0):
    return SwiGLU.apply(X, beta)
