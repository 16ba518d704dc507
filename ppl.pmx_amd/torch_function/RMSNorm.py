"""``opmx::RMSNorm`` (with and without the skip term) on MI355X.  Drop-in for
``torch_function/RMSNorm.py``: ``rms_norm`` (``RMSNorm.py:16-24``) and
``skip_rms_norm`` (``RMSNorm.py:44-56``), same positional signatures, same ONNX
symbolics (``RMSNorm.py:6-11``, ``:29-39``)."""
import torch

from . import _lib


def _run(name, X, weight, SkipIn, axis, eps, want_skip_out):
    dev = _lib.require_gpu(name, X, weight, SkipIn)
    if axis not in (-1, X.dim() - 1):
        raise ValueError("{}: only the last axis is supported (axis={})".format(name, axis))
    H = X.shape[-1]
    if weight.numel() != H:
        raise ValueError("{}: weight has {} elements, the normalised axis {}".format(name, weight.numel(), H))
    if weight.dtype != X.dtype or (SkipIn is not None and SkipIn.dtype != X.dtype):
        raise TypeError("{}: X, weight and SkipIn must share one dtype".format(name))
    if SkipIn is not None and SkipIn.shape != X.shape:
        raise ValueError("{}: SkipIn must have the shape of X".format(name))
    dt = _lib.dtype_id(X, name)
    Xf = X.reshape(-1, H).contiguous()
    Sf = None if SkipIn is None else SkipIn.reshape(-1, H).contiguous()
    Wc = weight.detach().reshape(-1).contiguous()
    Y = torch.empty_like(Xf)
    So = torch.empty_like(Xf) if (want_skip_out and Sf is not None) else None
    _lib.check(_lib.lib().opmx_rms_norm(_lib.ptr(Xf), _lib.ptr(Wc), _lib.ptr(Sf), Xf.shape[0], H, float(eps), dt,
                                        _lib.ptr(Y), _lib.ptr(So), _lib.stream_ptr(dev)), name)
    Y = Y.view(X.shape)
    if not want_skip_out:
        return Y
    # without a skip input the reference returns X itself as the skip output (RMSNorm.py:49-50)
    return Y, (X if So is None else So.view(X.shape))


class RMSNorm(torch.autograd.Function):
    @staticmethod
    def symbolic(g, X, weight, axis=-1, eps=1e-5):
        Y = g.op("opmx::RMSNorm", X, weight, axis_i=axis, eps_f=eps, skip_term_i=False)
        return Y.setTypeAs(X)

    @staticmethod
    def forward(ctx, X, weight, axis=-1, eps=1e-5):
        if torch.onnx.is_in_onnx_export():
            return X
        return _run("rms_norm", X, weight, None, axis, eps, False)


class SkipRMSNorm(torch.autograd.Function):
    @staticmethod
    def symbolic(g, X, weight, SkipIn=None, axis=-1, eps=1e-5):
        if SkipIn is None:
            Y, SkipOut = g.op("opmx::RMSNorm", X, weight, axis_i=axis, eps_f=eps, skip_term_i=True, outputs=2)
        else:
            Y, SkipOut = g.op("opmx::RMSNorm", X, weight, SkipIn, axis_i=axis, eps_f=eps, skip_term_i=True,
                              outputs=2)
        return Y.setTypeAs(X), SkipOut.setTypeAs(X)

    @staticmethod
    def forward(ctx, X, weight, SkipIn=None, axis=-1, eps=1e-5):
        if torch.onnx.is_in_onnx_export():
            return X, X
        return _run("skip_rms_norm", X, weight, SkipIn, axis, eps, True)


def rms_norm(X: torch.Tensor, weight: torch.Tensor, axis: int = -1, eps: float = 1e-5) -> torch.Tensor:
    return RMSNorm.apply(X, weight, axis, eps)


def skip_rms_norm(X: torch.Tensor, weight: torch.Tensor, SkipIn: torch.Tensor = None, axis: int = -1,
                  eps: float = 1e-5):
    return SkipRMSNorm.apply(X, weight, SkipIn, axis, eps)
