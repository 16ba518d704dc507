"""``opmx::Linear`` on MI355X, sized for the MoE router gate (few output features).

Drop-in for ``torch_function/Linear.py`` of OpenPPL/ppl.pmx (``F.linear(X, W, B)``,
``Linear.py:32``): fp32 accumulation, output in ``W.dtype``.
"""
import torch

from . import _lib


class Linear(torch.autograd.Function):
    @staticmethod
    def symbolic(g, X, W, B, in_features, out_features):
        inputs = [X, W] + ([B] if B is not None else [])
        return g.op("opmx::Linear", *inputs, in_features_i=in_features, out_features_i=out_features,
                    bias_term_i=B is not None)

    @staticmethod
    def forward(ctx, X, W, B, in_features, out_features):
        N, K = W.shape
        if torch.onnx.is_in_onnx_export():
            return torch.zeros(*X.shape[:-1], N, dtype=W.dtype, device=X.device)
        dev = _lib.require_gpu("linear", X, W, B)
        if X.shape[-1] != K:
            raise ValueError("linear: X has {} features, W expects {}".format(X.shape[-1], K))
        if X.dtype != W.dtype or (B is not None and B.dtype != W.dtype):
            raise TypeError("linear: X, W and B must share one dtype")
        dt = _lib.dtype_id(W, "linear")
        Xf = X.reshape(-1, K).contiguous()
        Wc = W.detach().contiguous()
        Bc = None if B is None else B.detach().contiguous()
        Y = torch.empty(Xf.shape[0], N, dtype=W.dtype, device=dev)
        _lib.check(_lib.lib().opmx_linear(_lib.ptr(Xf), _lib.ptr(Wc), _lib.ptr(Bc), Xf.shape[0], K, N, dt,
                                          _lib.ptr(Y), _lib.stream_ptr(dev)), "linear")
        return Y.view(*X.shape[:-1], N)


def linear(X: torch.Tensor, W: torch.Tensor, B: torch.Tensor, in_features: int, out_features: int):
    return Linear.apply(X, W, B, in_features, out_features)
