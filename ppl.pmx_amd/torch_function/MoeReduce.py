"""``opmx::MoeReduce`` on MI355X: gather, expert weighting and sum in one kernel.

Drop-in for ``torch_function/MoeReduce.py`` of OpenPPL/ppl.pmx (eager semantics
``MoeReduce.py:23-25``).
"""
import torch

from . import _lib


class MoeReduce(torch.autograd.Function):
    @staticmethod
    def symbolic(g, Y, expert_weights, invert_permutation, num_experts_per_token):
        node = g.op("opmx::MoeReduce", Y, expert_weights, invert_permutation,
                    num_experts_per_token_i=num_experts_per_token)
        return node.setTypeAs(Y)          # MoeReduce.py:10-12

    @staticmethod
    def forward(ctx, Y, expert_weights, invert_permutation, num_experts_per_token):
        k, N = int(num_experts_per_token), Y.shape[-1]
        lead = tuple(expert_weights.shape[:-1])
        if torch.onnx.is_in_onnx_export():
            return torch.zeros(*lead, N, dtype=Y.dtype, device=Y.device)
        dev = _lib.require_gpu("moe_reduce", Y, expert_weights, invert_permutation)
        if expert_weights.shape[-1] != k or invert_permutation.numel() != expert_weights.numel():
            raise ValueError("moe_reduce: expert_weights / invert_permutation must be [*, {}]".format(k))
        if Y.numel() != expert_weights.numel() * N:
            raise ValueError("moe_reduce: Y must hold one row per (token, slot)")
        if expert_weights.dtype != Y.dtype:
            raise TypeError("moe_reduce: Y and expert_weights must share one dtype")
        dt = _lib.dtype_id(Y, "moe_reduce")
        Yf = Y.reshape(-1, N).contiguous()
        wf = expert_weights.reshape(-1, k).contiguous()
        inv = invert_permutation.reshape(-1).to(torch.int64).contiguous()
        T = wf.shape[0]
        out = torch.empty(T, N, dtype=Y.dtype, device=dev)
        _lib.check(_lib.lib().opmx_moe_reduce(_lib.ptr(Yf), _lib.ptr(wf), _lib.ptr(inv), T, k, N, dt,
                                              _lib.ptr(out), _lib.stream_ptr(dev)), "moe_reduce")
        return out.view(*lead, N)


def moe_reduce(Y: torch.Tensor, expert_weights: torch.Tensor, invert_permutation: torch.Tensor,
               num_experts_per_token: int):
    return MoeReduce.apply(Y, expert_weights, invert_permutation, num_experts_per_token)
