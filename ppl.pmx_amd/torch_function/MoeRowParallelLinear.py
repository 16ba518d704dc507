"""``opmx::MoeRowParallelLinear`` on MI355X (grouped expert GEMM, K-sharded weights).

Drop-in for ``torch_function/MoeRowParallelLinear.py`` of OpenPPL/ppl.pmx
(eager semantics ``MoeRowParallelLinear.py:44-60`` at world size 1).  A bias,
if given, is ``[num_experts, out_features]`` and is added per expert segment.
"""
import torch

from . import _lib
from ._grouped import grouped_linear, linear_attrs


class MoeRowParallelLinear(torch.autograd.Function):
    @staticmethod
    def symbolic(g, X, expert_offset, W, B, proc_group, num_experts, in_features, out_features,
                 input_is_parallel=False):
        inputs = [X, expert_offset, W] + ([B] if B is not None else [])
        return g.op("opmx::MoeRowParallelLinear", *inputs,
                    **linear_attrs(num_experts, in_features, out_features, B is not None,
                                   input_is_parallel_i=input_is_parallel))

    @staticmethod
    def forward(ctx, X, expert_offset, W, B, proc_group, num_experts, in_features, out_features,
                input_is_parallel=False):
        if torch.onnx.is_in_onnx_export():
            return torch.zeros(*X.shape[:-1], W.shape[1], dtype=W.dtype, device=X.device)
        ws = _lib.world_size(proc_group)
        if ws > 1:
            raise NotImplementedError("moe_row_parallel_linear: tensor parallel world size {} (this build "
                                      "covers one GPU, TP=1)".format(ws))
        return grouped_linear("row", X, expert_offset, W, B, num_experts)


def moe_row_parallel_linear(X, expert_offset, W, B, proc_group, num_experts: int, in_features: int,
                            out_features: int, input_is_parallel: bool = False):
    return MoeRowParallelLinear.apply(X, expert_offset, W, B, proc_group, num_experts, in_features,
                                      out_features, input_is_parallel)
