"""The Mixtral mixture-of-experts feed-forward block on the MI355X operators.

Only ``MoeFeedForward`` of the reference's Mixtral model is mirrored here
(``model_zoo/mixtral/modeling/dynamic_batching/Model.py:155-214`` of
OpenPPL/ppl.pmx): the six-operator sequence router gate -> MoeSelect ->
gate/up grouped GEMM -> SwiGLU -> down grouped GEMM -> MoeReduce, with the
fused weight layout ``wu[e] = [w1[e]; w3[e]]`` of ``Model.py:399-413``.
"""
import os
import sys
from types import SimpleNamespace

import torch
from torch import nn

sys.path.append(os.path.join(os.path.dirname(os.path.abspath(__file__)), "../../../.."))
import torch_function as OPMX  # noqa: E402
from model_zoo.ModelLayers import Linear  # noqa: E402
from model_zoo.ModelParallel import MoeColumnParallelLinear, MoeRowParallelLinear  # noqa: E402


class MoeFeedForward(nn.Module):
    """``args`` needs ``hidden_dim, intermediate_dim, num_experts, num_experts_per_token``
    (the fields of the reference's ``ModelParams`` this block reads).

    ``fuse_swiglu_epilogue=True`` (only with ``fused_ffn_glu``) applies SwiGLU
    inside the gate/up GEMM instead of as a separate operator; results agree
    to rounding, the ONNX graph does not change because export always takes
    the operator-by-operator route.
    """

    def __init__(self, args, layer_id: int, fused_ffn_glu: bool, linear_bias_term: bool, proc_group,
                 dtype=None, device=None, fuse_swiglu_epilogue: bool = False):
        super().__init__()
        self.layer_id = layer_id
        self.fused_ffn_glu = fused_ffn_glu
        self.fuse_swiglu_epilogue = fuse_swiglu_epilogue and fused_ffn_glu
        self.num_experts = args.num_experts
        self.num_experts_per_token = args.num_experts_per_token
        kw = dict(dtype=dtype, device=device)
        H, I, E = args.hidden_dim, args.intermediate_dim, args.num_experts
        self.gate = Linear(H, E, bias_term=False, **kw)
        if fused_ffn_glu:
            self.wu = MoeColumnParallelLinear(proc_group, E, H, 2 * I, bias_term=linear_bias_term,
                                              gather_output=False, **kw)
        else:
            self.w1 = MoeColumnParallelLinear(proc_group, E, H, I, bias_term=linear_bias_term,
                                              gather_output=False, **kw)
            self.w3 = MoeColumnParallelLinear(proc_group, E, H, I, bias_term=linear_bias_term,
                                              gather_output=False, **kw)
        self.w2 = MoeRowParallelLinear(proc_group, E, I, H, bias_term=linear_bias_term,
                                       input_is_parallel=True, **kw)

    @staticmethod
    def params(hidden_dim, intermediate_dim, num_experts, num_experts_per_token):
        return SimpleNamespace(hidden_dim=hidden_dim, intermediate_dim=intermediate_dim,
                               num_experts=num_experts, num_experts_per_token=num_experts_per_token)

    def forward(self, x):
        k = self.num_experts_per_token
        router_logits = self.gate(x)
        x_experts, expert_weights, invert_permutation, expert_offset = OPMX.moe_select(
            x, router_logits, self.num_experts, k)
        if self.fused_ffn_glu:
            if self.fuse_swiglu_epilogue and not torch.onnx.is_in_onnx_export():
                x13 = OPMX.moe_column_parallel_linear_swiglu(
                    x_experts, expert_offset, self.wu.weight, self.wu.bias, self.num_experts,
                    self.wu.in_features, self.wu.out_features)
            else:
                x13 = OPMX.swiglu(self.wu(x_experts, expert_offset))
        else:
            x13 = OPMX.silu(self.w1(x_experts, expert_offset), self.w3(x_experts, expert_offset))
        x_out = self.w2(x13, expert_offset)
        return OPMX.moe_reduce(x_out, expert_weights, invert_permutation, k)
