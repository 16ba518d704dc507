"""Parameter-holding wrappers of the two grouped expert linears.

Mirrors ``model_zoo/ModelParallel.py:127-196`` of OpenPPL/ppl.pmx (constructor
arguments, attribute names, parameter shapes ``[E, out/world, in]`` and
``[E, out, in/world]``, forward signature) so a Mixtral ``MoeFeedForward`` can
switch packages without edits.  ``dtype``/``device`` keywords are additions.
"""
import os
import sys

import torch
from torch import nn

sys.path.append(os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import torch_function as OPMX  # noqa: E402


def _world(proc_group):
    return 1 if proc_group is None else proc_group.size()


class _MoeLinearBase(nn.Module):
    def __init__(self, proc_group, num_experts, in_features, out_features, w_shape, b_shape, bias_term,
                 dtype, device):
        super().__init__()
        self.proc_group = proc_group
        self.num_experts = num_experts
        self.in_features = in_features
        self.out_features = out_features
        kw = dict(dtype=dtype, device=device)
        self.weight = nn.Parameter(torch.ones(*w_shape, **kw), requires_grad=False)
        if bias_term:
            self.bias = nn.Parameter(torch.zeros(*b_shape, **kw), requires_grad=False)
        else:
            self.register_parameter("bias", None)


class MoeColumnParallelLinear(_MoeLinearBase):
    def __init__(self, proc_group, num_experts: int, in_features: int, out_features: int,
                 bias_term: bool = True, gather_output: bool = True, dtype=None, device=None) -> None:
        world = _world(proc_group)
        assert out_features % world == 0, "{} is not divisible by {}".format(out_features, world)
        per_part = out_features // world
        super().__init__(proc_group, num_experts, in_features, out_features,
                         (num_experts, per_part, in_features), (num_experts, per_part), bias_term, dtype, device)
        self.out_features_per_partition = per_part
        self.gather_output = gather_output

    def forward(self, X: torch.Tensor, expert_offset: torch.Tensor):
        return OPMX.moe_column_parallel_linear(X, expert_offset, self.weight, self.bias, self.proc_group,
                                               self.num_experts, self.in_features, self.out_features,
                                               self.gather_output)


class MoeRowParallelLinear(_MoeLinearBase):
    def __init__(self, proc_group, num_experts: int, in_features: int, out_features: int,
                 bias_term: bool = True, input_is_parallel: bool = False, dtype=None, device=None) -> None:
        world = _world(proc_group)
        assert in_features % world == 0, "{} is not divisible by {}".format(in_features, world)
        per_part = in_features // world
        super().__init__(proc_group, num_experts, in_features, out_features,
                         (num_experts, out_features, per_part), (num_experts, out_features), bias_term, dtype,
                         device)
        self.in_features_per_partition = per_part
        self.input_is_parallel = input_is_parallel

    def forward(self, X: torch.Tensor, expert_offset: torch.Tensor):
        return OPMX.moe_row_parallel_linear(X, expert_offset, self.weight, self.bias, self.proc_group,
                                            self.num_experts, self.in_features, self.out_features,
                                            self.input_is_parallel)
