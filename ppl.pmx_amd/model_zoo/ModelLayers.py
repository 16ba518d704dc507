"""Router gate module and the norm in front of the MoE layer.  Mirror
``model_zoo/ModelLayers.py:32-69`` of OpenPPL/ppl.pmx (``RMSNorm``, ``SkipRMSNorm``: weight
``[dim]`` of ones; ``Linear``: weight ``[out_features, in_features]``, optional bias)."""
import os
import sys

import torch
from torch import nn

sys.path.append(os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import torch_function as OPMX  # noqa: E402


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-6, dtype=None, device=None):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim, dtype=dtype, device=device), requires_grad=False)

    def forward(self, x):
        return OPMX.rms_norm(x, self.weight, -1, self.eps)


class SkipRMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-6, dtype=None, device=None):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim, dtype=dtype, device=device), requires_grad=False)

    def forward(self, x, skip):
        return OPMX.skip_rms_norm(x, self.weight, skip, -1, self.eps)


class Linear(nn.Module):
    def __init__(self, in_features: int, out_features: int, bias_term: bool = True, dtype=None,
                 device=None) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.weight = nn.Parameter(torch.ones(out_features, in_features, dtype=dtype, device=device),
                                   requires_grad=False)
        if bias_term:
            self.bias = nn.Parameter(torch.zeros(out_features, dtype=dtype, device=device), requires_grad=False)
        else:
            self.register_parameter("bias", None)

    def forward(self, X: torch.Tensor):
        return OPMX.linear(X, self.weight, self.bias, self.in_features, self.out_features)
