"""Router gate module.  Mirrors ``model_zoo/ModelLayers.py:51-69`` of
OpenPPL/ppl.pmx (weight ``[out_features, in_features]``, optional bias)."""
import os
import sys

import torch
from torch import nn

sys.path.append(os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import torch_function as OPMX  # noqa: E402


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
