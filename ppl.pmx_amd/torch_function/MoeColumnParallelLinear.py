"""``opmx::MoeColumnParallelLinear`` on MI355X (grouped expert GEMM, N-sharded weights).

Drop-in for ``torch_function/MoeColumnParallelLinear.py`` of OpenPPL/ppl.pmx:
same positional signature and ONNX node; the eager branch
(``MoeColumnParallelLinear.py:58-69``) is one grouped-GEMM launch scheduled on
the device from ``expert_offset``.  Tensor-parallel world size must be 1.
"""
import torch

from . import _lib
from ._grouped import grouped_linear, linear_attrs


class MoeColumnParallelLinear(torch.autograd.Function):
    @staticmethod
    def symbolic(g, X, expert_offset, W, B, proc_group, num_experts, in_features, out_features,
                 gather_output=True):
        inputs = [X, expert_offset, W] + ([B] if B is not None else [])
        return g.op("opmx::MoeColumnParallelLinear", *inputs,
                    **linear_attrs(num_experts, in_features, out_features, B is not None,
                                   gather_output_i=gather_output))

    @staticmethod
    def forward(ctx, X, expert_offset, W, B, proc_group, num_experts, in_features, out_features,
                gather_output=True):
        assert X.shape[-1] == in_features, "X.shape is {}, in_features is {}".format(X.shape, in_features)
        ws = _lib.world_size(proc_group)
        if torch.onnx.is_in_onnx_export():
            part = torch.zeros(*X.shape[:-1], W.shape[1], dtype=W.dtype, device=X.device)
            return torch.cat([part] * ws, dim=-1) if (gather_output and ws > 1) else part
        if ws > 1:
            raise NotImplementedError("moe_column_parallel_linear: tensor parallel world size {} (this build "
                                      "covers one GPU, TP=1)".format(ws))
        return grouped_linear("column", X, expert_offset, W, B, num_experts)


def moe_column_parallel_linear(X, expert_offset, W, B, proc_group, num_experts: int, in_features: int,
                               out_features: int, gather_output: bool = True) -> torch.Tensor:
    return MoeColumnParallelLinear.apply(X, expert_offset, W, B, proc_group, num_experts, in_features,
                                         out_features, gather_output)


def moe_column_parallel_linear_swiglu(X, expert_offset, W, B, num_experts: int, in_features: int,
                                      out_features: int) -> torch.Tensor:
    """Fused form of ``swiglu(moe_column_parallel_linear(...))`` for the fused
    gate/up weight ``wu = [w1; w3]``: SwiGLU (beta = 1) is applied to the fp32
    accumulators, the [R, 2I] intermediate never reaches memory in the MFMA
    kernels.  No counterpart operator in the reference (it is the composition
    of ``Model.py:198`` and ``Model.py:200``); eager only."""
    assert X.shape[-1] == in_features, "X.shape is {}, in_features is {}".format(X.shape, in_features)
    return grouped_linear("column", X, expert_offset, W, B, num_experts, epilogue=_lib.EPILOGUE_SWIGLU)


def moe_column_parallel_linear_indexed(X, row_token, expert_offset, W, B, num_experts: int, in_features: int,
                                       out_features: int, swiglu: bool = False,
                                       num_experts_per_token: int = 0) -> torch.Tensor:
    """``moe_column_parallel_linear`` (or its SwiGLU form) on the rows ``X[row_token]``: ``X`` ``[*, K]``
    holds the tokens, ``row_token`` is the int32 index ``moe_select_index`` returns in place of
    ``X_expand_permute``.  Bit for bit the result of the operator on ``X_expand_permute``
    (``MoeSelect.py:45-47`` followed by ``MoeColumnParallelLinear.py:58-67``), ``[*, k, N]``, without the
    ``[T*k, K]`` copy ever being written or read.  ``num_experts_per_token`` only shapes the (empty)
    result of an empty batch, where ``row_token`` does not tell k.  No counterpart operator in the
    reference; eager only."""
    assert X.shape[-1] == in_features, "X.shape is {}, in_features is {}".format(X.shape, in_features)
    return grouped_linear("column", X, expert_offset, W, B, num_experts,
                          epilogue=_lib.EPILOGUE_SWIGLU if swiglu else _lib.EPILOGUE_NONE, row_index=row_token,
                          rows_per_token=num_experts_per_token)
