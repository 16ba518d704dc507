"""MI355X-native implementation of the OPMX mixture-of-experts operators.

Import it the way the reference's consumers import theirs
(``import torch_function as OPMX`` with this package's parent directory on
``sys.path``); the functions below keep the reference's names and positional
signatures (``torch_function/__init__.py:15,17-20,29-30,37-38`` of OpenPPL/ppl.pmx):
the seven operators of the MoE layer and the RMSNorm pair in front of it, plus fused forms that
are not ONNX nodes (gate/up GEMM with SwiGLU, router gate with MoeSelect, and MoeSelect as an
index that the gate/up GEMM reads the tokens through, without the expanded copy).
"""
from .Linear import linear
from .MoeColumnParallelLinear import (moe_column_parallel_linear, moe_column_parallel_linear_indexed,
                                      moe_column_parallel_linear_swiglu)
from .MoeReduce import moe_reduce
from .MoeRowParallelLinear import moe_row_parallel_linear
from .MoeSelect import moe_route_select, moe_route_select_index, moe_select, moe_select_index
from .RMSNorm import rms_norm, skip_rms_norm
from .SiLU import silu
from .SwiGLU import swiglu

__all__ = ["linear", "moe_column_parallel_linear", "moe_column_parallel_linear_indexed",
           "moe_column_parallel_linear_swiglu", "moe_reduce", "moe_route_select", "moe_route_select_index",
           "moe_row_parallel_linear", "moe_select", "moe_select_index", "rms_norm", "silu", "skip_rms_norm", "swiglu"]
