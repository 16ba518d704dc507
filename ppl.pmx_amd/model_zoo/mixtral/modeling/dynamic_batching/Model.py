"""The Mixtral mixture-of-experts feed-forward block on the MI355X operators.

Only ``MoeFeedForward`` of the reference's Mixtral model is mirrored here
(``model_zoo/mixtral/modeling/dynamic_batching/Model.py:155-214`` of
OpenPPL/ppl.pmx): the six-operator sequence router gate -> MoeSelect ->
gate/up grouped GEMM -> SwiGLU -> down grouped GEMM -> MoeReduce, with the
fused weight layout ``wu[e] = [w1[e]; w3[e]]`` of ``Model.py:399-413``, and the part
of ``Transformer.load_state_dict`` (``Model.py:363-420``) that fills it from an OPMX
checkpoint (``layers.N.feed_forward.{gate,w1,w2,w3}.weight`` with the expert
weights stacked ``[E, out, in]`` by
``model_zoo/mixtral/huggingface/ConvertWeightToOpmx.py:98-128``).
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

    The block computes what the reference's operator sequence computes and, by default, runs it
    through the three fused forms below (all flags ``False``: one launch sequence per reference
    operator, the form ``bench.py`` reports as its headline value; ONNX export always takes the
    operator-by-operator route, so the exported graph is the reference's either way).

    ``fuse_swiglu_epilogue=True`` (only with ``fused_ffn_glu``) applies SwiGLU
    inside the gate/up GEMM instead of as a separate operator; results agree
    to rounding, the ONNX graph does not change because export always takes
    the operator-by-operator route.  ``fuse_router_select=True`` does the same for the router
    gate and MoeSelect (one launch up to 8 tokens; the routing is exact on the logits that
    launch computes, which can differ from the separate gate's in the last bit).
    ``fuse_x_gather=True`` folds the token gather of MoeSelect (``MoeSelect.py:45-47``) into the
    operand load of the gate/up GEMM: MoeSelect then returns an index instead of
    ``X_expand_permute`` and the ``[T*k, H]`` copy is never written; same bits as the separate
    operators.
    """

    def __init__(self, args, layer_id: int, fused_ffn_glu: bool, linear_bias_term: bool, proc_group,
                 dtype=None, device=None, fuse_swiglu_epilogue: bool = True, fuse_router_select: bool = True,
                 fuse_x_gather: bool = True):
        super().__init__()
        self.fuse_x_gather = fuse_x_gather
        self.layer_id = layer_id
        self.fused_ffn_glu = fused_ffn_glu
        self.fuse_swiglu_epilogue = fuse_swiglu_epilogue and fused_ffn_glu
        self.fuse_router_select = fuse_router_select
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

    def _forward_indexed(self, x):
        """The block with MoeSelect as an index (``fuse_x_gather``): same operator order as ``forward``.
        -> (output, router logits)"""
        k, E = self.num_experts_per_token, self.num_experts
        if self.fuse_router_select:
            expert_weights, invert_permutation, expert_offset, row_token, router_logits = OPMX.moe_route_select_index(
                x, self.gate.weight, self.gate.bias, E, k)
        else:
            router_logits = self.gate(x)
            expert_weights, invert_permutation, expert_offset, row_token = OPMX.moe_select_index(router_logits, E, k)
        col = lambda m, swiglu=False: OPMX.moe_column_parallel_linear_indexed(
            x, row_token, expert_offset, m.weight, m.bias, E, m.in_features, m.out_features, swiglu=swiglu,
            num_experts_per_token=k)
        if self.fused_ffn_glu:
            x13 = col(self.wu, True) if self.fuse_swiglu_epilogue else OPMX.swiglu(col(self.wu))
        else:
            x13 = OPMX.silu(col(self.w1), col(self.w3))
        x_out = self.w2(x13, expert_offset)
        return OPMX.moe_reduce(x_out, expert_weights, invert_permutation, k), router_logits

    def forward(self, x, return_router_logits: bool = False):
        """``return_router_logits`` (not in the reference's signature, ``Model.py:187``): also return the
        router logits ``[*, E]`` the tokens were routed by, as the block's router call computed them."""
        k = self.num_experts_per_token
        if self.fuse_x_gather and not torch.onnx.is_in_onnx_export():
            out, router_logits = self._forward_indexed(x)
            return (out, router_logits) if return_router_logits else out
        if self.fuse_router_select and not torch.onnx.is_in_onnx_export():
            x_experts, expert_weights, invert_permutation, expert_offset, router_logits = OPMX.moe_route_select(
                x, self.gate.weight, self.gate.bias, self.num_experts, k)
        else:
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
        out = OPMX.moe_reduce(x_out, expert_weights, invert_permutation, k)
        return (out, router_logits) if return_router_logits else out

    @torch.no_grad()
    def load_state_dict(self, state_dict, strict: bool = True, prefix=None):
        """Fills this block from an OPMX state dict (``Model.py:363-420``).

        Keys are taken under ``prefix`` (default ``layers.<layer_id>.feed_forward.``): ``gate.weight``
        ``[E,H]``, ``w2.weight`` ``[E,H,I]`` and either ``wu.weight`` ``[E,2I,H]`` or the pair
        ``w1.weight`` / ``w3.weight`` ``[E,I,H]`` -- with ``fused_ffn_glu`` the pair lands in the two
        halves of ``wu`` (``Model.py:399-413``); biases likewise.  Tensors are copied into the existing
        parameters (their dtype and device win), nothing is re-tiled.  Returns the keys it used;
        ``strict`` raises on a parameter left without a value or a shape mismatch.
        """
        prefix = "layers.{}.feed_forward.".format(self.layer_id) if prefix is None else prefix
        params = dict(self.named_parameters())
        used, filled = [], set()

        def put(name, value, rows=None):
            dst = params[name]
            view = dst if rows is None else dst[:, rows[0]:rows[1]]
            if tuple(view.shape) != tuple(value.shape):
                raise ValueError("{}{}: checkpoint has {}, the block expects {}".format(
                    prefix, name, tuple(value.shape), tuple(view.shape)))
            view.copy_(value)
            filled.add((name, rows))

        for key, value in state_dict.items():
            if not key.startswith(prefix):
                continue
            name = key[len(prefix):]
            module, _, leaf = name.rpartition(".")
            if name in params:
                put(name, value)
            elif self.fused_ffn_glu and module in ("w1", "w3") and "wu." + leaf in params:
                half = params["wu." + leaf].shape[1] // 2
                put("wu." + leaf, value, (0, half) if module == "w1" else (half, 2 * half))
            else:
                continue
            used.append(key)
        if strict:
            for name in params:
                whole = (name, None) in filled
                halves = name.startswith("wu.") and all(
                    (name, r) in filled for r in ((0, params[name].shape[1] // 2),
                                                  (params[name].shape[1] // 2, params[name].shape[1])))
                if not (whole or halves):
                    raise KeyError("no value for {}{} in the checkpoint".format(prefix, name))
        return used


class GraphedMoeFeedForward(nn.Module):
    """Replays a ``MoeFeedForward`` from HIP graphs, one per input shape (no counterpart in the
    reference, whose model runs eagerly under ``torch.inference_mode``, ``Model.py:318``).

    With few tokens the six operators take a few microseconds of GPU time each and the host's launch
    path sets the pace; a serving loop captures the layer once per batch size and replays it.  The
    first call with a new shape runs the block once eagerly (kernel attributes are set on first
    launch), captures it on a side stream into static buffers, and every call copies the input in,
    replays, and returns the static output -- valid until the next call with the same shape; clone
    it to keep it.  ``max_graphs`` bounds the number of shapes kept (oldest dropped first).
    """

    def __init__(self, block: MoeFeedForward, max_graphs: int = 16):
        super().__init__()
        self.block = block
        self.max_graphs = max_graphs
        self._graphs = {}          # (shape, dtype, device) -> (graph, static input, static output)

    @torch.inference_mode()
    def forward(self, x):
        if torch.onnx.is_in_onnx_export() or not x.is_cuda:
            return self.block(x)
        key = (tuple(x.shape), x.dtype, x.device)
        entry = self._graphs.get(key)
        if entry is None:
            static_x = x.clone()
            side = torch.cuda.Stream(device=x.device)
            side.wait_stream(torch.cuda.current_stream(x.device))
            with torch.cuda.stream(side):
                self.block(static_x)
            torch.cuda.current_stream(x.device).wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_out = self.block(static_x)
            if len(self._graphs) >= self.max_graphs:
                self._graphs.pop(next(iter(self._graphs)))
            entry = self._graphs[key] = (graph, static_x, static_out)
        graph, static_x, static_out = entry
        static_x.copy_(x)
        graph.replay()
        return static_out


def load_opmx_moe_block(path, layer_id: int, num_experts_per_token: int, fused_ffn_glu: bool = True,
                        dtype=None, device=None, fuse_swiglu_epilogue: bool = True, fuse_router_select: bool = True,
                        fuse_x_gather: bool = True):
    """Builds the MoE block of layer ``layer_id`` from an OPMX Mixtral ``.pth`` checkpoint.

    The file is opened with ``weights_only=True`` and memory-mapped, so only this layer's tensors are
    read; sizes come from the tensors themselves (``gate.weight`` is ``[E,H]``, ``w2.weight``
    ``[E,H,I]``).  ``num_experts_per_token`` is not stored in the checkpoint (the reference reads it
    from ``opmx_params.json``).
    """
    sd = torch.load(path, map_location="cpu", weights_only=True, mmap=True)
    prefix = "layers.{}.feed_forward.".format(layer_id)
    gate, w2 = sd[prefix + "gate.weight"], sd[prefix + "w2.weight"]
    E, H = gate.shape
    bias = (prefix + "w2.bias") in sd
    block = MoeFeedForward(MoeFeedForward.params(H, w2.shape[2], E, num_experts_per_token), layer_id, fused_ffn_glu,
                           bias, None, dtype=gate.dtype if dtype is None else dtype, device=device,
                           fuse_swiglu_epilogue=fuse_swiglu_epilogue, fuse_router_select=fuse_router_select,
                           fuse_x_gather=fuse_x_gather)
    block.load_state_dict(sd)
    return block
