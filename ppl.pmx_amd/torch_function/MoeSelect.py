"""``opmx::MoeSelect`` on MI355X.

Drop-in for ``torch_function/MoeSelect.py`` of OpenPPL/ppl.pmx: same positional
signature, same ONNX node, same eager results (``MoeSelect.py:37-64``) with the
tie rule fixed to "lower expert id first".  The eager branch is one call into
``opmx_moe_select``.
"""
import torch

from . import _lib


class MoeSelect(torch.autograd.Function):
    @staticmethod
    def symbolic(g, X, scores, num_experts, num_experts_per_token):
        # node layout of MoeSelect.py:5-17: two inputs, two int attributes, four outputs
        outs = g.op("opmx::MoeSelect", X, scores, outputs=4,
                    num_experts_i=num_experts, num_experts_per_token_i=num_experts_per_token)
        return tuple(outs)

    @staticmethod
    def forward(ctx, X, scores, num_experts, num_experts_per_token):
        E, k = int(num_experts), int(num_experts_per_token)
        lead, H = tuple(X.shape[:-1]), X.shape[-1]
        if torch.onnx.is_in_onnx_export():
            # shape/dtype placeholders, returned in the eager (documented) order
            z = lambda *shape, dtype: torch.zeros(*shape, dtype=dtype, device=X.device)
            return (z(*lead, k, H, dtype=X.dtype), z(*lead, k, dtype=X.dtype),
                    z(*lead, k, dtype=torch.int64), z(E + 1, dtype=torch.int64))

        dev = _lib.require_gpu("moe_select", X, scores)
        if scores.shape[-1] != E or tuple(scores.shape[:-1]) != lead:
            raise ValueError("moe_select: scores shape {} does not match X {} / num_experts {}".format(
                tuple(scores.shape), tuple(X.shape), E))
        if scores.dtype != X.dtype:
            raise TypeError("moe_select: X and scores must share one dtype")
        if not (1 <= k <= E):
            raise ValueError("moe_select: need 1 <= num_experts_per_token <= num_experts")
        dt = _lib.dtype_id(X, "moe_select")
        Xf = X.reshape(-1, H).contiguous()
        sf = scores.reshape(-1, E).contiguous()
        T = Xf.shape[0]
        x_expand = torch.empty(T * k, H, dtype=X.dtype, device=dev)
        weights = torch.empty(T, k, dtype=scores.dtype, device=dev)
        inv = torch.empty(T * k, dtype=torch.int64, device=dev)
        off = torch.empty(E + 1, dtype=torch.int64, device=dev)
        L = _lib.lib()
        ws = _lib.workspace(L.opmx_moe_select_workspace_bytes(T, E, k), dev)
        _lib.check(L.opmx_moe_select(_lib.ptr(Xf), _lib.ptr(sf), T, H, E, k, dt, _lib.ptr(x_expand),
                                     _lib.ptr(weights), _lib.ptr(inv), _lib.ptr(off), None,
                                     _lib.ptr(ws), ws.numel(), _lib.stream_ptr(dev)), "moe_select")
        return (x_expand.view(*lead, k, H), weights.view(*lead, k), inv.view(*lead, k), off)


def moe_select(X: torch.Tensor, scores: torch.Tensor, num_experts: int, num_experts_per_token: int):
    """-> (X_expand_permute [*,k,H], expert_weights [*,k], invert_permutation [*,k] i64,
    expert_offset [E+1] i64)"""
    return MoeSelect.apply(X, scores, num_experts, num_experts_per_token)


def moe_route_select(X: torch.Tensor, gate_weight: torch.Tensor, gate_bias, num_experts: int,
                     num_experts_per_token: int):
    """Router gate and ``moe_select`` in one call (``Model.py:188-190`` of the reference:
    ``router_logits = self.gate(x)`` followed by ``OPMX.moe_select``).

    -> the four outputs of ``moe_select`` plus the router logits ``[*, E]``.  Three regimes inside the
    library (fp16/bf16): at most 8 tokens and 16 experts run as a single launch; beyond 256 tokens
    (up to 64 experts) the router kernel routes its tokens in its epilogue and MoeSelect starts from
    the picks; everything else runs the router kernel and the MoeSelect kernels one after the
    other.  The routing is exact on the logits the call returns in every regime.  Not an ONNX node:
    a model that is being exported calls ``linear`` and ``moe_select``.
    """
    E, k = int(num_experts), int(num_experts_per_token)
    lead, H = tuple(X.shape[:-1]), X.shape[-1]
    dev = _lib.require_gpu("moe_route_select", X, gate_weight, gate_bias)
    if tuple(gate_weight.shape) != (E, H):
        raise ValueError("moe_route_select: gate weight {} does not match [num_experts, hidden] = [{}, {}]".format(
            tuple(gate_weight.shape), E, H))
    if gate_weight.dtype != X.dtype or (gate_bias is not None and gate_bias.dtype != X.dtype):
        raise TypeError("moe_route_select: X, gate weight and gate bias must share one dtype")
    if not (1 <= k <= E):
        raise ValueError("moe_route_select: need 1 <= num_experts_per_token <= num_experts")
    dt = _lib.dtype_id(X, "moe_route_select")
    Xf = X.reshape(-1, H).contiguous()
    Wg = gate_weight.contiguous()
    Bg = None if gate_bias is None else gate_bias.contiguous()
    T = Xf.shape[0]
    scores = torch.empty(T, E, dtype=X.dtype, device=dev)
    x_expand = torch.empty(T * k, H, dtype=X.dtype, device=dev)
    weights = torch.empty(T, k, dtype=X.dtype, device=dev)
    inv = torch.empty(T * k, dtype=torch.int64, device=dev)
    off = torch.empty(E + 1, dtype=torch.int64, device=dev)
    L = _lib.lib()
    ws = _lib.workspace(L.opmx_moe_select_workspace_bytes(T, E, k), dev)
    _lib.check(L.opmx_moe_route_select(_lib.ptr(Xf), _lib.ptr(Wg), _lib.ptr(Bg), T, H, E, k, dt, _lib.ptr(scores),
                                       _lib.ptr(x_expand), _lib.ptr(weights), _lib.ptr(inv), _lib.ptr(off), None,
                                       _lib.ptr(ws), ws.numel(), _lib.stream_ptr(dev)), "moe_route_select")
    return (x_expand.view(*lead, k, H), weights.view(*lead, k), inv.view(*lead, k), off, scores.view(*lead, E))


def _select_index(X, scores, gate_weight, gate_bias, num_experts, num_experts_per_token, what):
    E, k = int(num_experts), int(num_experts_per_token)
    routed = scores is None                     # router gate in front: scores are an output
    ref = X if routed else scores
    lead = tuple(ref.shape[:-1])
    dev = _lib.require_gpu(what, X, scores, gate_weight, gate_bias)
    if not (1 <= k <= E):
        raise ValueError("{}: need 1 <= num_experts_per_token <= num_experts".format(what))
    dt = _lib.dtype_id(ref, what)
    if routed:
        H = X.shape[-1]
        if tuple(gate_weight.shape) != (E, H):
            raise ValueError("{}: gate weight {} does not match [num_experts, hidden] = [{}, {}]".format(
                what, tuple(gate_weight.shape), E, H))
        if gate_weight.dtype != X.dtype or (gate_bias is not None and gate_bias.dtype != X.dtype):
            raise TypeError("{}: X, gate weight and gate bias must share one dtype".format(what))
        Xf = X.reshape(-1, H).contiguous()
        T = Xf.shape[0]
        sf = torch.empty(T, E, dtype=X.dtype, device=dev)
    else:
        if scores.shape[-1] != E:
            raise ValueError("{}: scores shape {} does not match num_experts {}".format(what, tuple(scores.shape), E))
        sf = scores.reshape(-1, E).contiguous()
        T = sf.shape[0]
    weights = torch.empty(T, k, dtype=ref.dtype, device=dev)
    inv = torch.empty(T * k, dtype=torch.int64, device=dev)
    off = torch.empty(E + 1, dtype=torch.int64, device=dev)
    row_token = torch.empty(T * k, dtype=torch.int32, device=dev)
    L = _lib.lib()
    ws = _lib.workspace(L.opmx_moe_select_workspace_bytes(T, E, k), dev)
    if routed:
        Wg = gate_weight.contiguous()
        Bg = None if gate_bias is None else gate_bias.contiguous()
        rc = L.opmx_moe_route_select_index(_lib.ptr(Xf), _lib.ptr(Wg), _lib.ptr(Bg), T, H, E, k, dt, _lib.ptr(sf),
                                           _lib.ptr(weights), _lib.ptr(inv), _lib.ptr(off), _lib.ptr(row_token), None,
                                           _lib.ptr(ws), ws.numel(), _lib.stream_ptr(dev))
    else:
        rc = L.opmx_moe_select_index(_lib.ptr(sf), T, E, k, dt, _lib.ptr(weights), _lib.ptr(inv), _lib.ptr(off),
                                     _lib.ptr(row_token), None, _lib.ptr(ws), ws.numel(), _lib.stream_ptr(dev))
    _lib.check(rc, what)
    return weights.view(*lead, k), inv.view(*lead, k), off, row_token, sf.view(*lead, E)


def moe_select_index(scores: torch.Tensor, num_experts: int, num_experts_per_token: int):
    """``moe_select`` without the row copy (``MoeSelect.py:37-64`` except ``:45-47``).

    -> (expert_weights [*,k], invert_permutation [*,k] i64, expert_offset [E+1] i64, row_token [T*k] i32):
    the three routing outputs of ``moe_select``, bit for bit, and the index that stands for
    ``X_expand_permute``: its row r would be ``X[row_token[r]]``.  ``moe_column_parallel_linear_indexed``
    reads the tokens through it.  Not an ONNX node: a model that is being exported calls ``moe_select``."""
    return _select_index(None, scores, None, None, num_experts, num_experts_per_token, "moe_select_index")[:4]


def moe_route_select_index(X: torch.Tensor, gate_weight: torch.Tensor, gate_bias, num_experts: int,
                           num_experts_per_token: int):
    """Router gate followed by ``moe_select_index`` in one call (see ``moe_route_select``).

    -> (expert_weights, invert_permutation, expert_offset, row_token, router logits [*, E])."""
    return _select_index(X, None, gate_weight, gate_bias, num_experts, num_experts_per_token, "moe_route_select_index")
