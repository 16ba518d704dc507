"""Shared eager path of the two grouped expert linears (one C-ABI call each)."""
import torch

from . import _lib


def grouped_linear(op, X, expert_offset, W, B, num_experts, epilogue=_lib.EPILOGUE_NONE, row_index=None,
                   rows_per_token=0):
    """``Y[off[e]:off[e+1]] = X[off[e]:off[e+1]] @ W[e]^T (+ B[e])`` on the GPU.

    ``op`` is "column" or "row".  Output dtype is ``W.dtype`` on ``X.device``
    (the reference's export branch states that dtype,
    ``MoeColumnParallelLinear.py:45``; its eager branch follows the process
    default dtype).  A row-parallel bias is applied per expert segment.
    ``row_index`` (int32 ``[R]``, column form only): GEMM row r is ``X.view(-1, K)[row_index[r]]``
    -- X holds the tokens and ``row_index`` is the ``row_token`` output of ``moe_select_index``;
    the result then has the shape ``[*, R / tokens, N]`` that the operator gives on
    ``X_expand_permute`` (an empty batch has no such ratio: ``rows_per_token`` names it then).
    """
    name = "moe_{}_parallel_linear".format(op)
    dev = _lib.require_gpu(name, X, expert_offset, W, B, row_index)
    E, N, K = W.shape
    if E != num_experts:
        raise ValueError("{}: W holds {} experts, num_experts is {}".format(name, E, num_experts))
    if X.shape[-1] != K:
        raise ValueError("{}: X has {} features, W expects {}".format(name, X.shape[-1], K))
    if expert_offset.numel() != E + 1:
        raise ValueError("{}: expert_offset must have num_experts + 1 entries".format(name))
    if X.dtype != W.dtype or (B is not None and B.dtype != W.dtype):
        raise TypeError("{}: X, W and B must share one dtype".format(name))
    if B is not None and tuple(B.shape) != (E, N):
        raise ValueError("{}: B must be [num_experts, out_features_per_partition]".format(name))
    dt = _lib.dtype_id(W, name)
    Xf = X.reshape(-1, K).contiguous()
    Wc = W.detach().contiguous()
    Bc = None if B is None else B.detach().contiguous()
    off = expert_offset.to(torch.int64).contiguous()
    tokens = Xf.shape[0]
    if row_index is not None:
        if op != "column" or row_index.dtype != torch.int32 or row_index.dim() != 1:
            raise ValueError("{}: row_index must be a 1-D int32 tensor (column form only)".format(name))
        if (tokens == 0 and row_index.numel() != 0) or (tokens != 0 and row_index.numel() % tokens):
            raise ValueError("{}: row_index has {} entries for {} rows of X".format(name, row_index.numel(), tokens))
        row_index = row_index.contiguous()
    R = tokens if row_index is None else row_index.numel()
    n_out = N // 2 if epilogue == _lib.EPILOGUE_SWIGLU else N
    # No bound on the rows of one expert is passed: the operator accepts any [*, K] input, so the
    # shape of X does not tell the token count, and the library then sizes its row tiles from
    # twice the mean rows per expert (the smaller of the two bounds in nearly every routing anyway).
    hint = 0
    Y = torch.empty(R, n_out, dtype=W.dtype, device=dev)
    L = _lib.lib()
    # optional scratch memory: with it the large-tile kernel balances its last rounds of tiles
    # over all CUs; small calls report a token size and run without
    ws = None
    ws_bytes = L.opmx_moe_grouped_gemm_workspace_bytes(E, R, K, N, dt)
    if ws_bytes > 256:
        ws = _lib.workspace(ws_bytes, dev)
    else:
        ws_bytes = 0
    if row_index is not None:
        rc = L.opmx_moe_column_parallel_linear_indexed(_lib.ptr(Xf), tokens, _lib.ptr(row_index), _lib.ptr(off), _lib.ptr(Wc),
                                                       _lib.ptr(Bc), E, R, K, N, dt, epilogue, hint, _lib.ptr(Y),
                                                       _lib.ptr(ws), ws_bytes, _lib.stream_ptr(dev))
    elif op == "column":
        rc = L.opmx_moe_column_parallel_linear(_lib.ptr(Xf), _lib.ptr(off), _lib.ptr(Wc), _lib.ptr(Bc), E, R, K, N,
                                               dt, epilogue, hint, _lib.ptr(Y), _lib.ptr(ws), ws_bytes,
                                               _lib.stream_ptr(dev))
    else:
        rc = L.opmx_moe_row_parallel_linear(_lib.ptr(Xf), _lib.ptr(off), _lib.ptr(Wc), _lib.ptr(Bc), E, R, K, N,
                                            dt, hint, _lib.ptr(Y), _lib.ptr(ws), ws_bytes, _lib.stream_ptr(dev))
    _lib.check(rc, name)
    if row_index is not None:
        return Y.view(*X.shape[:-1], R // tokens if tokens else int(rows_per_token), n_out)
    return Y.view(*X.shape[:-1], n_out)


def linear_attrs(num_experts, in_features, out_features, has_bias, **extra):
    """Attribute set shared by the two ``opmx::Moe*ParallelLinear`` nodes."""
    attrs = dict(num_experts_i=num_experts, in_features_i=in_features, out_features_i=out_features,
                 bias_term_i=bool(has_bias))
    attrs.update(extra)
    return attrs
