"""CPU oracle for the OPMX mixture-of-experts path.  TEST INFRASTRUCTURE ONLY.

This module restates, on PyTorch CPU tensors, what the reference operators
compute.  It is the checker for the HIP kernels: only the test-suite, the
smoke check and the ``cpu_baseline`` leg of the benchmark may import it.  The
product package never does.

Reference files restated (paths relative to the OpenPPL/ppl.pmx checkout):

* ``torch_function/Linear.py:32``                    -> :func:`linear`
* ``torch_function/MoeSelect.py:37-64``              -> :func:`moe_select`
* ``torch_function/MoeColumnParallelLinear.py:58-69``-> :func:`moe_column_parallel_linear`
* ``torch_function/SwiGLU.py:15-16``                 -> :func:`swiglu`
* ``torch_function/SiLU.py:18-21``                   -> :func:`silu`
* ``torch_function/MoeRowParallelLinear.py:44-60``   -> :func:`moe_row_parallel_linear`
* ``torch_function/MoeReduce.py:23-25``              -> :func:`moe_reduce`
* ``torch_function/RMSNorm.py:16-24,44-56``          -> :func:`rms_norm`, :func:`skip_rms_norm`
* ``model_zoo/mixtral/modeling/dynamic_batching/Model.py:187-214`` -> :func:`moe_layer`

Third-party arithmetic: the reference delegates every number to PyTorch
(``requirements.txt:5``, unpinned; ``model_zoo/mixtral/huggingface/requirements.txt:5``
pins torch==2.0.1).  The reference holds no test, golden vector or fixture for
these operators, so parity is pinned by: closed forms from library routines
(stable sort, bincount, cumsum), structural invariants, brute force on tiny
inputs, the permutation-free dense formulation in float64
(:func:`moe_layer_dense_fp64`) and an independent plain-C restatement
(``moe_oracle.c``).  See ``tests/test_oracle_*.py``.

Two deliberate, documented departures from the literal reference code:

* top-k ties go to the LOWER expert id (``torch.topk`` leaves tie order
  unspecified, ``MoeSelect.py:40``); NaN scores rank above every number, as
  in ``torch.topk``/``torch.sort``; -0.0 equals +0.0.
* the grouped linears produce ``W.dtype`` output on ``X.device`` (the
  reference's ``torch.zeros`` without dtype, ``MoeColumnParallelLinear.py:59``,
  follows the process default) and the row-parallel bias is applied per expert
  row-segment (``MoeRowParallelLinear.py:59-60`` broadcasts the whole [E,N]
  tensor, which only works for ``B is None``).

All arithmetic is done in ``acc`` precision (float32 by default, float64 on
request) on up-cast inputs and rounded ONCE to the output dtype, which is what
"fp32-accumulated reference" means in the parity bar.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

__all__ = [
    "linear", "topk_lower_id", "moe_select", "moe_column_parallel_linear",
    "moe_row_parallel_linear", "swiglu", "silu", "moe_reduce", "moe_layer",
    "moe_layer_dense_fp64", "make_inputs", "zipf_router_bias", "moe_select_as_written",
]


def _acc(t: torch.Tensor, acc: torch.dtype) -> torch.Tensor:
    return t.to(acc)


# --------------------------------------------------------------------------
# a1  router gate                                               Linear.py:32
# --------------------------------------------------------------------------
def linear(X: torch.Tensor, W: torch.Tensor, B: Optional[torch.Tensor] = None,
           acc: torch.dtype = torch.float32, out_dtype: Optional[torch.dtype] = None):
    """``F.linear(X, W, B)`` with ``acc`` accumulation, rounded once."""
    out_dtype = out_dtype or W.dtype
    Y = _acc(X, acc) @ _acc(W, acc).transpose(-1, -2)
    if B is not None:
        Y = Y + _acc(B, acc)
    return Y.to(out_dtype)


# --------------------------------------------------------------------------
# a2  MoeSelect                                          MoeSelect.py:37-64
# --------------------------------------------------------------------------
def topk_lower_id(scores: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Top-k along the last dim ordered by (value descending, id ascending).

    ``MoeSelect.py:40`` + the tie rule.  A stable descending sort keeps equal
    values in ascending index order, so its first k columns ARE the rule.
    Comparison happens on the exact float32 image of the scores (fp16/bf16
    up-cast exactly), so no tie is created or destroyed by the cast.
    """
    s = scores.to(torch.float32)
    s = torch.where(s == 0, torch.zeros_like(s), s)          # -0.0 == +0.0
    v, idx = torch.sort(s, dim=-1, descending=True, stable=True)
    idx = idx[..., :k].contiguous()
    vals = torch.gather(scores, -1, idx)
    return vals, idx


def moe_select(X: torch.Tensor, scores: torch.Tensor, num_experts: int,
               num_experts_per_token: int, acc: torch.dtype = torch.float32,
               return_indices: bool = False):
    """Restates ``MoeSelect.forward`` (eager branch, ``MoeSelect.py:37-64``).

    Returns ``(X_expand_permute [*,k,H], expert_weights [*,k],
    invert_permutation [*,k] int64, expert_offset [E+1] int64)``; with
    ``return_indices`` also the picked expert ids ``[*,k]`` int64.
    """
    E, k = int(num_experts), int(num_experts_per_token)
    assert scores.shape[-1] == E and 0 < k <= E
    lead = X.shape[:-1]
    Xf = X.reshape(-1, X.shape[-1])
    sf = scores.reshape(-1, E)
    T = Xf.shape[0]
    R = T * k

    vals, idx = topk_lower_id(sf, k)                                   # :40
    w = torch.softmax(_acc(vals, acc), dim=-1).to(scores.dtype)       # :41
    flat = idx.reshape(-1)                                             # :42
    _, perm = torch.sort(flat, stable=True)                            # :44
    Xp = Xf.repeat_interleave(k, dim=0)[perm]                          # :45-47
    inv = torch.empty(R, dtype=torch.int64)
    inv[perm] = torch.arange(R, dtype=torch.int64)                     # :49-52
    counts = torch.bincount(flat, minlength=E)[:E]
    off = torch.zeros(E + 1, dtype=torch.int64)
    off[1:] = torch.cumsum(counts, 0)                                  # :54-60
    out = (Xp.view(*lead, k, Xf.shape[-1]), w.view(*lead, k), inv.view(*lead, k), off)
    if return_indices:
        return out + (idx.view(*lead, k),)
    return out


def moe_select_as_written(X, scores, num_experts, num_experts_per_token, acc=torch.float32):
    """Same results as :func:`moe_select`, but with the bookkeeping done the way the
    reference does it: one interpreted loop over the R sorted positions to invert the
    permutation (``MoeSelect.py:49-52``) and a pointer walk over the sorted expert ids
    for the offsets (``MoeSelect.py:54-60``).  Only used as the "as-written" CPU
    baseline of the benchmark and to cross-check the vectorised form."""
    E, k = int(num_experts), int(num_experts_per_token)
    lead = X.shape[:-1]
    Xf = X.reshape(-1, X.shape[-1])
    vals, idx = topk_lower_id(scores.reshape(-1, E), k)
    w = torch.softmax(_acc(vals, acc), dim=-1).to(scores.dtype)
    sorted_ids, perm = torch.sort(idx.reshape(-1), stable=True)
    Xp = Xf.repeat_interleave(k, dim=0)[perm]
    R = perm.numel()
    inv = torch.full((R,), -1, dtype=torch.int64)
    for i in range(R):                                   # per-element tensor get/set
        inv[perm[i]] = i
    off = torch.full((E + 1,), -1, dtype=torch.int64)
    ptr = 0
    for e in range(E):
        while ptr < R and sorted_ids[ptr] < e:
            ptr += 1
        off[e] = ptr
    off[E] = R
    return Xp.view(*lead, k, Xf.shape[-1]), w.view(*lead, k), inv.view(*lead, k), off


# --------------------------------------------------------------------------
# a3 / a5  grouped expert GEMMs
# --------------------------------------------------------------------------
def _grouped_linear(X, expert_offset, W, B, acc, out_dtype):
    E, N, K = W.shape
    assert X.shape[-1] == K, "X.shape is {}, in_features is {}".format(tuple(X.shape), K)
    Xf = X.reshape(-1, K)
    Y = torch.zeros(Xf.shape[0], N, dtype=acc)
    off = [int(v) for v in expert_offset.tolist()]
    for e in range(E):
        lo, hi = off[e], off[e + 1]
        if hi - lo <= 0:
            continue
        y = _acc(Xf[lo:hi], acc) @ _acc(W[e], acc).t()
        if B is not None:
            y = y + _acc(B[e], acc)
        Y[lo:hi] = y
    return Y.to(out_dtype or W.dtype).view(*X.shape[:-1], N)


def moe_column_parallel_linear(X, expert_offset, W, B=None, acc=torch.float32, out_dtype=None):
    """``MoeColumnParallelLinear.py:58-69``: per expert e,
    ``Y[off[e]:off[e+1]] = X[off[e]:off[e+1]] @ W[e]^T + B[e]``; rows outside
    every segment stay 0."""
    return _grouped_linear(X, expert_offset, W, B, acc, out_dtype)


def moe_row_parallel_linear(X, expert_offset, W, B=None, acc=torch.float32, out_dtype=None):
    """``MoeRowParallelLinear.py:44-60`` at world size 1 (bias per expert)."""
    return _grouped_linear(X, expert_offset, W, B, acc, out_dtype)


# --------------------------------------------------------------------------
# a4  activations
# --------------------------------------------------------------------------
def swiglu(X: torch.Tensor, beta: float = 1.0, acc=torch.float32, out_dtype=None):
    """``SwiGLU.py:15-16``: first half x, second half g; ``g * x * sigmoid(beta*x)``."""
    D = X.shape[-1] // 2
    x = _acc(X[..., :D], acc)
    g = _acc(X[..., D:], acc)
    return (g * x * torch.sigmoid(beta * x)).to(out_dtype or X.dtype)


def silu(X: torch.Tensor, gate: Optional[torch.Tensor] = None, acc=torch.float32, out_dtype=None):
    """``SiLU.py:18-21``: ``gate * silu(X)`` (``silu(X)`` when gate is None)."""
    x = _acc(X, acc)
    y = x * torch.sigmoid(x)
    if gate is not None:
        y = _acc(gate, acc) * y
    return y.to(out_dtype or X.dtype)


# --------------------------------------------------------------------------
# a6  MoeReduce                                          MoeReduce.py:23-25
# --------------------------------------------------------------------------

def skip_rms_norm(X, weight, SkipIn=None, eps=1e-5):
    """SkipRMSNorm over the last axis with the reference's roundings
    (torch_function/RMSNorm.py:44-56; RMSNorm.forward :16-24 is the SkipIn=None case):
    s = X + SkipIn in X's dtype; y = float(s) * rsqrt(mean(float(s)^2) + eps);
    Y = y.type_as(X) * weight (a product in X's dtype); SkipOut = s.  Returns (Y, s)."""
    s = X if SkipIn is None else X + SkipIn
    x = s.float()
    y = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
    return y.to(X.dtype) * weight, s


def rms_norm(X, weight, eps=1e-5):
    """RMSNorm (torch_function/RMSNorm.py:16-24)."""
    return skip_rms_norm(X, weight, None, eps)[0]


def moe_reduce(Y: torch.Tensor, expert_weights: torch.Tensor, invert_permutation: torch.Tensor,
               num_experts_per_token: int, acc=torch.float32, out_dtype=None):
    """``out[t] = sum_s w[t,s] * Y_flat[inv[t,s]]`` summed in slot order."""
    N = Y.shape[-1]
    Yf = _acc(Y.reshape(-1, N), acc)
    g = Yf[invert_permutation.reshape(-1)].view(*expert_weights.shape, N)
    out = (g * _acc(expert_weights, acc).unsqueeze(-1)).sum(dim=-2)
    return out.to(out_dtype or Y.dtype)


# --------------------------------------------------------------------------
# whole layer                                         Model.py:187-214
# --------------------------------------------------------------------------
def moe_layer(x, Wg, wu, w2, num_experts, num_experts_per_token, *, router_bias=None,
              bu=None, b2=None, round_between_ops: bool = True, acc=torch.float32,
              scores=None, return_all: bool = False, as_written: bool = False):
    """The six-step layer of ``MoeFeedForward.forward`` (fused gate/up form).

    ``round_between_ops=True`` rounds every operator output to the input dtype,
    exactly like running the reference operators one after the other on
    low-precision tensors with fp32 accumulation.  ``False`` keeps every
    intermediate in ``acc`` and rounds only the final output ("fp32 end to
    end from the same low-precision inputs").  ``scores`` overrides the router
    logits (to feed two implementations the same bits).  ``router_bias`` is
    the per-expert logit bias of the skewed-routing benchmark config.
    """
    dt = x.dtype
    mid = dt if round_between_ops else acc
    if scores is None:
        scores = linear(x, Wg, router_bias, acc=acc, out_dtype=dt)          # 188
    if as_written:
        xe, w, inv, off = moe_select_as_written(x, scores, num_experts, num_experts_per_token, acc=acc)
        idx = None
    else:
        xe, w, inv, off, idx = moe_select(x, scores, num_experts, num_experts_per_token,
                                          acc=acc, return_indices=True)     # 191
    x13 = moe_column_parallel_linear(xe, off, wu, bu, acc=acc, out_dtype=mid)   # 198
    a = swiglu(x13, acc=acc, out_dtype=mid)                                 # 200
    y = moe_row_parallel_linear(a, off, w2, b2, acc=acc, out_dtype=mid)     # 208
    out = moe_reduce(y, w, inv, num_experts_per_token, acc=acc, out_dtype=dt)   # 211
    if return_all:
        return dict(scores=scores, x_expand=xe, weights=w, inv=inv, off=off, idx=idx,
                    x13=x13, act=a, y=y, out=out)
    return out


def moe_layer_dense_fp64(x, Wg, wu, w2, num_experts, num_experts_per_token, *, scores=None,
                         router_bias=None):
    """Permutation-free textbook MoE in float64:
    ``out[t] = sum_s softmax(top-k scores)[s] * w2[e] @ swiglu(wu[e] @ x[t])``
    with ``e = idx[t, s]``.  Shares only :func:`topk_lower_id` with the
    operator-by-operator path: no sort, no inverse permutation, no offsets."""
    f8 = torch.float64
    k = num_experts_per_token
    if scores is None:
        scores = linear(x, Wg, router_bias, acc=torch.float32, out_dtype=x.dtype)
    vals, idx = topk_lower_id(scores.reshape(-1, num_experts), k)
    gate = torch.softmax(vals.to(torch.float32), -1).to(scores.dtype).to(f8)
    xf = x.reshape(-1, x.shape[-1]).to(f8)
    I = w2.shape[-1]
    out = torch.zeros(xf.shape[0], w2.shape[1], dtype=f8)
    for e in range(num_experts):
        hit = (idx == e)
        tok = hit.any(-1).nonzero().flatten()
        if tok.numel() == 0:
            continue
        h = xf[tok] @ wu[e].to(f8).t()
        a = h[:, I:] * h[:, :I] * torch.sigmoid(h[:, :I])
        y = a @ w2[e].to(f8).t()
        g = (gate[tok] * hit[tok].to(f8)).sum(-1, keepdim=True)
        out[tok] += g * y
    return out.view(*x.shape[:-1], -1)


# --------------------------------------------------------------------------
# synthetic inputs shared by tests, smoke check and benchmark
# --------------------------------------------------------------------------
def make_inputs(T, H, E, I, dtype=torch.float16, seed=0, with_w=True):
    """Seeded inputs in the fixed order x, Wg, wu, w2 (fp32 draws, then cast):
    x~N(0,1), router W~N(0,0.02), expert weights~N(0,0.02)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g).to(dtype)
    Wg = (torch.randn(E, H, generator=g) * 0.02).to(dtype)
    if not with_w:
        return x, Wg
    wu = torch.empty(E, 2 * I, H, dtype=dtype)
    w2 = torch.empty(E, H, I, dtype=dtype)
    for e in range(E):                      # per expert: bounded fp32 temporaries
        wu[e] = (torch.randn(2 * I, H, generator=g) * 0.02).to(dtype)
    for e in range(E):
        w2[e] = (torch.randn(H, I, generator=g) * 0.02).to(dtype)
    return x, Wg, wu, w2


def zipf_router_bias(E: int, alpha: float, s: float = 1.2) -> torch.Tensor:
    """Per-expert logit bias ``alpha * log p_e`` with ``p_e ~ (e+1)^-s``."""
    p = torch.arange(1, E + 1, dtype=torch.float64) ** (-s)
    p = p / p.sum()
    return (alpha * torch.log(p)).to(torch.float32)
