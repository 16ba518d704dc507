"""Operator calls whose exported ONNX nodes are compared between the reference's
``torch_function`` package and this build's.  ``cases(OPMX)`` returns (name, module, inputs)
triples for whichever package is passed in; ``export_nodes`` runs the TorchScript exporter on a
module and lists its ``opmx::`` nodes as (kind, number of inputs, number of outputs, attributes).
Used by ``make_symbolic_fixture.py`` (reference side, build container only) and by
``tests/test_host_wrappers.py`` (this build's side, against the committed fixture)."""
import contextlib
import io
import warnings

import torch


def export_nodes(mod, args):
    from torch.onnx._internal.torchscript_exporter import utils as U
    from torch.onnx._internal.torchscript_exporter._globals import GLOBALS
    GLOBALS.export_onnx_opset_version = 11
    with warnings.catch_warnings(), contextlib.redirect_stdout(io.StringIO()):
        warnings.simplefilter("ignore")
        with U.exporter_context(mod, torch.onnx.TrainingMode.EVAL, False):
            GLOBALS.in_onnx_export = True
            try:
                graph, _, _ = U._model_to_graph(mod, args)
            finally:
                GLOBALS.in_onnx_export = False
    found = []
    for n in graph.nodes():
        if n.kind().startswith("opmx::"):
            attrs = {a: (n.f(a) if n.kindOf(a) == "f" else n.i(a)) for a in sorted(n.attributeNames())}
            found.append([n.kind(), len(list(n.inputs())), len(list(n.outputs())), attrs])
    return found


class _Call(torch.nn.Module):
    def __init__(self, fn):
        super().__init__()
        self.fn = fn

    def forward(self, *a):
        return self.fn(*a)


def cases(OPMX):
    T, H, E, k, I = 6, 32, 8, 2, 48
    x, s = torch.randn(T, H), torch.randn(T, E)
    xe, off = torch.randn(T, k, H), torch.zeros(E + 1, dtype=torch.int64)
    wu, bu = torch.randn(E, 2 * I, H), torch.randn(E, 2 * I)
    w2, b2 = torch.randn(E, H, I), torch.randn(E, H)
    a, y = torch.randn(T, k, I), torch.randn(T, k, H)
    w, inv = torch.rand(T, k), torch.zeros(T, k, dtype=torch.int64)
    wg, bg = torch.randn(E, H), torch.randn(E)
    norm_w = torch.ones(H)
    out = [
        ("linear", _Call(lambda X, W: OPMX.linear(X, W, None, H, E)), (x, wg)),
        ("linear_bias", _Call(lambda X, W, B: OPMX.linear(X, W, B, H, E)), (x, wg, bg)),
        ("moe_select", _Call(lambda X, S: OPMX.moe_select(X, S, E, k)), (x, s)),
        ("moe_column_parallel_linear",
         _Call(lambda X, O_, W: OPMX.moe_column_parallel_linear(X, O_, W, None, None, E, H, 2 * I, False)), (xe, off, wu)),
        ("moe_column_parallel_linear_bias_gather",
         _Call(lambda X, O_, W, B: OPMX.moe_column_parallel_linear(X, O_, W, B, None, E, H, 2 * I, True)), (xe, off, wu, bu)),
        ("moe_row_parallel_linear",
         _Call(lambda X, O_, W: OPMX.moe_row_parallel_linear(X, O_, W, None, None, E, I, H, True)), (a, off, w2)),
        ("moe_row_parallel_linear_bias",
         _Call(lambda X, O_, W, B: OPMX.moe_row_parallel_linear(X, O_, W, B, None, E, I, H, False)), (a, off, w2, b2)),
        ("moe_reduce", _Call(lambda Y, W, P: OPMX.moe_reduce(Y, W, P, k)), (y, w, inv)),
        ("swiglu", _Call(lambda X: OPMX.swiglu(X)), (torch.randn(T, k, 2 * I),)),
        ("swiglu_beta", _Call(lambda X: OPMX.swiglu(X, 1.5)), (torch.randn(T, k, 2 * I),)),
        ("silu", _Call(lambda X: OPMX.silu(X)), (a,)),
        ("silu_gate", _Call(lambda X, G: OPMX.silu(X, G)), (a, a.clone())),
        ("rms_norm", _Call(lambda X, W: OPMX.rms_norm(X, W, -1, 1e-6)), (x, norm_w)),
        ("skip_rms_norm", _Call(lambda X, W, S: OPMX.skip_rms_norm(X, W, S, -1, 1e-5)), (x, norm_w, x.clone())),
    ]
    return out
