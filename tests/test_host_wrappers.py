"""CPU checks of the host-side mirror of the reference interface: names and
signatures, ONNX symbolics (node type, input order, attribute names and values
as in the reference's symbolic() functions), export placeholders, and the "no
CPU fallback" rule."""
import contextlib
import inspect
import io
import re
import warnings

import pytest
import torch

import torch_function as OPMX
from model_zoo.mixtral.modeling.dynamic_batching.Model import MoeFeedForward


def test_public_names_and_signatures():
    # torch_function/__init__.py:15,17-20,37-38 and the wrapper defs of each file
    sig = lambda f: list(inspect.signature(f).parameters)
    assert sig(OPMX.moe_select) == ["X", "scores", "num_experts", "num_experts_per_token"]
    assert sig(OPMX.moe_reduce) == ["Y", "expert_weights", "invert_permutation", "num_experts_per_token"]
    assert sig(OPMX.moe_column_parallel_linear) == ["X", "expert_offset", "W", "B", "proc_group", "num_experts",
                                                    "in_features", "out_features", "gather_output"]
    assert sig(OPMX.moe_row_parallel_linear) == ["X", "expert_offset", "W", "B", "proc_group", "num_experts",
                                                 "in_features", "out_features", "input_is_parallel"]
    assert sig(OPMX.swiglu) == ["X", "beta"] and sig(OPMX.silu) == ["X", "gate"]
    assert sig(OPMX.linear) == ["X", "W", "B", "in_features", "out_features"]
    assert sig(OPMX.rms_norm) == ["X", "weight", "axis", "eps"]                       # RMSNorm.py:59-61
    assert sig(OPMX.skip_rms_norm) == ["X", "weight", "SkipIn", "axis", "eps"]        # RMSNorm.py:64-66
    assert inspect.signature(OPMX.skip_rms_norm).parameters["eps"].default == 1e-5
    p = inspect.signature(OPMX.moe_column_parallel_linear).parameters
    assert p["gather_output"].default is True
    assert inspect.signature(OPMX.moe_row_parallel_linear).parameters["input_is_parallel"].default is False


def test_no_cpu_fallback():
    x = torch.randn(4, 16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        OPMX.moe_select(x, torch.randn(4, 8), 8, 2)
    with pytest.raises(RuntimeError, match="no CPU path"):
        OPMX.swiglu(x)
    with pytest.raises(RuntimeError, match="no CPU path"):
        OPMX.moe_reduce(torch.randn(4, 2, 8), torch.rand(4, 2), torch.arange(8).view(4, 2), 2)
    with pytest.raises(RuntimeError, match="no CPU path"):
        OPMX.linear(x, torch.randn(8, 16), None, 16, 8)
    with pytest.raises(RuntimeError, match="no CPU path"):
        OPMX.skip_rms_norm(x, torch.ones(16), x)
    with pytest.raises(AssertionError):          # the reference's in_features assert comes first
        OPMX.moe_column_parallel_linear(x, torch.arange(3), torch.randn(2, 8, 16), None, None, 2, 15, 8, False)


def export_graph(mod, args):
    """TorchScript-exporter graph of `mod` at opset 11 (what torch.onnx.export
    builds before serialising; the `onnx` package is not needed for this)."""
    from torch.onnx._internal.torchscript_exporter import utils as U
    from torch.onnx._internal.torchscript_exporter._globals import GLOBALS
    GLOBALS.export_onnx_opset_version = 11
    with warnings.catch_warnings(), contextlib.redirect_stdout(io.StringIO()):
        warnings.simplefilter("ignore")
        with U.exporter_context(mod, torch.onnx.TrainingMode.EVAL, False):
            GLOBALS.in_onnx_export = True
            try:
                graph, _, out = U._model_to_graph(mod, args)
            finally:
                GLOBALS.in_onnx_export = False
    return graph, out


def nodes_of(graph):
    found = []
    for n in graph.nodes():
        if n.kind().startswith("opmx::"):
            attrs = {a: (n.f(a) if n.kindOf(a) == "f" else n.i(a)) for a in n.attributeNames()}
            found.append((n.kind(), len(list(n.inputs())), len(list(n.outputs())), attrs))
    return found


def test_symbolics_match_the_reference_fixture():
    """Node kind, input / output counts and attribute names and values of every operator against
    tests/golden/reference_symbolics.json, which tests/golden/make_symbolic_fixture.py wrote by
    exporting the same calls through the reference's own torch_function package (MoeSelect.py:5-17,
    MoeColumnParallelLinear.py:8-27, MoeRowParallelLinear.py:8-26, MoeReduce.py:5-12, SwiGLU.py:5-8,
    SiLU.py, Linear.py:7-22, RMSNorm.py:6-11,29-39)."""
    import json
    import os
    import sys
    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    sys.path.insert(0, golden)
    try:
        from symbolic_cases import cases, export_nodes
    finally:
        sys.path.remove(golden)
    want = json.load(open(os.path.join(golden, "reference_symbolics.json")))["nodes"]
    mine = cases(OPMX)
    assert sorted(want) == sorted(name for name, _, _ in mine)
    for name, mod, args in mine:
        got = export_nodes(mod, args)
        assert len(got) == len(want[name]) >= 1, name
        for g, w in zip(got, want[name]):
            assert g[:3] == w[:3], (name, g, w)
            assert sorted(g[3]) == sorted(w[3]), (name, g[3], w[3])
            for key, val in w[3].items():
                assert abs(g[3][key] - val) <= 1e-9 * max(1.0, abs(val)), (name, key, g[3][key], val)


@pytest.mark.parametrize("fused,bias", [(True, False), (False, True)])
def test_mixtral_block_exports_reference_nodes(fused, bias):
    H, I, E, k = 64, 96, 8, 2
    m = MoeFeedForward(MoeFeedForward.params(H, I, E, k), 0, fused, bias, None, fuse_swiglu_epilogue=True)
    graph, out = export_graph(m, (torch.randn(5, H),))
    got = nodes_of(graph)
    nb = 1 if bias else 0
    col = lambda n: ("opmx::MoeColumnParallelLinear", 3 + nb, 1,
                     dict(num_experts=E, in_features=H, out_features=n, bias_term=nb, gather_output=0))
    want = [("opmx::Linear", 2, 1, dict(in_features=H, out_features=E, bias_term=0)),
            ("opmx::MoeSelect", 2, 4, dict(num_experts=E, num_experts_per_token=k))]
    if fused:
        want += [col(2 * I), ("opmx::SwiGLU", 1, 1, dict(beta=1.0))]
    else:
        want += [col(I), col(I), ("opmx::SiLU", 2, 1, {})]
    want += [("opmx::MoeRowParallelLinear", 3 + nb, 1,
              dict(num_experts=E, in_features=I, out_features=H, bias_term=nb, input_is_parallel=1)),
             ("opmx::MoeReduce", 3, 1, dict(num_experts_per_token=k))]
    assert got == want
    assert tuple(out.shape) == (5, H)


def test_rms_norm_exports_reference_nodes():
    """opmx::RMSNorm with axis / eps / skip_term and one or two outputs (RMSNorm.py:6-11, 29-39)."""
    from model_zoo.ModelLayers import RMSNorm, SkipRMSNorm

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a, self.b = RMSNorm(16, 1e-6), SkipRMSNorm(16, 1e-6)

        def forward(self, x, skip):
            y, so = self.b(x, skip)
            return self.a(y), so
    graph, out = export_graph(Block(), (torch.randn(3, 16), torch.randn(3, 16)))
    got = nodes_of(graph)
    assert [(k, i, o) for k, i, o, _ in got] == [("opmx::RMSNorm", 3, 2), ("opmx::RMSNorm", 2, 1)]
    assert got[0][3]["axis"] == -1 and got[0][3]["skip_term"] == 1 and abs(got[0][3]["eps"] - 1e-6) < 1e-12
    assert got[1][3]["skip_term"] == 0
    assert tuple(out[0].shape) == (3, 16) and tuple(out[1].shape) == (3, 16)


def test_export_placeholders_have_eager_order_and_types():
    class Sel(torch.nn.Module):
        def forward(self, x, s):
            return OPMX.moe_select(x, s, 8, 2)
    graph, out = export_graph(Sel(), (torch.randn(3, 4, 16).half(), torch.randn(3, 4, 8).half()))
    xe, w, inv, off = out
    assert xe.shape == (3, 4, 2, 16) and xe.dtype == torch.float16
    assert w.shape == (3, 4, 2) and w.dtype == torch.float16
    assert inv.shape == (3, 4, 2) and inv.dtype == torch.int64
    assert off.shape == (9,) and off.dtype == torch.int64
    text = str(graph)
    assert re.search(r"Half\(.*\), %\d+ : Half\(.*\), %\d+ : Long\(.*\), %\d+ : Long\(.*\) = opmx::MoeSelect", text)


def test_tensor_parallel_is_refused():
    class FakeGroup:
        def size(self):
            return 2
    import unittest.mock as mock
    with mock.patch("torch.distributed.get_world_size", return_value=2):
        with pytest.raises(NotImplementedError):
            OPMX.moe_row_parallel_linear(torch.randn(4, 16), torch.arange(3), torch.randn(2, 8, 16), None,
                                         FakeGroup(), 2, 16, 8, True)
        with pytest.raises(NotImplementedError):
            OPMX.moe_column_parallel_linear(torch.randn(4, 16), torch.arange(3), torch.randn(2, 8, 16), None,
                                            FakeGroup(), 2, 16, 8, False)


def _fake_checkpoint(E=4, H=16, I=24, layers=2, bias=False, seed=0):
    g = torch.Generator().manual_seed(seed)
    sd = {}
    for n in range(layers):
        p = "layers.{}.feed_forward.".format(n)
        sd[p + "gate.weight"] = torch.randn(E, H, generator=g)
        sd[p + "w1.weight"] = torch.randn(E, I, H, generator=g)
        sd[p + "w3.weight"] = torch.randn(E, I, H, generator=g)
        sd[p + "w2.weight"] = torch.randn(E, H, I, generator=g)
        if bias:
            sd[p + "w1.bias"] = torch.randn(E, I, generator=g)
            sd[p + "w3.bias"] = torch.randn(E, I, generator=g)
            sd[p + "w2.bias"] = torch.randn(E, H, generator=g)
        sd["layers.{}.ffn_norm.weight".format(n)] = torch.ones(H)
        sd["layers.{}.attention.wo.weight".format(n)] = torch.randn(H, H, generator=g)
    return sd


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("bias", [False, True])
def test_moe_block_loads_an_opmx_checkpoint(tmp_path, fused, bias):
    """Checkpoint keys and stacked expert layout of ConvertWeightToOpmx.py:98-128; w1 / w3 land in the
    halves of wu as in Model.py:399-413."""
    from model_zoo.mixtral.modeling.dynamic_batching.Model import load_opmx_moe_block
    E, H, I = 4, 16, 24
    sd = _fake_checkpoint(E, H, I, bias=bias)
    m = MoeFeedForward(MoeFeedForward.params(H, I, E, 2), 1, fused, bias, None)
    used = m.load_state_dict(sd)
    p = "layers.1.feed_forward."
    assert sorted(used) == sorted(k for k in sd if k.startswith(p))
    assert torch.equal(m.gate.weight, sd[p + "gate.weight"]) and torch.equal(m.w2.weight, sd[p + "w2.weight"])
    if fused:
        assert torch.equal(m.wu.weight[:, :I], sd[p + "w1.weight"]) and torch.equal(m.wu.weight[:, I:], sd[p + "w3.weight"])
        if bias:
            assert torch.equal(m.wu.bias[:, :I], sd[p + "w1.bias"]) and torch.equal(m.wu.bias[:, I:], sd[p + "w3.bias"])
    else:
        assert torch.equal(m.w1.weight, sd[p + "w1.weight"]) and torch.equal(m.w3.weight, sd[p + "w3.weight"])
    # strictness: a missing tensor and a wrong shape are refused
    broken = {k: v for k, v in sd.items() if not k.endswith("1.feed_forward.w3.weight")}
    with pytest.raises(KeyError):
        MoeFeedForward(MoeFeedForward.params(H, I, E, 2), 1, fused, bias, None).load_state_dict(broken)
    wrong = dict(sd)
    wrong[p + "w2.weight"] = torch.zeros(E, H, I + 1)
    with pytest.raises(ValueError):
        MoeFeedForward(MoeFeedForward.params(H, I, E, 2), 1, fused, bias, None).load_state_dict(wrong)
    # from a file: sizes come from the tensors, dtype can be converted on the way in
    path = tmp_path / "model.pth"
    torch.save(sd, path)
    b = load_opmx_moe_block(str(path), 0, 2, fused_ffn_glu=fused, dtype=torch.float16)
    assert b.num_experts == E and b.w2.weight.dtype == torch.float16 and (b.w2.bias is not None) == bias
    assert torch.equal(b.w2.weight, sd["layers.0.feed_forward.w2.weight"].half())
