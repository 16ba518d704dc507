"""GPU parity of a block loaded from an OPMX checkpoint file.

The file has the keys and stacked expert layout that
model_zoo/mixtral/huggingface/ConvertWeightToOpmx.py:98-128 writes (separate ``w1`` / ``w3``);
``load_opmx_moe_block`` fills the device layout of Model.py:399-413 (``wu = [w1; w3]``) from it.
The loaded block runs on the GPU and is checked against the oracle layer built from the same
state dict: routing bit-exact, output within max-abs 2e-2 / mean-abs 2e-3."""
import pytest
import torch

from _util import dev
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu
MAX_ABS, MEAN_ABS = 2e-2, 2e-3


def opmx_checkpoint(E, H, I, layers, bias, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *shape, scale=0.03: (torch.randn(*shape, generator=g) * scale).to(dtype)
    sd = {"tok_embeddings.weight": r(32, H)}
    for n in range(layers):
        p = "layers.{}.feed_forward.".format(n)
        sd[p + "gate.weight"] = r(E, H)
        sd[p + "w1.weight"] = r(E, I, H)
        sd[p + "w2.weight"] = r(E, H, I)
        sd[p + "w3.weight"] = r(E, I, H)
        if bias:
            sd[p + "w1.bias"] = r(E, I, scale=0.2)
            sd[p + "w3.bias"] = r(E, I, scale=0.2)
            sd[p + "w2.bias"] = r(E, H, scale=0.2)
        sd["layers.{}.ffn_norm.weight".format(n)] = torch.ones(H, dtype=dtype)
    return sd


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("fused_ffn_glu,fuse_epilogue", [(True, False), (True, True), (False, False)])
@pytest.mark.parametrize("T,E,k,H,I,dtype", [
    (48, 8, 2, 512, 1024, torch.float16),       # few rows per expert: weight-streaming kernels
    (1536, 8, 2, 256, 640, torch.bfloat16),     # hundreds of rows per expert: MFMA tile kernels
])
def test_checkpoint_loaded_block_matches_oracle(tmp_path, T, E, k, H, I, dtype, fused_ffn_glu, fuse_epilogue, bias):
    from model_zoo.mixtral.modeling.dynamic_batching.Model import load_opmx_moe_block
    import torch_function as OPMX
    layer_id = 1
    sd = opmx_checkpoint(E, H, I, layers=2, bias=bias, dtype=dtype, seed=T + I)
    path = tmp_path / "model.pth"
    torch.save(sd, path)

    block = load_opmx_moe_block(str(path), layer_id, k, fused_ffn_glu=fused_ffn_glu, device=dev(),
                                fuse_swiglu_epilogue=fuse_epilogue)
    p = "layers.{}.feed_forward.".format(layer_id)
    assert block.num_experts == E and block.gate.weight.is_cuda and block.w2.weight.dtype == dtype
    # the device layout: w1 and w3 are the two halves of wu (Model.py:399-413)
    if fused_ffn_glu:
        assert torch.equal(block.wu.weight[:, :I].cpu(), sd[p + "w1.weight"])
        assert torch.equal(block.wu.weight[:, I:].cpu(), sd[p + "w3.weight"])

    x = torch.randn(T, H, generator=torch.Generator().manual_seed(5)).to(dtype)
    xd = x.to(dev())
    out = block(xd)
    scores = OPMX.linear(xd, block.gate.weight, None, H, E)
    _, w, inv, off = OPMX.moe_select(xd, scores, E, k)
    torch.cuda.synchronize()

    # the oracle layer from the same state dict, routed by the same low-precision logits
    wu = torch.cat([sd[p + "w1.weight"], sd[p + "w3.weight"]], dim=1)
    bu = torch.cat([sd[p + "w1.bias"], sd[p + "w3.bias"]], dim=1) if bias else None
    b2 = sd[p + "w2.bias"] if bias else None
    ref = O.moe_layer(x, sd[p + "gate.weight"], wu, sd[p + "w2.weight"], E, k, bu=bu, b2=b2, scores=scores.cpu(),
                      round_between_ops=False, return_all=True)
    assert torch.equal(inv.cpu(), ref["inv"]) and torch.equal(off.cpu(), ref["off"]), "routing differs from the oracle"
    err = (out.cpu().double() - ref["out"].double()).abs()
    assert float(err.max()) <= MAX_ABS and float(err.mean()) <= MEAN_ABS, (float(err.max()), float(err.mean()))
