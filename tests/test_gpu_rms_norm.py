"""GPU parity: RMSNorm / SkipRMSNorm (the norm in front of the MoE layer) against the CPU
oracle on identical inputs, through the C ABI.  The skip output is a single rounded sum and must
be bit-exact; the normalised output may differ by the fp32 summation order of the mean square:
tolerance 2 ulp of the output dtype (fp32: 64 ulp)."""
import pytest
import torch

from _util import assert_close_ulp, dev
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def opmx():
    import torch_function as OPMX
    return OPMX


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(32, 4096), (3, 5, 2048), (7, 6144), (4, 1000), (9, 77), (2, 20000), (1, 8)])
def test_skip_rms_norm_matches_oracle(dtype, shape):
    OPMX = opmx()
    g = torch.Generator().manual_seed(sum(shape))
    X = (torch.randn(*shape, generator=g) * 2.0).to(dtype)
    S = torch.randn(*shape, generator=g).to(dtype)
    w = (torch.rand(shape[-1], generator=g) + 0.5).to(dtype)
    f32 = dtype == torch.float32
    for eps in (1e-5, 1e-6):
        Y, so = OPMX.skip_rms_norm(X.to(dev()), w.to(dev()), S.to(dev()), -1, eps)
        Yr, sor = O.skip_rms_norm(X, w, S, eps)
        assert Y.dtype == dtype and so.dtype == dtype and Y.shape == X.shape
        assert torch.equal(so.cpu(), sor)
        assert_close_ulp(Y, Yr.double(), dtype, ulps=64 if f32 else 2, floor=0.25 if f32 else 0.02,
                         what="skip_rms_norm {} {}".format(shape, dtype))
    Y1 = OPMX.rms_norm(X.to(dev()), w.to(dev()), -1, 1e-5)
    assert_close_ulp(Y1, O.rms_norm(X, w, 1e-5).double(), dtype, ulps=64 if f32 else 2, floor=0.25 if f32 else 0.02,
                     what="rms_norm {} {}".format(shape, dtype))
    # no skip input: the skip output is the input itself, as in the reference
    Xd = X.to(dev())
    Y2, so2 = OPMX.skip_rms_norm(Xd, w.to(dev()))
    assert so2.data_ptr() == Xd.data_ptr() and torch.equal(Y2, Y1)


def test_rms_norm_special_rows_and_errors():
    OPMX = opmx()
    w = torch.ones(64, dtype=torch.float16, device=dev())
    z = torch.zeros(3, 64, dtype=torch.float16, device=dev())
    assert torch.equal(OPMX.rms_norm(z, w, -1, 1e-5), z)                  # eps keeps a zero row finite
    c = torch.full((2, 64), -3.0, dtype=torch.float16, device=dev())
    assert torch.allclose(OPMX.rms_norm(c, w, -1, 0.0).float(), -torch.ones(2, 64, device=dev()), atol=1e-3)
    e = torch.empty(0, 64, dtype=torch.float16, device=dev())
    assert OPMX.rms_norm(e, w).shape == (0, 64)
    with pytest.raises(ValueError):
        OPMX.rms_norm(c, w, 0, 1e-5)                                      # only the last axis
    with pytest.raises(ValueError):
        OPMX.rms_norm(c, w[:32])
    with pytest.raises(TypeError):
        OPMX.skip_rms_norm(c, w, c.float())


def OPMX_scores(y, ffn):
    return opmx().linear(y, ffn.gate.weight, None, ffn.gate.in_features, ffn.gate.out_features)


def test_norm_feeds_the_moe_layer():
    """ffn_norm -> MoE layer as in the reference's TransformerBlock (Model.py:261-264)."""
    from model_zoo.ModelLayers import SkipRMSNorm
    from model_zoo.mixtral.modeling.dynamic_batching.Model import MoeFeedForward
    T, H, I, E, k = 48, 512, 1024, 8, 2
    dtype = torch.float16
    _, Wg, wu, w2 = O.make_inputs(T, H, E, I, dtype=dtype, seed=11)
    g = torch.Generator().manual_seed(12)
    attn, skip = torch.randn(T, H, generator=g).to(dtype), torch.randn(T, H, generator=g).to(dtype)
    wn = (torch.rand(H, generator=g) + 0.5).to(dtype)
    norm = SkipRMSNorm(H, 1e-6, dtype=dtype, device=dev())
    norm.weight.data = wn.to(dev())
    ffn = MoeFeedForward(MoeFeedForward.params(H, I, E, k), 0, True, False, None, dtype=dtype, device=dev())
    ffn.gate.weight.data = Wg.to(dev())
    ffn.wu.weight.data = wu.to(dev())
    ffn.w2.weight.data = w2.to(dev())
    y, h = norm(attn.to(dev()), skip.to(dev()))
    out = ffn(y)
    yr, hr = O.skip_rms_norm(attn, wn, skip, 1e-6)
    # the layer on the GPU's own norm output, router logits shared so both take the same routes
    scores = OPMX_scores(y, ffn)
    ref = O.moe_layer(y.cpu(), Wg, wu, w2, E, k, scores=scores.cpu(), round_between_ops=False)
    assert torch.equal(h.cpu(), hr)
    assert (y.cpu().float() - yr.float()).abs().max() <= 2e-2
    err = (out.cpu().float() - ref.float()).abs()
    assert err.max() <= 2e-2 and err.mean() <= 2e-3


def test_block_from_checkpoint_runs_on_the_gpu(tmp_path):
    """OPMX checkpoint file -> MoE block on the GPU (stacked expert weights, w1 / w3 into wu)."""
    from model_zoo.mixtral.modeling.dynamic_batching.Model import load_opmx_moe_block
    T, H, I, E, k = 40, 256, 384, 8, 2
    x, Wg, wu, w2 = O.make_inputs(T, H, E, I, dtype=torch.float16, seed=21)
    p = "layers.3.feed_forward."
    sd = {p + "gate.weight": Wg, p + "w1.weight": wu[:, :I].contiguous(), p + "w3.weight": wu[:, I:].contiguous(),
          p + "w2.weight": w2, "layers.3.ffn_norm.weight": torch.ones(H, dtype=torch.float16)}
    path = tmp_path / "model.pth"
    torch.save(sd, path)
    block = load_opmx_moe_block(str(path), 3, k, device=dev())
    assert block.wu.weight.device.type == "cuda" and torch.equal(block.wu.weight.cpu(), wu)
    out = block(x.to(dev()))
    scores = opmx().linear(x.to(dev()), block.gate.weight, None, H, E)
    ref = O.moe_layer(x, Wg, wu, w2, E, k, scores=scores.cpu(), round_between_ops=False)
    err = (out.cpu().float() - ref.float()).abs()
    assert err.max() <= 2e-2 and err.mean() <= 2e-3
