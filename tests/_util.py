"""Helpers shared by the GPU parity tests."""
import torch

ULP = {torch.float32: 2.0 ** -23, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}


def dev():
    return torch.device("cuda:0")


def gpu_inputs(T, H, E, I, dtype, seed=0):
    """Seeded x, Wg, wu, w2, returned as (device tensors, host copies): both paths under test see
    identical bits.  x and the router weight are the CPU draws of the oracle's `make_inputs`
    (x first), so the routing is that of the seeded tensor set; the expert weights, which would
    take minutes to draw on the host at the large configurations, are drawn on the GPU."""
    from oracle import moe_oracle as O
    d = dev()
    xc, Wgc = O.make_inputs(T, H, E, I, dtype=dtype, seed=seed, with_w=False)
    x, Wg = xc.to(d), Wgc.to(d)
    g = torch.Generator(device="cuda").manual_seed(seed)
    wu = torch.empty(E, 2 * I, H, dtype=dtype, device=d)
    w2 = torch.empty(E, H, I, dtype=dtype, device=d)
    for e in range(E):
        wu[e] = (torch.randn(2 * I, H, generator=g, device=d) * 0.02).to(dtype)
        w2[e] = (torch.randn(H, I, generator=g, device=d) * 0.02).to(dtype)
    dev_t = (x, Wg, wu, w2)
    return dev_t, (xc, Wgc, wu.cpu(), w2.cpu())


def assert_close_ulp(got, ref, dtype, ulps=2.0, what="", floor=1e-2):
    """|got-ref| <= ulps * ulp(dtype) * max(|ref|, floor): one rounding plus the
    reordering of an fp32 accumulation; `floor` (fraction of max|ref|) bounds the
    relative test away from zero, where sums cancel."""
    got, ref = got.double().cpu(), ref.double().cpu()
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    tol = ulps * ULP[dtype] * torch.clamp(ref.abs(), min=float(ref.abs().max()) * floor + 1e-30)
    bad = (got - ref).abs() > tol
    assert not bool(bad.any()), "{}: {} of {} elements off, worst {:.3e} (ref scale {:.3e})".format(
        what, int(bad.sum()), bad.numel(), float((got - ref).abs().max()), float(ref.abs().max()))


def tie_heavy_scores(T, E, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randint(-3, 4, (T, E), generator=g).float() * 0.25).to(dtype)
