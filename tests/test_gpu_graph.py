"""The MoE layer under HIP graph capture: a captured layer, replayed, gives the eager result.

Small-batch decode is bound by the host's launch path (six operators, a few microseconds of GPU
work each), so a serving loop captures the layer once and replays it.  That only works if no
operator allocates, synchronises or reads device data on the host, and if nothing the library
records into the graph misbehaves on replay: every replay is checked bit for bit against an eager
run on the same input, with eager work and synchronisation between the replays.  Cases cover the
weight-streaming kernels, the tiled kernels with the split-K exchange (its counters are cleared by
the main GEMM launch, inside the graph), the persistent tiled kernel, and both select paths."""
import pytest
import torch

from _util import dev, gpu_inputs
from test_gpu_layer import build_layer

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("T,H,I,E,k,dtype,fuse,route,gather", [
    (1, 1024, 2816, 8, 2, torch.float16, False, False, False),    # single token: 16-row stream kernel, small select
    (32, 1024, 2816, 8, 2, torch.float16, True, False, False),    # stream kernel with the SwiGLU epilogue
    (8, 1024, 2816, 8, 2, torch.float16, True, True, False),      # ... and router gate + select in one launch
    (8, 1024, 2816, 8, 2, torch.float16, True, True, True),       # ... and the rows read through the index
    (40, 512, 1408, 64, 8, torch.bfloat16, False, False, False),  # 64 experts, short K
    (256, 1024, 3584, 8, 2, torch.float16, False, False, False),  # 128 x 256 tiles, down projection split over K
    (3000, 512, 1024, 8, 2, torch.float16, False, True, False),   # large select path, persistent 256 x 256 tiles
    (5000, 512, 1024, 8, 2, torch.float16, True, True, True),     # every fused form: routing in the router kernel's
                                                                  # epilogue, rows through the index, persistent tiles
    (700, 512, 1408, 64, 8, torch.bfloat16, True, True, True),    # the same with 64 experts
])
def test_captured_layer_replays_the_eager_result(T, H, I, E, k, dtype, fuse, route, gather):
    (x, Wg, wu, w2), _ = gpu_inputs(T, H, E, I, dtype, seed=3)
    layer = build_layer(H, I, E, k, dtype, Wg, wu, w2, fuse=fuse, route=route, gather=gather)
    gen = torch.Generator(device="cuda").manual_seed(11)
    inputs = [x] + [torch.randn(T, H, generator=gen, device=dev()).to(dtype) for _ in range(3)]
    with torch.inference_mode():
        eager = [layer(xi).clone() for xi in inputs]
        static_x = inputs[0].clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):                   # warm-up off the capture: one-time kernel attributes
            layer(static_x)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_out = layer(static_x)
        for rep in range(2):
            for xi, want in zip(inputs, eager):
                static_x.copy_(xi)
                graph.replay()
                got = static_out.clone()
                # eager work of the same kind and a synchronisation between replays
                other = layer(inputs[(rep + 1) % len(inputs)])
                torch.cuda.synchronize()
                assert torch.equal(got, want), (rep, float((got.float() - want.float()).abs().max()))
                assert other.shape == want.shape


def test_graphed_block_matches_the_eager_block():
    """GraphedMoeFeedForward: one graph per input shape, results equal to the eager block bit for
    bit, shapes interleaved, the oldest graph dropped when the bound is reached."""
    from model_zoo.mixtral.modeling.dynamic_batching.Model import GraphedMoeFeedForward
    H, I, E, k, dtype = 512, 1408, 8, 2, torch.float16
    (x, Wg, wu, w2), _ = gpu_inputs(64, H, E, I, dtype, seed=5)
    block = build_layer(H, I, E, k, dtype, Wg, wu, w2)
    graphed = GraphedMoeFeedForward(block, max_graphs=2)
    gen = torch.Generator(device="cuda").manual_seed(2)
    with torch.inference_mode():
        for T in (1, 32, 1, 64, 32, 1):               # three shapes through a bound of two
            xi = torch.randn(T, H, generator=gen, device=dev()).to(dtype)
            want = block(xi)
            got = graphed(xi).clone()
            torch.cuda.synchronize()
            assert torch.equal(got, want), T
            assert len(graphed._graphs) <= 2
