"""The library enqueues kernels only (no allocation, no synchronisation, no memset), so a quantised layer can be
captured into a HIP graph and replayed: decode-size calls are launch-bound otherwise.  Every replay is checked
against the eager result, with eager work and synchronisations between the replays."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.mark.parametrize("M,K,N", [(8, 512, 12288), (200, 512, 12288), (1024, 512, 12288),
                                   (200, 4096, 512),    # K split over workgroups, workspace from torch's allocator
                                   (16, 4096, 1024), (40, 4096, 1024),   # the weight-streaming kernel: one and three operand tiles of x
                                   (48, 8192, 520)])    # ... on K slices: workspace and the reduce kernel inside the capture
def test_fused_layer_replays_from_a_graph(M, K, N):
    from mase_hip import _lib
    from mase_hip.mxfp.layers import MXFPLinearPTQ
    from mase_hip.mxfp.meta import MXFP8_E4M3_fn, OCP_MXFP6_E3M2

    _lib.load()
    lin = torch.nn.Linear(K, N, bias=True, dtype=torch.bfloat16, device=DEV)
    layer = MXFPLinearPTQ.from_linear(lin, MXFP8_E4M3_fn, OCP_MXFP6_E3M2, None, "XqWqB", "fused")
    g = torch.Generator(device=DEV).manual_seed(M)
    static_x = torch.randn(M, K, generator=g, device=DEV).to(torch.bfloat16)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up outside the capture: first-call set-up of the kernels happens here
        for _ in range(3):
            layer(static_x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = layer(static_x)
    for i in range(4):
        x = torch.randn(M, K, generator=g, device=DEV).to(torch.bfloat16) * (i + 1)
        want = layer(x)                     # eager work between the replays
        torch.cuda.synchronize()
        static_x.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y.view(torch.int16), want.view(torch.int16)), f"replay {i}"
