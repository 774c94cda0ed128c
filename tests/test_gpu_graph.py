"""The headline block recorded into a HIP graph: replays must equal eager runs, also with eager work
and synchronisations between the replays."""
import pytest
import torch

import fairseq_apollo_amd as M
from gpu_util import DEV

pytestmark = pytest.mark.gpu


def test_block_replays_from_a_graph():
    torch.manual_seed(51)
    B, L, D = 2, 1024, 256
    norm = M.TimestepNorm(D, num_groups=16).to(DEV).eval()
    ema = M.MultiHeadComplexEMA(D, ndim=16).to(DEV).eval()
    with torch.no_grad():
        norm.weight.normal_(0, 0.3)
        norm.bias.normal_(0, 0.3)

    def block(x):
        with torch.no_grad():
            return ema(norm(x).transpose(1, 2))

    static_x = torch.randn(B, L, D, device=DEV, dtype=torch.bfloat16)
    # warm-up on a side stream: workspaces, the cached kernel image and the library itself exist before capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            block(static_x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = block(static_x)
    for i in range(4):
        fresh = torch.randn(B, L, D, device=DEV, dtype=torch.bfloat16) * (1.0 + i)
        eager = block(fresh)                         # eager work between the replays, on the same workspaces
        torch.cuda.synchronize()
        static_x.copy_(fresh)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, eager), f"replay {i}"
