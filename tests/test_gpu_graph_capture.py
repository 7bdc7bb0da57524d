"""The per-step entry points allocate nothing and launch only kernels (no memset nodes), so a
caller may capture them in a HIP graph.  Every replay is checked against the eager result,
with eager work and synchronisation between replays."""
import pytest
import torch

from rannc_amd.multi_tensor import TensorPlan
from tests.helpers import assert_bits_equal

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_fused_step_replays_from_a_graph():
    g = torch.Generator().manual_seed(9)
    cpu = [(torch.randn(s, generator=g) * 1e-2 * 4096).to(torch.float16) for s in [(100003,), (17,), (8192,)]]
    srcs = [t.to(DEV) for t in cpu]
    eager_out = [torch.zeros(t.shape, device=DEV) for t in cpu]
    graph_out = [torch.zeros(t.shape, device=DEV) for t in cpu]
    eager = TensorPlan(srcs, eager_out)
    captured = TensorPlan(srcs, graph_out)
    eager.fused_step(1 / 4096.0, 0.5)
    want = eager.result()
    torch.cuda.synchronize()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        captured.fused_step(1 / 4096.0, 0.5)          # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured.fused_step(1 / 4096.0, 0.5)
    for replay in range(4):
        for o in graph_out:
            o.fill_(float(replay + 1))                # eager work between replays; must be overwritten
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = captured.result()
        assert (got.norm, got.coef, got.overflow, got.clipped) == (want.norm, want.coef, want.overflow, want.clipped)
        for a, b in zip(graph_out, eager_out):
            assert_bits_equal(a.cpu(), b.cpu(), f"replay {replay}")
    # new gradient values in the same buffers are picked up by the next replay
    for s in srcs:
        s.mul_(0.5)
    eager.fused_step(1 / 4096.0, 0.5)
    want2 = eager.result()
    graph.replay()
    torch.cuda.synchronize()
    got2 = captured.result()
    assert (got2.norm, got2.coef) == (want2.norm, want2.coef) and got2.norm != want.norm
    for a, b in zip(graph_out, eager_out):
        assert_bits_equal(a.cpu(), b.cpu(), "replay after new gradients")
