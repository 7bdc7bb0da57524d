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


def test_unscale_pack_zero_and_sgd_replay_from_a_graph():
    """One captured graph: zero the bucket, unscale + pack the gradients into it, SGD step with
    the model copy.  Replays must track new gradient values and keep updating the parameters."""
    from oracle import gradpath as oracle
    from oracle import optim as oracle_optim
    from rannc_amd import _lib
    from rannc_amd.multi_tensor import stream_handle
    g = torch.Generator().manual_seed(10)
    shapes = [(50001,), (33,), (4096,)]
    grads_cpu = [(torch.randn(s, generator=g) * 64).to(torch.float16) for s in shapes]
    grads = [t.to(DEV) for t in grads_cpu]
    bucket = [torch.full(s, 7.0, device=DEV) for s in shapes]
    params_cpu = [torch.randn(s, generator=g) for s in shapes]
    params = [t.to(DEV) for t in params_cpu]
    copies = [torch.zeros(s, device=DEV, dtype=torch.float16) for s in shapes]
    plan = TensorPlan(grads, bucket)
    table = _lib.OptimTable(0, [t.data_ptr() for t in params], [t.data_ptr() for t in bucket], None, None,
                            [t.data_ptr() for t in copies], [t.numel() for t in params], [_lib.RG_F32] * 3, [_lib.RG_F16] * 3)

    def step():
        plan.zero()
        plan.unscale_pack(1.0 / 64.0)
        table.sgd_step(0.1, weight_decay=0.01, stream=stream_handle(torch.device(DEV)))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                            # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    unscaled, _ = oracle.unscale_and_check(grads_cpu, 1.0 / 64.0)
    oracle_optim.sgd_step(params_cpu, unscaled, None, 0.1, weight_decay=0.01)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for replay in range(4):
        if replay == 2:                                   # new gradients in the same buffers
            for gc, gd in zip(grads_cpu, grads):
                gc.mul_(0.5)
                gd.copy_(gc)
            unscaled, _ = oracle.unscale_and_check(grads_cpu, 1.0 / 64.0)
        for b in bucket:
            b.fill_(float(replay + 3))                    # eager work between replays; must be overwritten
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        oracle_optim.sgd_step(params_cpu, unscaled, None, 0.1, weight_decay=0.01)
        assert plan.result().overflow == 0
        for b, u in zip(bucket, unscaled):
            assert_bits_equal(b.cpu(), u, f"bucket replay {replay}")
        for p, w, c in zip(params, params_cpu, copies):
            torch.testing.assert_close(p.cpu(), w, rtol=2e-6, atol=2e-7)
            assert_bits_equal(c.cpu(), p.cpu().to(torch.float16), f"model copy replay {replay}")
            w.copy_(p.cpu())                              # continue from the GPU's trajectory
    table.close()
