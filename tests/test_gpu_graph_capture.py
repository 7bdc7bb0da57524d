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


def test_capturable_adam_matches_the_host_counted_step():
    """``FusedAdam(capturable=True)`` keeps its step count on the device; run eagerly it must walk the same
    trajectory as the host-counted optimizer (the factors are computed in double on both sides)."""
    from rannc_amd.fused_optim import FusedAdam
    g = torch.Generator().manual_seed(12)
    shapes = [(30001,), (17,), (4096, 3)]
    init = [torch.randn(s, generator=g) for s in shapes]
    runs = {}
    for capturable in (False, True):
        ps = [torch.nn.Parameter(t.clone().to(DEV)) for t in init]
        opt = FusedAdam(ps, lr=1e-2, betas=(0.9, 0.99), weight_decay=0.01, capturable=capturable)
        gg = torch.Generator().manual_seed(13)
        for _ in range(5):
            for p in ps:
                p.grad = torch.randn(p.shape, generator=gg).to(DEV)
            opt.step()
        torch.cuda.synchronize()
        runs[capturable] = ([p.detach().cpu() for p in ps], [opt.state[p]["exp_avg_sq"].cpu() for p in ps], opt)
    for a, b in zip(runs[False][0] + runs[False][1], runs[True][0] + runs[True][1]):
        torch.testing.assert_close(b, a, rtol=2e-6, atol=1e-8)
    opt = runs[True][2]
    step = opt.state[opt.param_groups[0]["params"][0]]["step"]
    assert step.is_cuda and step.dtype == torch.float32 and float(step) == 5.0
    # the state dict round trip re-seeds the device count
    ps2 = [torch.nn.Parameter(t.clone()) for t in runs[True][0]]
    ps2 = [torch.nn.Parameter(p.detach().to(DEV)) for p in ps2]
    opt2 = FusedAdam(ps2, lr=1e-2, betas=(0.9, 0.99), weight_decay=0.01, capturable=True)
    import copy
    opt2.load_state_dict(copy.deepcopy(opt.state_dict()))     # as torch.save / torch.load would hand it over
    gg = torch.Generator().manual_seed(14)
    grads = [torch.randn(p.shape, generator=gg).to(DEV) for p in ps2]
    for p, q, gr in zip(opt.param_groups[0]["params"], ps2, grads):
        p.grad, q.grad = gr.clone(), gr.clone()
    opt.step()
    opt2.step()
    torch.cuda.synchronize()
    for p, q in zip(opt.param_groups[0]["params"], ps2):
        assert_bits_equal(q.detach().cpu(), p.detach().cpu(), "after a state-dict round trip")
    assert float(opt2.state[ps2[0]]["step"]) == 6.0


def test_whole_optimizer_phase_replays_from_a_graph_with_a_skipped_step():
    """Unscale + flag + norm + clip decision (``rg_step_begin`` / ``rg_step_decide``), the device-side step count and
    the Adam step that reads the still-scaled fp16 gradients through the gate - one HIP graph, nothing decided on
    the host.  Replayed with new gradients each time; a replay whose gradients hold an inf must leave the
    parameters, the moments and the step count as they were; every replay is compared with the CPU oracle."""
    from oracle import gradpath as oracle
    from oracle import optim as oracle_optim
    from rannc_amd.fused_optim import FusedAdam
    gen = torch.Generator().manual_seed(15)
    shapes = [(20001,), (5,), (3000, 7)]
    scale, max_norm = 128.0, 0.5
    masters_cpu = [torch.randn(s, generator=gen) for s in shapes]
    m_cpu = [torch.zeros(s) for s in shapes]
    v_cpu = [torch.zeros(s) for s in shapes]
    masters = [torch.nn.Parameter(t.clone().to(DEV)) for t in masters_cpu]
    models = [t.detach().to(torch.float16) for t in masters]
    static_grads = [torch.zeros(s, dtype=torch.float16, device=DEV) for s in shapes]
    bucket = [torch.zeros(s, device=DEV) for s in shapes]                 # never written on this route
    plan = TensorPlan(static_grads, bucket)
    opt = FusedAdam(masters, lr=1e-2, capturable=True)
    opt.set_model_copies(masters, models)
    opt.set_grad_sources(masters, static_grads)
    opt.grad_scale = 1.0 / scale
    opt.gate = plan.plan.result_device_ptr()

    def phase():
        plan.plan.step_begin(1.0 / scale, stream_of())
        plan.plan.step_decide(max_norm, 0, stream_of())
        opt.step()

    def stream_of():
        from rannc_amd.multi_tensor import stream_handle
        return stream_handle(torch.device(DEV))

    def new_grads(poison=False):
        out = [(torch.randn(s, generator=gen) * 0.1 * scale).to(torch.float16) for s in shapes]
        if poison:
            out[2].view(-1)[1234] = float("inf")
        return out

    steps_done = 0

    def oracle_step(grads_cpu):
        nonlocal steps_done
        want = oracle.fused_step(grads_cpu, ["f32"] * len(shapes), 1.0 / scale, max_norm)
        if want.overflow:
            return want
        steps_done += 1
        unscaled, _ = oracle.unscale_and_check(grads_cpu, 1.0 / scale)
        if want.coef is not None:
            unscaled = [u * torch.tensor(want.coef, dtype=torch.float32) for u in unscaled]
        oracle_optim.adam_step(masters_cpu, unscaled, m_cpu, v_cpu, steps_done, lr=1e-2)
        return want

    # one eager step outside the capture: allocates the state and the tables
    g0 = new_grads()
    for s, g in zip(static_grads, g0):
        s.copy_(g)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        phase()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    oracle_step(g0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        phase()
    # the capture itself does not run the kernels
    assert float(opt.state[masters[0]]["step"]) == 1.0
    for replay, poison in enumerate([False, True, False, False]):
        gc = new_grads(poison)
        for s, g in zip(static_grads, gc):
            s.copy_(g)                                         # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = oracle_step(gc)
        res = plan.result()
        assert res.overflow == want.overflow == (1 if poison else 0)
        assert float(opt.state[masters[0]]["step"]) == float(steps_done)
        for p, w, c in zip(masters, masters_cpu, models):
            torch.testing.assert_close(p.detach().cpu(), w, rtol=2e-6, atol=2e-8, msg=f"replay {replay}")
            assert_bits_equal(c.cpu(), p.detach().cpu().to(torch.float16), f"model copy, replay {replay}")
        for p, w in zip(masters, m_cpu):
            torch.testing.assert_close(opt.state[p]["exp_avg"].cpu(), w, rtol=2e-6, atol=1e-9)
        for p, w in zip(masters, masters_cpu):
            w.copy_(p.detach().cpu())                          # continue from the GPU's trajectory
        for p, w, x in zip(masters, m_cpu, v_cpu):
            w.copy_(opt.state[p]["exp_avg"].cpu())
            x.copy_(opt.state[p]["exp_avg_sq"].cpu())
    assert steps_done == 4
    plan.close()


def test_dynamic_loss_scale_on_the_device_replays_from_a_graph():
    """The whole mixed-precision optimizer phase with a *dynamic* loss scale and no host read: the unscale reads
    ``1 / scale`` from the scaler's state on the device (``rg_step_begin_scaled``), the clip decision and the Adam
    step (device-resident count, gated) follow, then one thread applies the schedule (``rg_scaler_update``: halve
    and truncate on overflow, double after ``scale_window`` clean steps).  Seven replays of one HIP graph - two with
    an inf, two window doublings - against the oracle's ``patched_update_scale`` sequence and its Adam step."""
    import ctypes
    from oracle import gradpath as oracle
    from oracle import optim as oracle_optim
    from rannc_amd import _lib
    from rannc_amd.fused_optim import FusedAdam
    from rannc_amd.multi_tensor import stream_handle
    dev = torch.device(DEV)
    gen = torch.Generator().manual_seed(16)
    shapes = [(20001,), (5,), (3000, 7)]
    max_norm = 0.5
    want_scaler = oracle.LossScalerState(loss_scale=25.0, unskipped=0, scale_window=2, min_loss_scale=None,
                                         max_loss_scale=2.0 ** 24, dynamic=True)
    masters_cpu = [torch.randn(s, generator=gen) for s in shapes]
    m_cpu = [torch.zeros(s) for s in shapes]
    v_cpu = [torch.zeros(s) for s in shapes]
    masters = [torch.nn.Parameter(t.clone().to(DEV)) for t in masters_cpu]
    models = [t.detach().to(torch.float16) for t in masters]
    static_grads = [torch.zeros(s, dtype=torch.float16, device=DEV) for s in shapes]
    bucket = [torch.zeros(s, device=DEV) for s in shapes]                 # never written on this route
    plan = TensorPlan(static_grads, bucket)
    state = torch.zeros(_lib.SCALER_STATE_BYTES // 4, dtype=torch.float32, device=DEV)
    _lib.scaler_init(state.data_ptr(), 25.0, 0.0, 2.0 ** 24, 2, 2.0, 0, stream_handle(dev))
    inv_ptr = state.data_ptr() + _lib.SCALER_INV_SCALE_OFFSET
    opt = FusedAdam(masters, lr=1e-2, capturable=True)
    opt.set_model_copies(masters, models)
    opt.set_grad_sources(masters, static_grads)
    opt.grad_scale_ptr = inv_ptr
    opt.gate = plan.plan.result_device_ptr()

    def phase():
        s = stream_handle(dev)
        plan.plan.step_begin_scaled(inv_ptr, s)
        plan.plan.step_decide(max_norm, 0, s)
        opt.step()
        _lib.scaler_update(state.data_ptr(), plan.plan.result_device_ptr(), _lib.RG_SCALER_DYNAMIC | _lib.RG_SCALER_TRUNCATE, 0, s)

    def device_scaler():
        raw = state.cpu().numpy().tobytes()
        return _lib.ScalerState.from_buffer_copy(raw)

    def new_grads(scale, poison=False):
        out = [(torch.randn(s, generator=gen) * 0.1 * scale).to(torch.float16) for s in shapes]
        if poison:
            out[0].view(-1)[77] = float("nan")
        return out

    steps_done = 0

    def oracle_step(grads_cpu):
        nonlocal steps_done
        inv = 1.0 / want_scaler.loss_scale
        want = oracle.fused_step(grads_cpu, ["f32"] * len(shapes), inv, max_norm)
        skipped = oracle.patched_update_scale(want_scaler, bool(want.overflow))
        assert skipped == bool(want.overflow)
        if want.overflow:
            return want
        steps_done += 1
        unscaled, _ = oracle.unscale_and_check(grads_cpu, inv)
        if want.coef is not None:
            unscaled = [u * torch.tensor(want.coef, dtype=torch.float32) for u in unscaled]
        oracle_optim.adam_step(masters_cpu, unscaled, m_cpu, v_cpu, steps_done, lr=1e-2)
        return want

    g0 = new_grads(want_scaler.loss_scale)
    for s, g in zip(static_grads, g0):
        s.copy_(g)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        phase()                                                # eager: allocates the state and the tables
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    oracle_step(g0)
    assert (device_scaler().loss_scale, device_scaler().unskipped) == (25.0, 1)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        phase()
    scales_seen = []
    # scale 25, one clean step done: clean -> 50 (window), inf -> 25, clean, inf -> 12 (12.5 truncated), clean, clean -> 24
    for replay, poison in enumerate([False, True, False, True, False, False, False]):
        gc = new_grads(want_scaler.loss_scale, poison)
        for s, g in zip(static_grads, gc):
            s.copy_(g)                                         # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = oracle_step(gc)
        res = plan.result()
        got = device_scaler()
        assert res.overflow == want.overflow == (1 if poison else 0) and res.skipped == res.overflow
        assert (got.loss_scale, got.unskipped) == (float(want_scaler.loss_scale), want_scaler.unskipped), f"replay {replay}"
        assert got.inv_scale == torch.tensor(1.0 / want_scaler.loss_scale, dtype=torch.float32).item()
        scales_seen.append(got.loss_scale)
        assert float(opt.state[masters[0]]["step"]) == float(steps_done)
        for p, w, c in zip(masters, masters_cpu, models):
            torch.testing.assert_close(p.detach().cpu(), w, rtol=2e-6, atol=2e-8, msg=f"replay {replay}")
            assert_bits_equal(c.cpu(), p.detach().cpu().to(torch.float16), f"model copy, replay {replay}")
        for p, w in zip(masters, masters_cpu):
            w.copy_(p.detach().cpu())                          # continue from the GPU's trajectory
        for p, w, x in zip(masters, m_cpu, v_cpu):
            w.copy_(opt.state[p]["exp_avg"].cpu())
            x.copy_(opt.state[p]["exp_avg_sq"].cpu())
    assert scales_seen == [50.0, 25.0, 25.0, 12.0, 12.0, 24.0, 24.0]      # written by hand from the schedule
    assert steps_done == 6 and device_scaler().skipped_steps == 2
    plan.close()


def test_paced_flat_fill_replays_from_a_graph():
    """A fill above 256 MiB holds every wavefront for a fixed wall-clock time before its stores (pacing); the kernel
    reads only the clock, so it can be captured like the others.  Guard bytes around the range stay as they were."""
    from rannc_amd.multi_tensor import fill_zero_
    n = (300 << 20) + 24                                   # bytes; the range starts 8 bytes into the allocation
    arena = torch.full((n + 16,), 0x5A, dtype=torch.uint8, device=DEV)
    target = arena[8:8 + n]
    fill_zero_(target)                                     # eager once: also the warm-up
    torch.cuda.synchronize()
    assert int(target.max()) == 0 and int(arena[:8].min()) == 0x5A and int(arena[8 + n:].min()) == 0x5A
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fill_zero_(target)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fill_zero_(target)
    for replay in range(3):
        arena.fill_(0x5A + replay)                         # eager work between replays; the range must be cleared again
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert int(target.max()) == 0, f"replay {replay}"
        assert int(arena[:8].min()) == 0x5A + replay and int(arena[8 + n:].min()) == 0x5A + replay
