"""GPU parity of the multi-tensor optimizer step against the CPU oracle (which is
torch.optim bit for bit).  Floating point: parameter and moments must agree with the oracle
to 2e-6 relative (plus 2e-6 of the learning rate for parameters near zero - an update is at
most about lr); the model copy must be the bit-exact rounding of the GPU's own parameter."""
import pytest
import torch

import rannc_amd
from oracle import gradpath as oracle
from oracle import optim as oracle_optim
from rannc_amd import _lib, amp
from rannc_amd.fused_optim import FusedAdam, FusedAdamW, FusedSGD
from rannc_amd.multi_tensor import TensorPlan, stream_handle
from tests.helpers import TORCH_DTYPE, assert_bits_equal, place_in_arena

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SHAPES = [(1,), (5,), (31,), (32,), (33,), (1023,), (1024,), (1025,), (3, 700), (16384,), (16385,), (16384 + 31,), (50001,)]
RTOL = 2e-6


def close(got, want, atol, what):
    torch.testing.assert_close(got.detach().cpu(), want, rtol=RTOL, atol=atol, msg=lambda m: f"{what}: {m}")


def _rand(seed, scale, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(s, generator=g) * scale).to(dtype) for s in SHAPES]


@pytest.mark.parametrize("grad_name,copy_name", [("f32", "bf16"), ("f32", "f16"), ("f32", None), ("bf16", "bf16"), ("f16", None), ("f32", "f32")])
@pytest.mark.parametrize("param_lead,grad_lead", [(0, 0), (1, 3), (5, 0)])
def test_adam_table_matches_oracle(grad_name, copy_name, param_lead, grad_lead):
    gdt = TORCH_DTYPE[grad_name]
    p_cpu = _rand(1, 1.0)
    m_cpu = [torch.zeros_like(p) for p in p_cpu]
    v_cpu = [torch.zeros_like(p) for p in p_cpu]
    p_dev = place_in_arena(p_cpu, DEV, 32 + param_lead, 0 if param_lead == 0 else 1)
    m_dev = place_in_arena(m_cpu, DEV, 32 + param_lead, 0 if param_lead == 0 else 1)
    v_dev = place_in_arena(v_cpu, DEV, 32, 2)
    g_dev = place_in_arena(_rand(2, 1e-2, gdt), DEV, 32 + grad_lead, 0 if grad_lead == 0 else 1)
    copies = None
    if copy_name is not None:
        cdt = TORCH_DTYPE[copy_name]
        copies = place_in_arena([torch.zeros(s, dtype=cdt) for s in SHAPES], DEV, 64 + param_lead, 1)
    table = _lib.OptimTable(0, [t.data_ptr() for t in p_dev], [t.data_ptr() for t in g_dev], [t.data_ptr() for t in m_dev],
                            [t.data_ptr() for t in v_dev], [t.data_ptr() for t in copies] if copies else None,
                            [t.numel() for t in p_dev], [_lib.DTYPE_CODES[grad_name]] * len(SHAPES),
                            [_lib.DTYPE_CODES[copy_name]] * len(SHAPES) if copy_name else None)
    kw = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.01)
    for step in range(1, 5):
        grads = _rand(10 + step, 1e-2, gdt)
        for d, g in zip(g_dev, grads):
            d.copy_(g)
        table.adam_step(kw["lr"], kw["beta1"], kw["beta2"], kw["eps"], kw["weight_decay"], step,
                        stream=stream_handle(torch.device(DEV)))
        oracle_optim.adam_step(p_cpu, grads, m_cpu, v_cpu, step, **kw)
        for i in range(len(SHAPES)):
            close(p_dev[i], p_cpu[i], kw["lr"] * RTOL, f"param {i} step {step}")
            close(m_dev[i], m_cpu[i], 1e-12, f"exp_avg {i} step {step}")
            close(v_dev[i], v_cpu[i], 1e-16, f"exp_avg_sq {i} step {step}")
            if copies:
                assert_bits_equal(copies[i].cpu(), oracle_optim.model_copy(p_dev[i].cpu(), copies[i].dtype), f"model copy {i}")
        # keep the two trajectories from drifting apart: continue from the GPU's state
        for i in range(len(SHAPES)):
            p_cpu[i].copy_(p_dev[i]); m_cpu[i].copy_(m_dev[i]); v_cpu[i].copy_(v_dev[i])
    table.close()


def _models(seed=0):
    torch.manual_seed(seed)
    mk = lambda: torch.nn.Sequential(torch.nn.Linear(40, 64), torch.nn.Tanh(), torch.nn.Linear(64, 64), torch.nn.Tanh(),
                                     torch.nn.Linear(64, 3))
    a = mk()
    b = mk()
    b.load_state_dict(a.state_dict())
    return a, b.to(DEV)


@pytest.mark.parametrize("fused_cls,ref_cls,kw", [
    (FusedAdam, torch.optim.Adam, dict(lr=1e-3)),
    (FusedAdam, torch.optim.Adam, dict(lr=2e-3, betas=(0.8, 0.95), eps=1e-6, weight_decay=0.02)),
    (FusedAdam, torch.optim.Adam, dict(lr=1e-2, betas=(0.4, 0.9))),
    (FusedAdam, torch.optim.Adam, dict(lr=1e-3, maximize=True)),
    (FusedAdamW, torch.optim.AdamW, dict(lr=1e-3, weight_decay=0.1)),
    (FusedSGD, torch.optim.SGD, dict(lr=0.01)),
    (FusedSGD, torch.optim.SGD, dict(lr=0.05, momentum=0.9)),
    (FusedSGD, torch.optim.SGD, dict(lr=0.05, momentum=0.9, dampening=0.2, weight_decay=1e-3)),
    (FusedSGD, torch.optim.SGD, dict(lr=0.05, momentum=0.7, nesterov=True)),
])
def test_fused_optimizer_tracks_torch_optim(fused_cls, ref_cls, kw):
    cpu_model, gpu_model = _models()
    ref = ref_cls(cpu_model.parameters(), foreach=False, **kw)
    opt = fused_cls(gpu_model.parameters(), **kw)
    g = torch.Generator().manual_seed(5)
    for step in range(6):
        x = torch.randn(16, 40, generator=g)
        for model, inp in ((cpu_model, x), (gpu_model, x.to(DEV))):
            model.zero_grad(set_to_none=True)
            model(inp).pow(2).mean().backward()
        if step == 2:                                   # a parameter without a gradient is skipped (its step count lags)
            cpu_model[4].bias.grad = None
            gpu_model[4].bias.grad = None
        # same gradients on both sides: the comparison is of the optimizer, not of the matmuls
        for pc, pg in zip(cpu_model.parameters(), gpu_model.parameters()):
            if pc.grad is not None:
                pc.grad.copy_(pg.grad)
        ref.step()
        opt.step()
        for i, (pc, pg) in enumerate(zip(cpu_model.parameters(), gpu_model.parameters())):
            close(pg, pc.detach(), kw["lr"] * RTOL, f"param {i} step {step}")
            pc.data.copy_(pg.data)                      # resynchronise, as above
            for k, v in ref.state[pc].items():
                if k == "step":
                    assert float(opt.state[pg]["step"]) == float(v)
                elif v is not None:
                    close(opt.state[pg][k], v, 1e-12, f"{k} {i} step {step}")
                    v.copy_(opt.state[pg][k])
    sd, ref_sd = opt.state_dict()["state"], ref.state_dict()["state"]
    assert sd.keys() == ref_sd.keys()
    for k in sd:
        assert set(sd[k].keys()) == set(ref_sd[k].keys())


def test_gate_applies_the_clip_coefficient_and_skips_on_overflow():
    gdt = torch.float16
    grads = _rand(7, 64.0, gdt)
    g_dev = place_in_arena(grads, DEV, 0, 0)
    master_grads = [torch.zeros(s, device=DEV) for s in SHAPES]
    plan = TensorPlan(g_dev, master_grads)
    p_cpu = _rand(8, 1.0)
    p_dev = [p.to(DEV) for p in p_cpu]
    for p, mg in zip(p_dev, master_grads):
        p.grad = mg
    opt = FusedAdam(p_dev, lr=1e-3)
    opt.gate = plan.plan.result_device_ptr()
    # unscale without clipping, then let the optimizer consume the coefficient of a later clip decision
    plan.step_begin(1.0 / 64.0)
    plan.step_finish(0.0)                                # writes unclipped values, coef = 1
    plan.grad_norm()                                     # leaves coef = 1 in the result block
    res = plan.result()
    assert res.coef == 1.0
    opt.step()
    m = [torch.zeros_like(p) for p in p_cpu]
    v = [torch.zeros_like(p) for p in p_cpu]
    unscaled, _ = oracle.unscale_and_check(grads, 1.0 / 64.0)
    oracle_optim.adam_step(p_cpu, unscaled, m, v, 1)
    for a, b in zip(p_dev, p_cpu):
        close(a, b, 1e-9, "gate with coef 1")
    # overflow: the result block says skipped, the step must leave everything untouched
    before = [p.clone() for p in p_dev]
    grads[3][0] = float("inf")
    g_dev[3].copy_(grads[3])
    plan.step_begin(1.0 / 64.0)
    assert plan.result().overflow == 1
    plan.step_finish(1.0)
    opt.step()
    for a, b in zip(p_dev, before):
        assert torch.equal(a, b)
    # a clipped step: master grads hold the unclipped values (unscale_pack), the optimizer applies coef
    grads[3][0] = 0.0
    g_dev[3].copy_(grads[3])
    plan2 = TensorPlan(g_dev, master_grads)
    plan2.unscale_pack(1.0 / 64.0)
    norm = plan2.result().norm
    opt.gate = 0
    opt.grad_scale = float(torch.tensor(oracle.clip_coefficient(norm, 1.0) or 1.0, dtype=torch.float32))
    p_cpu = [p.cpu().clone() for p in p_dev]
    m = [opt.state[p]["exp_avg"].cpu().clone() for p in p_dev]
    v = [opt.state[p]["exp_avg_sq"].cpu().clone() for p in p_dev]
    opt.step()
    unscaled, _ = oracle.unscale_and_check(grads, 1.0 / 64.0)
    oracle_optim.adam_step(p_cpu, unscaled, m, v, int(opt.state[p_dev[0]]["step"]), grad_scale=opt.grad_scale)
    for a, b in zip(p_dev, p_cpu):
        close(a, b, 1e-9, "grad_scale")


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("half", [torch.float16, torch.bfloat16])
def test_amp_with_fused_adam_writes_model_copies_from_the_step(half, fused):
    torch.manual_seed(3)
    model = torch.nn.Sequential(torch.nn.Linear(32, 48), torch.nn.Tanh(), torch.nn.Linear(48, 8)).to(DEV)
    opt = FusedAdam(model.parameters(), lr=1e-2)
    model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8, half_dtype=half, fused=fused)
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    masters_before = None
    for it in range(3):
        x = torch.randn(16, 32, device=DEV, dtype=half)
        loss = rm(x).float().pow(2).mean()
        with amp.scale_loss(loss, opt) as scaled:
            scaled.backward()
            model_grads = [p.grad.detach().cpu().clone() for p in opt._amp_stash.all_fp16_params]
        stash = opt._amp_stash
        assert getattr(stash, "optimizer_copies_back", False) and stash.copy_back_plan is None
        masters = stash.all_fp32_from_fp16_params
        m_cpu = [m.detach().cpu().clone() for m in masters]
        if fused:       # the master gradients are never written: the step kernel unscales the model gradients itself
            assert stash.pending_finish
            g_cpu, _ = oracle.unscale_and_check(model_grads, 1.0 / 256.0)
        else:
            g_cpu = [m.grad.detach().cpu().clone() for m in masters]
        ms = [opt.state[m]["exp_avg"].cpu().clone() if m in opt.state and len(opt.state[m]) else torch.zeros_like(c) for m, c in zip(masters, m_cpu)]
        vs = [opt.state[m]["exp_avg_sq"].cpu().clone() if m in opt.state and len(opt.state[m]) else torch.zeros_like(c) for m, c in zip(masters, m_cpu)]
        opt.step()
        oracle_optim.adam_step(m_cpu, g_cpu, ms, vs, it + 1, lr=1e-2)
        for m, want, p in zip(masters, m_cpu, stash.all_fp16_params):
            close(m, want, 1e-2 * RTOL, f"master it {it}")
            assert_bits_equal(p.detach().cpu(), oracle_optim.model_copy(m.detach().cpu(), half), "model copy written by the step")
        opt.zero_grad()
        rm.zero_grad()
    assert stash.copy_back_plan is None                   # the separate copy-back pass never ran


def test_bad_arguments_are_value_errors():
    p = torch.zeros(10, device=DEV)
    g = torch.zeros(10, device=DEV)
    t = _lib.OptimTable(0, [p.data_ptr()], [g.data_ptr()], None, None, None, [10], [_lib.RG_F32])
    with pytest.raises(ValueError, match="exp_avg"):
        t.adam_step(1e-3, 0.9, 0.999, 1e-8, 0.0, 1)
    with pytest.raises(ValueError, match="momentum"):
        t.sgd_step(0.1, momentum=0.9)
    t.sgd_step(0.1)
    with pytest.raises(ValueError):
        _lib.OptimTable(0, [p.data_ptr() + 2], [g.data_ptr()], None, None, None, [4], [_lib.RG_F32])
    with pytest.raises(ValueError):
        _lib.OptimTable(0, [p.data_ptr()], [0], None, None, None, [4], [_lib.RG_F32])
    m, v = torch.zeros(10, device=DEV), torch.zeros(10, device=DEV)
    t2 = _lib.OptimTable(0, [p.data_ptr()], [g.data_ptr()], [m.data_ptr()], [v.data_ptr()], None, [10], [_lib.RG_F32])
    with pytest.raises(ValueError, match="hyper"):
        t2.adam_step(1e-3, 1.0, 0.999, 1e-8, 0.0, 1)
    with pytest.raises(ValueError, match="hyper"):
        t2.adam_step(1e-3, 0.9, 0.999, 1e-8, 0.0, 0)
    with pytest.raises(ValueError, match="fp32"):
        q = torch.zeros(4, device=DEV, dtype=torch.bfloat16, requires_grad=True)
        q.grad = torch.zeros_like(q)
        FusedAdam([q]).step()


def test_whole_step_fused_unscale_clip_then_fused_adam():
    """scale_loss (read pass) -> clip_grad_norm -> FusedAdam.step, two ways: (A) the clipped master
    gradients are written (write pass) and Adam reads them; (B) nothing is written, the step kernel
    reads the scaled model gradients and the clip decision from the device.  A is checked against
    the oracle's sequence unscale -> norm -> clip -> Adam -> half(master); B must equal A bit for bit."""
    import copy
    half = torch.bfloat16
    torch.manual_seed(11)
    base = torch.nn.Sequential(torch.nn.Linear(64, 96), torch.nn.Tanh(), torch.nn.Linear(96, 10)).to(DEV)
    flows = {}
    for name in ("A", "B"):
        model = copy.deepcopy(base)
        opt = FusedAdam(model.parameters(), lr=5e-3, weight_decay=0.01)
        model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 10, half_dtype=half, fused=True)
        flows[name] = (model, opt, rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True))
    ms = vs = None
    g = torch.Generator().manual_seed(12)
    for it in range(3):
        x = torch.randn(32, 64, generator=g).to(DEV).to(half)
        results = {}
        for name, (model, opt, rm) in flows.items():
            loss = rm(x).float().pow(2).sum()
            with amp.scale_loss(loss, opt) as scaled:
                scaled.backward()
                model_grads = [p.grad.detach().cpu().clone() for p in opt._amp_stash.all_fp16_params]
            stash = opt._amp_stash
            masters = stash.all_fp32_from_fp16_params
            rm.clip_grad_norm(0.5)
            assert stash.pending_finish and stash.decided_max_norm == 0.5          # only the decision was taken
            if name == "A":
                amp.finish_unscale(opt)                                             # write the clipped master gradients
                want = oracle.fused_step(model_grads, ["f32"] * len(model_grads), 1.0 / 2.0 ** 10, 0.5)
                assert want.coef is not None, "the test is meant to clip"
                offs = 0
                for m in masters:
                    w = want.buckets["f32"][offs:offs + m.numel()].view(m.shape)
                    torch.testing.assert_close(m.grad.cpu(), w, rtol=2e-6, atol=0.0)  # coef agrees to 1e-6, values follow
                    offs += m.numel()
                m_cpu = [m.detach().cpu().clone() for m in masters]
                g_cpu = [m.grad.detach().cpu().clone() for m in masters]
                if ms is None:
                    ms = [torch.zeros_like(t) for t in m_cpu]
                    vs = [torch.zeros_like(t) for t in m_cpu]
            opt.step()
            assert not stash.pending_finish
            if name == "A":
                oracle_optim.adam_step(m_cpu, g_cpu, ms, vs, it + 1, lr=5e-3, weight_decay=0.01)
                for m, w, p in zip(masters, m_cpu, stash.all_fp16_params):
                    close(m, w, 5e-3 * RTOL, f"master it {it}")
                    assert_bits_equal(p.detach().cpu(), oracle_optim.model_copy(m.detach().cpu(), half), "model copy")
                for a, b, m in zip(ms, vs, masters):
                    a.copy_(opt.state[m]["exp_avg"]); b.copy_(opt.state[m]["exp_avg_sq"])
            results[name] = ([m.detach().cpu().clone() for m in masters],
                             [p.detach().cpu().clone() for p in stash.all_fp16_params],
                             [opt.state[m]["exp_avg_sq"].cpu().clone() for m in masters])
            opt.zero_grad()          # master gradients go back to None: the next unscale overwrites (else it accumulates)
        for k in range(3):
            for a, b in zip(results["A"][k], results["B"][k]):
                assert_bits_equal(b, a, f"direct step vs materialised step, it {it}")


def test_direct_step_skips_on_overflow_and_without_clip_call():
    half = torch.float16
    torch.manual_seed(13)
    model = torch.nn.Sequential(torch.nn.Linear(16, 16), torch.nn.Linear(16, 4)).to(DEV)
    opt = FusedSGD(model.parameters(), lr=0.1)
    model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8, half_dtype=half, fused=True)
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    x = torch.randn(8, 16, device=DEV, dtype=half)
    # no clip_grad_norm at all: the step takes the (no-clip) decision itself
    loss = rm(x).float().pow(2).mean()
    with amp.scale_loss(loss, opt) as scaled:
        scaled.backward()
        grads = [p.grad.detach().cpu().clone() for p in opt._amp_stash.all_fp16_params]
    masters = opt._amp_stash.all_fp32_from_fp16_params
    before = [m.detach().cpu().clone() for m in masters]
    opt.step()
    unscaled, _ = oracle.unscale_and_check(grads, 1.0 / 256.0)
    oracle_optim.sgd_step(before, unscaled, None, 0.1)
    for m, w in zip(masters, before):
        close(m, w, 1e-8, "sgd from model grads")
    opt.zero_grad()
    # overflow: the scaler arms the skip; nothing may change
    loss = rm(x).float().pow(2).mean() * float("inf")
    with amp.scale_loss(loss, opt) as scaled:
        scaled.backward()
    snap = [m.detach().clone() for m in masters]
    opt.step()
    for m, s0 in zip(masters, snap):
        assert torch.equal(m, s0)
    assert amp._amp_state.loss_scalers[0].loss_scale() == 128.0


@pytest.mark.gpu
def test_optimizer_step_on_a_tensor_beyond_two_to_the_31_elements():
    """Plain SGD on one parameter of 2^31 + 4099 elements: the optimizer kernel's offsets inside a tensor are 64-bit.
    ``p - lr * g`` evaluated by torch on the device, slice by slice, is the yardstick (2e-6 relative, the bar of the
    optimizer step)."""
    dev = torch.device("cuda", 0)
    n = 2 ** 31 + 4099
    gen = torch.Generator(device=dev).manual_seed(9)
    p = torch.nn.Parameter(torch.empty(n, device=dev))
    g = torch.empty(n, device=dev)
    step = 2 ** 28
    with torch.no_grad():
        for lo in range(0, n, step):
            hi = min(n, lo + step)
            p[lo:hi] = torch.randn(hi - lo, generator=gen, device=dev)
            g[lo:hi] = torch.randn(hi - lo, generator=gen, device=dev)
    before = p.detach().clone()
    p.grad = g
    opt = FusedSGD([p], lr=0.25)
    opt.step()
    torch.cuda.synchronize()
    with torch.no_grad():
        for lo in range(0, n, step):                     # every element, slice by slice
            hi = min(n, lo + step)
            torch.testing.assert_close(p[lo:hi], before[lo:hi] - 0.25 * g[lo:hi], rtol=2e-6, atol=1e-7)


@pytest.mark.parametrize("fused_cls,kw", [(FusedAdam, dict(lr=1e-2)), (FusedSGD, dict(lr=0.05, momentum=0.9))])
def test_gradients_that_move_away_and_back_are_followed(fused_cls, kw):
    """Gradients at addresses A (full step), at B (steady step: the device table is re-pointed), one step with a
    missing gradient (full path again), then all gradients back at A: the table must read A, not the B it was last
    pointed at.  Compared step by step with a twin optimizer that is handed the same values in fresh tensors."""
    torch.manual_seed(3)
    shapes = [(257,), (64, 33), (5,)]
    params = [torch.nn.Parameter(torch.randn(s, device=DEV)) for s in shapes]
    twins = [torch.nn.Parameter(p.detach().clone()) for p in params]
    opt, ref = fused_cls(params, **kw), fused_cls(twins, **kw)
    set_a = [torch.randn(s, device=DEV) for s in shapes]
    set_b = [torch.randn(s, device=DEV) for s in shapes]
    plan = [(set_a, None), (set_a, None), (set_b, None), (set_b, 1), (set_a, None), (set_a, None)]
    for step, (grads, missing) in enumerate(plan):
        for i, (p, t, g) in enumerate(zip(params, twins, grads)):
            g.normal_()                                           # new values at the same addresses
            p.grad = None if i == missing else g
            t.grad = None if i == missing else g.clone()          # the twin always sees fresh tensors
        if step == 3:
            ref.invalidate_tables()
        opt.step()
        ref.step()
        for i, (p, t) in enumerate(zip(params, twins)):
            assert_bits_equal(p.detach(), t.detach(), f"param {i} after step {step}")


def test_invalidate_tables_after_rehoming_a_parameter():
    """A parameter whose storage is replaced between steps (``p.data = ...``, what the offload wrapper and
    ``_sync_orig_params`` do) is followed once ``invalidate_tables`` has been called."""
    torch.manual_seed(4)
    params = [torch.nn.Parameter(torch.randn(s, device=DEV)) for s in ((100,), (33, 7), (4096,))]
    twins = [torch.nn.Parameter(p.detach().clone()) for p in params]
    opt, ref = FusedAdam(params, lr=1e-2), FusedAdam(twins, lr=1e-2)
    grads = [torch.randn(p.shape, device=DEV) for p in params]
    for step in range(4):
        for p, t, g in zip(params, twins, grads):
            g.normal_()
            p.grad, t.grad = g, g.clone()
        if step == 2:
            with torch.no_grad():
                params[1].data = params[1].data.clone()           # middle parameter: not seen by the first / last check
            opt.invalidate_tables()
        opt.step()
        ref.step()
        for i, (p, t) in enumerate(zip(params, twins)):
            assert_bits_equal(p.detach(), t.detach(), f"param {i} after step {step}")


@pytest.mark.parametrize("fused_cls", [FusedAdam, FusedSGD])
def test_step_hooks_grad_mode_and_schedulers_behave_as_with_torch_optim(fused_cls):
    """The fused optimizers bring their own wrapper around ``step`` (torch's costs about 10 us per call); what torch's
    does for a caller must still happen: registered and global step hooks run in torch's order and may replace the
    arguments, gradient mode is off inside the step and back afterwards, a closure runs with it on, a learning-rate
    scheduler counts the steps, and a recording profiler sees the ``Optimizer.step#...`` range."""
    from torch.optim.optimizer import register_optimizer_step_post_hook, register_optimizer_step_pre_hook
    p = torch.nn.Parameter(torch.ones(1000, device=DEV))
    opt = fused_cls([p], lr=0.1)
    sched = torch.optim.lr_scheduler.StepLR(opt, step_size=2, gamma=0.5)
    calls = []
    closure_modes = []

    def closure():
        closure_modes.append(torch.is_grad_enabled())
        return torch.tensor(3.0)

    def swap_in_closure(o, args, kwargs):
        calls.append("pre")
        return (args[0], closure), kwargs           # new positional arguments: (self, closure)

    handles = [register_optimizer_step_pre_hook(lambda o, a, k: calls.append("global_pre")),
               opt.register_step_pre_hook(swap_in_closure),
               opt.register_step_post_hook(lambda o, a, k: calls.append(("post", len(a)))),
               register_optimizer_step_post_hook(lambda o, a, k: calls.append("global_post"))]
    try:
        for step in range(3):
            p.grad = torch.full_like(p, 0.5)
            assert torch.is_grad_enabled()
            out = opt.step()
            assert torch.is_grad_enabled()
            assert float(out) == 3.0                 # the closure the pre-hook put in was called
            sched.step()
        assert calls == ["global_pre", "pre", ("post", 2), "global_post"] * 3
        assert closure_modes == [True] * 3
        assert opt.param_groups[0]["lr"] == pytest.approx(0.05)      # halved once after two counted steps
    finally:
        for h in handles:
            h.remove()
    ref = torch.nn.Parameter(torch.ones(1000))
    ref_opt = {FusedAdam: torch.optim.Adam, FusedSGD: torch.optim.SGD}[fused_cls]([ref], lr=0.1)
    ref_sched = torch.optim.lr_scheduler.StepLR(ref_opt, step_size=2, gamma=0.5)
    for step in range(3):
        ref.grad = torch.full_like(ref, 0.5)
        ref_opt.step()
        ref_sched.step()
    torch.testing.assert_close(p.detach().cpu(), ref.detach(), rtol=2e-6, atol=1e-7)
    # a recording profiler still sees the range torch's wrapper would have opened
    p.grad = torch.full_like(p, 0.5)
    with torch.profiler.profile(activities=[torch.profiler.ProfilerActivity.CPU]) as prof:
        opt.step()
    assert any(e.key == f"Optimizer.step#{fused_cls.__name__}.step" for e in prof.key_averages())
    # an exception inside the step must not leave gradient mode off
    def failing_closure():
        raise ValueError("from the closure")

    with pytest.raises(ValueError, match="from the closure"):
        opt.step(failing_closure)
    assert torch.is_grad_enabled()
