"""GPU tests of the host-side mirror of the reference interface: ParamStorage /
GradConsolidation / locators, the _pyrannc surface, dist_param, amp and RaNNCModule.
Every expected value comes from the CPU oracle (or from plain slicing, which the reference's
own test uses as its invariant: ``segment == full.flatten()[range]``, test/common.py:57-63)."""
import math

import pytest
import torch

import rannc_amd
from oracle import gradpath as oracle
from rannc_amd import _pyrannc, amp
from rannc_amd import dist_param as dp
from rannc_amd.param_storage import DistributedGradLocator, GradConsolidation, ParamStorage
from tests.helpers import assert_bits_equal

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True)
def _fresh_registry():
    _pyrannc.clear()
    yield
    _pyrannc.clear()


def _params(shapes, dtypes, seed=0, requires_grad=True):
    g = torch.Generator().manual_seed(seed)
    return [torch.nn.Parameter(torch.randn(s, generator=g).to(dt).to(DEV), requires_grad=requires_grad)
            for s, dt in zip(shapes, dtypes)]


# ----------------------------------------------------------------------------- GradConsolidation

def test_consolidate_packs_copies_and_zeroes():
    shapes = [(3, 5), (7,), (2, 2, 2), (1,), (129,)]
    dts = [torch.float32, torch.bfloat16, torch.float32, torch.bfloat16, torch.float16]
    ps = _params(shapes, dts)
    st = ParamStorage()
    for p in ps:
        st.register_param(id(p), p)
    g = torch.Generator().manual_seed(1)
    grads_cpu = [torch.randn(s, generator=g).to(dt) for s, dt in zip(shapes, dts)]
    for i, p in enumerate(ps):
        if i != 3:                      # parameter 3 has no gradient: its view must read zero
            p.grad = grads_cpu[i].to(DEV)
    con = GradConsolidation(st, [id(p) for p in ps], False, False)
    con.consolidate()
    torch.cuda.synchronize()
    names = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}
    want = oracle.consolidate([None if i == 3 else gc for i, gc in enumerate(grads_cpu)],
                              [gc.numel() for gc in grads_cpu], [names[d] for d in dts])
    for dt, bucket in con.consolidated_grads.items():
        assert_bits_equal(bucket.cpu(), want[names[dt]], f"bucket {dt}")
    for p in ps:                         # every .grad is now the bucket view (ParamStorage.cpp:163-171)
        assert p.grad.data_ptr() == con.grad_tensors[id(p)].data_ptr() and p.grad.shape == p.shape
    # steady state: grads already alias the bucket -> nothing moves
    before = {dt: b.clone() for dt, b in con.consolidated_grads.items()}
    con.consolidate()
    for dt, b in con.consolidated_grads.items():
        assert torch.equal(b, before[dt])


def test_consolidate_amp_double_buffer_and_master_bucket():
    ps = _params([(10,), (6,)], [torch.float32, torch.float16])
    st = ParamStorage()
    for p in ps:
        st.register_param(id(p), p)
    master = ps[1].detach().clone().float().requires_grad_(True)
    st.register_amp_master_param(id(ps[1]), id(master), master)
    con = GradConsolidation(st, [id(p) for p in ps], True, True)
    assert torch.float16 in con.consolidated_master_grads and con.consolidated_master_grads[torch.float16].dtype == torch.float32
    first = con.consolidated_grads[torch.float32].data_ptr()
    con.consolidate()
    second = con.consolidated_grads[torch.float32].data_ptr()
    con.consolidate()
    assert first != second and con.consolidated_grads[torch.float32].data_ptr() == first   # swapped each time
    assert master.grad is not None and master.grad.dtype == torch.float32 and bool((master.grad == 0).all())
    assert master.grad.data_ptr() == con.amp_master_grad_tensors[id(ps[1])].data_ptr()


def test_unsupported_dtype_is_a_value_error():
    p = torch.nn.Parameter(torch.zeros(4, dtype=torch.float64, device=DEV))
    st = ParamStorage()
    st.register_param(id(p), p)
    with pytest.raises(ValueError, match="dtype"):
        GradConsolidation(st, [id(p)], False, False)
    with pytest.raises(ValueError, match="not found"):
        st.get_param_tensor(12345)


# ----------------------------------------------------------------------------- clip / norm / zero

@pytest.mark.parametrize("consolidate", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_module_clip_norm_zero(consolidate, dtype):
    torch.manual_seed(0)
    model = torch.nn.Sequential(torch.nn.Linear(64, 129), torch.nn.Linear(129, 7)).to(DEV).to(dtype)
    rm = rannc_amd.RaNNCModule(model, consolidate_grads=consolidate)
    x = torch.randn(16, 64, device=DEV, dtype=dtype)
    rm(x).float().pow(2).sum().backward()
    if consolidate:
        rm.prepare_backward()
    names = sorted(n for n, _ in model.named_parameters())
    named = dict(model.named_parameters())
    grads_cpu = [named[n].grad.detach().cpu().clone() for n in names]
    norm = rm._calc_grad_norm()
    assert math.isclose(norm, oracle.grad_global_l2_norm(grads_cpu), rel_tol=1e-6)
    max_norm = norm / 3.0
    rm.clip_grad_norm(max_norm)
    ref = [g.clone() for g in grads_cpu]
    want_norm, coef = oracle.clip_grad_norm(ref, max_norm)
    assert coef is not None
    # the coefficient is held to 1e-6; the clipped values must then be the unclipped ones times
    # that coefficient narrowed to fp32 (one multiply, rounded to the gradient's dtype)
    for n, g0 in zip(names, grads_cpu):
        got = named[n].grad.cpu()
        nz = g0.float() != 0
        ratio = (got.float()[nz].double() / g0.float()[nz].double()).median().item()
        assert math.isclose(ratio, coef, rel_tol=1e-2 if dtype == torch.bfloat16 else 1e-6)
        c32 = torch.tensor(coef, dtype=torch.float64).float()
        close = (g0.float() * c32).to(dtype)
        # same bits when the GPU's coefficient is the oracle's; otherwise within one ulp of it
        assert torch.allclose(got.float(), close.float(), rtol=2e-2 if dtype == torch.bfloat16 else 1e-6, atol=0)
    clipped = [named[n].grad.detach().cpu().clone() for n in names]
    rm.clip_grad_norm(1e9)               # far above the norm: nothing changes
    for n, c in zip(names, clipped):
        assert_bits_equal(named[n].grad.cpu(), c, n)
    rm.zero_grad()
    for n in names:
        assert bool((named[n].grad == 0).all())


def test_scale_and_unscale_grads():
    ps = _params([(100,), (33,)], [torch.float32, torch.float32])
    st = ParamStorage()
    ids = {}
    for i, p in enumerate(ps):
        st.register_param(id(p), p)
        p.grad = torch.full_like(p, 3.0)
        ids[f"p{i}"] = id(p)
    st.deploy("g", ids)
    st.scale_grads("g", False, world_size=4)
    assert all(bool((p.grad == 0.75).all()) for p in ps)
    st.unscale_grads("g", False, world_size=4)
    assert all(bool((p.grad == 3.0).all()) for p in ps)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("world", [3, 8])
def test_scale_and_unscale_grads_random_values(dtype, world):
    """``doScaleGrads`` (``src/comp/ParamStorage.cpp:598-615``) on random gradients of odd sizes, one of them
    missing: ``grad.mul_(ratio)`` / ``grad.mul_(1 / ratio)`` with ``ratio = 1 / world`` in double, i.e. ATen's
    multiply by ``float(ratio)`` rounded to the gradient's dtype - checked bit for bit against torch on the CPU."""
    gen = torch.Generator().manual_seed(11)
    shapes = [(257, 3), (1,), (4099,), (64, 65)]
    ps = _params(shapes, [dtype] * len(shapes))
    st = ParamStorage()
    ids, host = {}, []
    for i, p in enumerate(ps):
        st.register_param(id(p), p)
        ids[f"p{i}"] = id(p)
        if i == 1:
            host.append(None)          # no gradient: left alone
            continue
        g = (torch.randn(p.shape, generator=gen) * 3.0).to(dtype)
        host.append(g.clone())
        p.grad = g.to(p.device)
    st.deploy("g", ids)
    ratio = 1.0 / float(world)
    st.scale_grads("g", False, world_size=world)
    want = [None if g is None else g.clone().mul_(ratio) for g in host]
    for p, w in zip(ps, want):
        assert (p.grad is None) == (w is None)
        if w is not None:
            assert_bits_equal(p.grad.cpu(), w, "scaled")
    st.unscale_grads("g", False, world_size=world)
    for p, w in zip(ps, want):
        if w is not None:
            assert_bits_equal(p.grad.cpu(), w.clone().mul_(1.0 / ratio), "unscaled")


# ----------------------------------------------------------------------------- ZeRO views

def test_zero_locator_views_and_staging():
    ps = _params([(10, 3), (5,)], [torch.float16, torch.float32])
    st = ParamStorage()
    ids = {}
    for i, p in enumerate(ps):
        st.register_param(id(p), p)
        ids[f"p{i}"] = id(p)
    st.allreduce_amp_master_params = True
    st.deploy("g", ids, enable_zero=True, allreduce_amp_master_params=True)
    before = [p.detach().cpu().clone() for p in ps]
    st.align_buffer_zero("g")
    torch.cuda.synchronize()
    loc = st.zero_grad_locators["g"]
    for p, b in zip(ps, before):
        assert torch.equal(p.detach().cpu(), b)                       # values preserved
        buf = loc.get_buffer(id(p))
        assert_bits_equal(buf.cpu(), oracle.align_buffer(b, 1), "aligned buffer")
        assert p.data_ptr() == buf.data_ptr()                         # param re-homed into it
        lo, hi = st.get_local_param_range("g", id(p))
        assert (lo, hi) == (0, p.numel())
        seg = st.get_local_param_segment("g", id(p))
        assert seg.data_ptr() == p.data_ptr() and seg.numel() == p.numel() and seg.requires_grad
        assert loc.get_buffer_segment(id(p), 0).numel() == buf.numel()
    for p in ps:
        p.grad = torch.randn_like(p)
    grads = [p.grad.detach().cpu().clone() for p in ps]
    st.set_grad_to_local_param_segment("g")
    for p in ps:
        seg = st.get_local_param_segment("g", id(p))
        assert seg.grad.data_ptr() == p.grad.data_ptr()
    bufs = st.allreduce_param_grads_zero("g")
    torch.cuda.synchronize()
    assert bufs[0].dtype == torch.float32 and bufs[1].dtype == torch.float32    # half widened to fp32
    for b, g in zip(bufs, grads):
        assert_bits_equal(b.cpu(), oracle.zero_staging_pack(g, 1, True), "staging")
    for p, g in zip(ps, grads):
        assert torch.equal(p.grad.cpu(), g)                           # copy-back of a sum over one rank


@pytest.mark.parametrize("nranks", [1, 2, 8])
def test_grad_locator_layout_for_more_ranks(nranks):
    # layout arithmetic for larger groups (views only; the collectives are not part of this build)
    p = torch.nn.Parameter(torch.arange(100, dtype=torch.float16, device=DEV))
    for r in range(nranks):
        loc = DistributedGradLocator()
        loc.register_grad(1, p, nranks, r)
        lay = oracle.segment_layout(100, 2, nranks)
        assert loc.get_segment_range(1) == lay.range(r)
        seg = loc.get_local_param_segment(1)
        assert torch.equal(seg.detach().cpu(), torch.arange(100, dtype=torch.float16)[lay.range(r)[0]:lay.range(r)[1]])


# ----------------------------------------------------------------------------- dist params

@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_dist_param_store_set_load_roundtrip(dtype):
    g = torch.Generator().manual_seed(3)
    full = torch.randn(37, 5, generator=g).to(dtype)
    p = torch.nn.Parameter(full.clone().to(DEV))
    dp.store_dist_param(p)
    assert p.distributed and _pyrannc.dist_param_registered(id(p))
    rng = dp.get_dist_param_range(id(p))
    assert_bits_equal(dp.get_dist_param_segment(id(p)).detach().cpu(), full.flatten()[rng], "segment == full[range]")
    assert p.data.data_ptr() == dp.get_dist_param_segment(id(p)).data_ptr()
    loaded = dp.load_dist_param(id(p))
    assert loaded.device.type == "cpu" and loaded.shape == full.shape and loaded.requires_grad
    assert_bits_equal(loaded.detach(), full, "load")
    new = torch.randn(37, 5, generator=g).to(dtype)
    dp.set_dist_param(id(p), new.to(DEV))
    assert_bits_equal(dp.load_dist_param(id(p)).detach(), new, "set then load")
    dp.set_dist_param_dtype(id(p), torch.float32)
    assert dp.get_dist_param_segment(id(p)).dtype == torch.float32
    assert_bits_equal(dp.load_dist_param(id(p)).detach(), new.float(), "cast then load")
    dp.remove_dist_param(id(p))
    assert not _pyrannc.dist_param_registered(id(p))
    with pytest.raises(ValueError, match="not registered"):
        dp.load_dist_param(id(p))


def test_distribute_model_params_context():
    with rannc_amd.DistributeModelParams():
        torch.manual_seed(0)
        lin = torch.nn.Linear(8, 4)
        want_w, want_b = None, None
    # built on the host inside the context: every direct parameter became a GPU segment
    assert getattr(lin, "_dist_params", False)
    assert "_old_init" not in vars(torch.nn.Linear)
    for p in lin.parameters():
        assert p.is_cuda and p.dim() == 1 and _pyrannc.dist_param_registered(id(p))
        full = dp.load_dist_param(id(p))
        assert full.numel() == p.numel()
        assert_bits_equal(p.detach().cpu(), full.flatten().detach(), "segment == full[range]")
    y = lin(torch.randn(3, 8, device=DEV))          # hooks swap the full tensors in and out
    assert y.shape == (3, 4)
    for p in lin.parameters():
        assert p.dim() == 1


# ----------------------------------------------------------------------------- amp end to end

def _tiny_model(seed=0):
    torch.manual_seed(seed)
    return torch.nn.Sequential(torch.nn.Linear(32, 48), torch.nn.Tanh(), torch.nn.Linear(48, 8)).to(DEV)


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("half", [torch.float16, torch.bfloat16])
def test_amp_step_matches_oracle_sequence(fused, half):
    model = _tiny_model()
    opt = torch.optim.SGD(model.parameters(), lr=0.1)
    model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8, half_dtype=half, fused=fused)
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    scaler = amp._amp_state.loss_scalers[0]
    assert scaler.loss_scale() == 256.0
    x = torch.randn(16, 32, device=DEV, dtype=half)
    loss = rm(x).float().pow(2).mean()
    with amp.scale_loss(loss, opt) as scaled:
        scaled.backward()
        model_grads = [p.grad.detach().cpu().clone() for p in opt._amp_stash.all_fp16_params]
    # oracle: unscale + flag, then clip on the master grads, in the stash order
    want_unscaled, flag = oracle.unscale_and_check(model_grads, 1.0 / 256.0)
    assert flag == 0
    masters = opt._amp_stash.all_fp32_from_fp16_params
    max_norm = 1e-3
    rm.clip_grad_norm(max_norm)
    ref = [w.clone() for w in want_unscaled]
    norm, coef = oracle.clip_grad_norm(ref, max_norm)
    assert coef is not None
    res = opt._amp_stash.last_result
    assert math.isclose(res.norm, norm, rel_tol=1e-6)
    for m, w in zip(masters, want_unscaled):
        got = m.grad.cpu()
        ratio = got.double().abs().sum() / w.double().abs().sum()
        assert math.isclose(float(ratio), coef, rel_tol=1e-5)
    masters_before = [m.detach().cpu().clone() for m in masters]
    grads_now = [m.grad.detach().cpu().clone() for m in masters]
    opt.step()
    for m, b, g, p in zip(masters, masters_before, grads_now, opt._amp_stash.all_fp16_params):
        # torch's own SGD kernel (not part of this path) fuses the update into one fma
        assert torch.allclose(m.detach().cpu(), b - 0.1 * g, rtol=1e-6, atol=1e-9), "sgd on masters"
        assert_bits_equal(p.detach().cpu(), oracle.cast(m.detach().cpu(), half), "master -> model copy-back")
    rm.zero_grad()


@pytest.mark.parametrize("fused,fused_opt", [(False, False), (True, False), (True, True)])
def test_amp_gradient_accumulation_adds_into_live_master_grads(fused, fused_opt):
    from rannc_amd.fused_optim import FusedSGD
    model = _tiny_model()
    opt = (FusedSGD if fused_opt else torch.optim.SGD)(model.parameters(), lr=0.1)
    model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8, fused=fused)
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    xs = [torch.randn(16, 32, device=DEV, dtype=torch.float16) for _ in range(3)]
    want = None
    for x in xs:                                             # three micro-batches, no zero_grad between
        loss = rm(x).float().pow(2).mean()
        with amp.scale_loss(loss, opt) as scaled:
            scaled.backward()
            grads = [p.grad.detach().cpu().clone() for p in opt._amp_stash.all_fp16_params]
        if want is None:
            want, _ = oracle.unscale_and_check(grads, 1.0 / 256.0)
        else:
            oracle.unscale_accumulate(want, grads, 1.0 / 256.0)
    for m, w in zip(opt._amp_stash.all_fp32_from_fp16_params, want):
        assert_bits_equal(m.grad.cpu(), w, "accumulated master grad")
    opt.step()
    opt.zero_grad()
    assert all(m.grad is None or bool((m.grad == 0).all()) for m in opt._amp_stash.all_fp32_from_fp16_params)


def test_amp_overflow_skips_the_step_and_halves_the_scale():
    model = _tiny_model()
    opt = torch.optim.SGD(model.parameters(), lr=0.1)
    model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8, min_loss_scale=1.0)
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    rm._setup_amp_params() if rm.ready else None
    x = torch.randn(16, 32, device=DEV, dtype=torch.float16)
    loss = rm(x).float().pow(2).mean()
    rm.clip_grad_norm(1.0) if False else None
    rm._deploy() if not rm.ready else None
    rm._setup_amp_params()                      # patches update_scale as the reference does
    before = [m.detach().clone() for m in opt._amp_stash.all_fp32_from_fp16_params]
    with amp.scale_loss(loss, opt) as scaled:
        scaled.backward()
        opt._amp_stash.all_fp16_params[0].grad.view(-1)[3] = float("inf")
    scaler = amp._amp_state.loss_scalers[0]
    assert scaler.loss_scale() == 128 and scaler._unskipped == 0
    opt.step()                                  # skipped once
    for m, b in zip(opt._amp_stash.all_fp32_from_fp16_params, before):
        assert torch.equal(m.detach(), b)
    want = oracle.LossScalerState(loss_scale=256.0, max_loss_scale=256.0)
    assert oracle.patched_update_scale(want, True) is True and want.loss_scale == scaler.loss_scale()


@pytest.mark.parametrize("fused", [False, True])
def test_amp_keeps_one_device_table_across_steps(fused):
    """The unscale table is created once: later steps re-point it (or find the gradients where they were)
    instead of destroying and rebuilding it, and the model gradients are let go once their last reader is queued."""
    model = _tiny_model()
    opt = torch.optim.SGD(model.parameters(), lr=0.01)
    model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8, fused=fused)
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    handles = set()
    for step in range(5):
        x = torch.randn(16, 32, device=DEV, dtype=torch.float16)
        loss = rm(x).float().pow(2).mean()
        with amp.scale_loss(loss, opt) as scaled:
            scaled.backward()
            if step == 2:       # make backward's next allocation land elsewhere: the table must follow, not be rebuilt
                hold = [torch.empty_like(p.grad) for p in opt._amp_stash.all_fp16_params]
        stash = opt._amp_stash
        plan = stash.unscale_plan                  # a table of the compiled module, or a TensorPlan over ctypes
        handles.add(plan.gp.handle if hasattr(plan, "gp") else plan.plan._handle.value)
        rm.clip_grad_norm(1.0)
        opt.step()
        held = plan.gp.held() if hasattr(plan, "gp") else sum(s is not None for s in plan._srcs)
        assert held == 0 and stash.pending_model_grads == []
        opt.zero_grad()
    assert len(handles) == 1
    del hold


@pytest.mark.parametrize("fused,fused_opt", [(False, False), (True, False), (True, True)])
def test_amp_static_scale_overflow_reaches_the_parameters(fused, fused_opt):
    """A static loss scale never skips a step (Apex): an overflow must not leave the previous step's master
    gradients in place.  The inf lands in the master gradients, clipGradNorm's arithmetic turns it into NaN
    (inf * (max / inf) = inf * 0), and the optimizer steps on that - in every mode."""
    from rannc_amd.fused_optim import FusedSGD
    model = _tiny_model()
    opt = (FusedSGD if fused_opt else torch.optim.SGD)(model.parameters(), lr=0.1)
    model, opt = amp.initialize(model, opt, opt_level="O2", loss_scale=128.0, fused=fused)
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    x = torch.randn(16, 32, device=DEV, dtype=torch.float16)
    for step in range(2):
        loss = rm(x).float().pow(2).mean()
        with amp.scale_loss(loss, opt) as scaled:
            scaled.backward()
            if step == 1:
                opt._amp_stash.all_fp16_params[0].grad.view(-1)[3] = float("inf")
        scaler = amp._amp_state.loss_scalers[0]
        assert scaler.loss_scale() == 128.0
        rm.clip_grad_norm(1e-3)
        opt.step()
        masters = opt._amp_stash.all_fp32_from_fp16_params
        if step == 0:
            assert all(bool(torch.isfinite(m).all()) for m in masters)
        else:
            assert opt._amp_stash.last_result.overflow == 1
            assert not bool(torch.isfinite(masters[0]).all()), "the overflow was swallowed"
            assert bool(torch.isnan(masters[0].view(-1)[3]))
        opt.zero_grad()


def test_patch_optimizer_zero_mode_bookkeeping():
    model = _tiny_model()
    opt = torch.optim.Adam(model.parameters(), lr=1e-3)
    model, opt = amp.initialize(model, opt, opt_level="O2")
    n_params = len(list(model.parameters()))
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True, enable_zero=True)
    x = torch.randn(4, 32, device=DEV, dtype=torch.float16)
    rm(x)
    assert len(opt.order_local_to_global) == n_params and len(opt.global_order_to_id) == n_params
    assert all(isinstance(v, slice) for v in opt.param_zero_range.values())
    sd = opt.state_dict(from_global=True)
    assert sorted(sd.keys()) == ["param_groups", "state"]
    with pytest.raises(ValueError, match="enable_apex_amp"):
        rannc_amd.RaNNCModule(model, opt, enable_zero=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_clone_grad_summer_matches_the_reference_loop(dtype):
    from rannc_amd.shared_params import CloneGradSummer
    g = torch.Generator().manual_seed(31)
    shapes = [(1000,), (33, 7), (70001,), (5,)]
    n_clones = [2, 3, 0, 1]
    params = [torch.zeros(s, dtype=dtype, device=DEV, requires_grad=True) for s in shapes]
    clones = [[torch.zeros(s, dtype=dtype, device=DEV, requires_grad=True) for _ in range(k)] for s, k in zip(shapes, n_clones)]
    summer = CloneGradSummer(params, clones)
    for step in range(2):                    # second round: parameter gradients exist and are added to
        cpu_clone_grads = []
        for i, cl in enumerate(clones):
            row = []
            for k, c in enumerate(cl):
                if (i, k) == (1, 1) and step == 0:
                    c.grad = None            # a clone that received no gradient
                    row.append(None)
                else:
                    val = (torch.randn(shapes[i], generator=g) * 300).to(dtype)
                    c.grad = val.to(DEV)
                    row.append(val.clone())
            cpu_clone_grads.append(row)
        cpu_param_grads = [None if p.grad is None else p.grad.cpu().clone() for p in params]
        summer.sum_into_params()
        oracle.sum_clone_grads(cpu_param_grads, cpu_clone_grads)
        for i, p in enumerate(params):
            if n_clones[i] == 0:
                assert p.grad is None
                continue
            assert_bits_equal(p.grad.cpu(), cpu_param_grads[i], f"param {i} step {step}")
            for c in clones[i]:
                assert c.grad is None or bool((c.grad == 0).all())
    with pytest.raises(ValueError):
        CloneGradSummer([params[0]], [[params[1]]])


def test_state_dict_returns_masters_under_every_shared_name_and_load_redeploys():
    class Tied(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = torch.nn.Embedding(20, 16)
            self.proj = torch.nn.Linear(16, 20, bias=False)
            self.proj.weight = self.emb.weight                 # shared parameter, two names
            self.register_buffer("steps", torch.zeros(1))

        def forward(self, idx):
            return self.proj(self.emb(idx))

    torch.manual_seed(9)
    model = Tied().to(DEV)
    opt = torch.optim.SGD(model.parameters(), lr=0.1)
    model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8)
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    before = rm.state_dict()
    assert "steps" in before                                    # not deployed yet: the model's own state_dict
    idx = torch.randint(0, 20, (8,), device=DEV)
    loss = rm(idx).float().pow(2).mean()
    with amp.scale_loss(loss, opt) as scaled:
        scaled.backward()
    rm.clip_grad_norm(1.0)
    opt.step()
    sd = rm.state_dict()
    assert set(sd.keys()) == {"emb.weight", "proj.weight"}      # parameters only, every alias
    assert sd["emb.weight"] is sd["proj.weight"] and sd["emb.weight"].dtype == torch.float32
    master = opt._amp_stash.all_fp32_from_fp16_params[0]
    assert sd["emb.weight"].data_ptr() == master.data_ptr()
    half = rm.state_dict(amp_master_params=False)
    assert half["emb.weight"].dtype == torch.float16
    assert_bits_equal(half["emb.weight"].cpu(), oracle.cast(master.detach().cpu(), torch.float16), "model copy of the master")
    # loading undeploys; the next call deploys again with the loaded values
    new_vals = {k: torch.full_like(v, 0.5) for k, v in model.state_dict().items()}
    rm.load_state_dict(new_vals)
    assert not rm.ready
    rm(idx)
    assert rm.ready and float(rm.get_param("emb.weight").detach().float().mean()) == 0.5


def test_amp_accumulates_fp32_parameter_gradients_too():
    # batch norm stays fp32 under O2: its gradients live on the model parameter and must
    # accumulate as  grad = grad + new_scaled_grad * inv_scale  over scale_loss contexts
    torch.manual_seed(4)
    model = torch.nn.Sequential(torch.nn.Linear(16, 24), torch.nn.BatchNorm1d(24), torch.nn.Linear(24, 4)).to(DEV)
    opt = torch.optim.SGD(model.parameters(), lr=0.1)
    model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8)
    assert model[1].weight.dtype == torch.float32 and model[0].weight.dtype == torch.float16
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    want_w = None
    for it in range(3):
        x = torch.randn(32, 16, device=DEV, dtype=torch.float16)
        loss = rm(x).float().pow(2).mean()
        with amp.scale_loss(loss, opt) as scaled:
            scaled.backward()
            scaled_grad = model[1].weight.grad.detach().cpu().clone()    # what this backward produced, still scaled
        if want_w is None:
            want_w, _ = oracle.unscale_and_check([scaled_grad], 1.0 / 256.0)
        else:
            oracle.unscale_accumulate(want_w, [scaled_grad], 1.0 / 256.0)
        assert_bits_equal(model[1].weight.grad.cpu(), want_w[0], f"bn weight grad after {it + 1} micro-batches")
    opt.step()


@pytest.mark.parametrize("fused,fused_opt", [(False, False), (True, False), (True, True)])
def test_zero_mode_trains_exactly_like_the_plain_mode(fused, fused_opt):
    """The reference's own invariant for ZeRO (test/common.py compares the partitioned run with the
    plain one): with one process the segments are the whole parameters, so three training steps with
    ``enable_zero`` must leave bit-identical masters and model parameters."""
    import copy
    from rannc_amd.fused_optim import FusedAdam
    torch.manual_seed(21)
    base = torch.nn.Sequential(torch.nn.Linear(32, 50), torch.nn.Tanh(), torch.nn.Linear(50, 9)).to(DEV)   # odd sizes: padded segments
    g = torch.Generator().manual_seed(22)
    xs = [torch.randn(16, 32, generator=g).to(DEV).half() for _ in range(3)]
    finals = {}
    for zero in (False, True):
        _pyrannc.clear()
        model = copy.deepcopy(base)
        opt = FusedAdam(model.parameters(), lr=1e-2) if fused_opt else torch.optim.SGD(model.parameters(), lr=0.1, momentum=0.9)
        model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8, fused=fused)
        rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True, enable_zero=zero)
        for x in xs:
            loss = rm(x).float().pow(2).mean()
            with amp.scale_loss(loss, opt) as scaled:
                scaled.backward()
            rm.clip_grad_norm(0.05)
            opt.step()
            opt.zero_grad()
        finals[zero] = ([p.detach().cpu().clone().flatten() for p in model.parameters()],
                        [m.detach().cpu().clone().flatten() for m in opt._amp_stash.all_fp32_from_fp16_params])
        assert not torch.equal(finals[zero][0][0], base[0].weight.detach().cpu().half().flatten()), "the step did nothing"
    for k in (0, 1):
        for a, b in zip(finals[False][k], finals[True][k]):
            assert_bits_equal(b[:a.numel()], a, "zero vs plain")


def test_sync_param_and_sync_orig_params():
    """``sync_param`` / ``sync_param_grad`` (``src/main.cpp:357-366`` -> ``ParamStorage::doSyncParam``) hand back host
    copies of the parameter and of its gradient (zeros when there is none, ``None`` for an unknown id), and
    ``_sync_orig_params`` (``pyrannc/__init__.py:539-573``) writes them into the user's module - with one rank: what it
    already holds, plus a zero gradient for parameters without one."""
    _pyrannc.clear()
    torch.manual_seed(31)
    model = torch.nn.Sequential(torch.nn.Linear(7, 5), torch.nn.Linear(5, 3)).to(DEV)
    rm = rannc_amd.RaNNCModule(model, None)
    rm(torch.randn(4, 7, device=DEV)).pow(2).mean().backward()
    model[1].bias.grad = None
    before = {n: (p.detach().cpu().clone(), None if p.grad is None else p.grad.detach().cpu().clone().view(p.shape))
              for n, p in model.named_parameters()}
    for n, p in model.named_parameters():
        pid = rm.name_to_pid[n]
        got = rm.sync_param(pid)
        assert got.device.type == "cpu" and got.data_ptr() != p.data_ptr()
        assert_bits_equal(got.view(p.shape), before[n][0], n)
        gg = rm.sync_param_grad(pid)
        want = before[n][1] if before[n][1] is not None else torch.zeros_like(before[n][0])
        assert_bits_equal(gg.view(p.shape), want, n + ".grad")
    assert rm.sync_param(12345) is None and rm.sync_param_grad(12345) is None
    rm._sync_orig_params(sync_grad=True, name_pattern="1.")
    assert model[1].bias.grad is not None and bool((model[1].bias.grad == 0).all())
    rm._sync_orig_params(sync_grad=True)
    for n, p in model.named_parameters():
        assert_bits_equal(p.detach().cpu(), before[n][0], n)
        want = before[n][1] if before[n][1] is not None else torch.zeros_like(before[n][0])
        assert_bits_equal(p.grad.detach().cpu().view(p.shape), want, n + ".grad")


def test_scale_loss_restores_stashed_gradients_when_the_body_raises():
    torch.manual_seed(5)
    model = torch.nn.Sequential(torch.nn.Linear(8, 8), torch.nn.BatchNorm1d(8)).to(DEV)
    opt = torch.optim.SGD(model.parameters(), lr=0.1)
    model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8)
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    x = torch.randn(4, 8, device=DEV, dtype=torch.float16)
    with amp.scale_loss(rm(x).float().sum(), opt) as scaled:
        scaled.backward()
    kept = model[1].weight.grad.clone()
    with pytest.raises(RuntimeError, match="boom"):
        with amp.scale_loss(rm(x).float().sum(), opt) as scaled:
            raise RuntimeError("boom")
    assert torch.equal(model[1].weight.grad, kept)


def test_amp_fused_mode_picks_its_strategy_from_the_last_step():
    """Default (fused) amp: a step after one that clipped defers the write and applies the coefficient in it; a
    step after one that did not clip writes eagerly while summing and multiplies in place only if it clips after
    all.  Either way the master gradients are the oracle's: unscale, then clip by the norm."""
    model = _tiny_model()
    opt = torch.optim.SGD(model.parameters(), lr=0.0)
    model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8)
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    stash = opt._amp_stash
    assert stash.fused
    seen = []
    #            bound     deferred write expected at this step
    for bound, deferred in ((1e9, True), (1e9, False), (1e-3, False), (1e-3, True), (1e9, True), (1e-3, False)):
        x = torch.randn(16, 32, device=DEV, dtype=torch.float16)
        loss = rm(x).float().pow(2).mean()
        with amp.scale_loss(loss, opt) as scaled:
            scaled.backward()
            grads = [p.grad.detach().cpu().clone() for p in stash.all_fp16_params]
        assert stash.pending_finish == deferred
        seen.append(stash.pending_finish)
        rm.clip_grad_norm(bound)
        want, flag = oracle.unscale_and_check(grads, 1.0 / 256.0)
        norm, coef = oracle.clip_grad_norm(want, bound)
        assert flag == 0 and (coef is not None) == (bound == 1e-3)
        res = stash.unscale_plan.result()
        assert res.clipped == (1 if coef is not None else 0) and math.isclose(res.norm, norm, rel_tol=1e-6)
        unscaled, _ = oracle.unscale_and_check(grads, 1.0 / 256.0)
        for m, u in zip(stash.all_fp32_from_fp16_params, unscaled):
            assert_bits_equal(m.grad.cpu(), u * torch.tensor(res.coef) if res.clipped else u, "master gradient")
        opt.step()
        opt.zero_grad()
    assert seen == [True, False, False, True, True, False]


def test_amp_master_params_completes_a_deferred_write():
    model = _tiny_model()
    opt = torch.optim.SGD(model.parameters(), lr=0.1)
    model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8)
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    x = torch.randn(16, 32, device=DEV, dtype=torch.float16)
    loss = rm(x).float().pow(2).mean()
    with amp.scale_loss(loss, opt) as scaled:
        scaled.backward()
        grads = [p.grad.detach().cpu().clone() for p in opt._amp_stash.all_fp16_params]
    assert opt._amp_stash.pending_finish
    masters = list(amp.master_params(opt))          # the Apex recipe: clip_grad_norm_(amp.master_params(optimizer), ...)
    assert not opt._amp_stash.pending_finish
    want, _ = oracle.unscale_and_check(grads, 1.0 / 256.0)
    for m, w in zip(masters, want):
        assert_bits_equal(m.grad.cpu(), w, "master gradient handed out by master_params")


@pytest.mark.parametrize("reader", ["named_master_params", "zip_params"])
def test_amp_named_master_params_completes_a_deferred_write(reader):
    """The reference's own tests read the unscaled gradients as ``p.grad for n, p in named_master_params(...)``
    (``test/common.py:86``): right after ``scale_loss`` exits - on the first step and after a step that clipped,
    when the default fused mode has deferred the write - that must hand out what a ``fused=False`` run holds."""
    def run(fused):
        torch.manual_seed(11)
        model = _tiny_model()
        opt = torch.optim.SGD(model.parameters(), lr=0.0)
        model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8, fused=fused)
        rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
        gen = torch.Generator().manual_seed(3)
        seen = []
        for step in range(3):
            x = torch.randn(16, 32, generator=gen).to(DEV, torch.float16)
            loss = rm(x).float().pow(2).mean()
            with amp.scale_loss(loss, opt) as scaled:
                scaled.backward()
            if fused and step != 1:
                assert opt._amp_stash.pending_finish          # step 0, and step 2 (step 1 clipped): write deferred
            if reader == "named_master_params":
                grads = [p.grad.detach().cpu().clone() for _, p in amp.named_master_params(model, opt)]
            else:
                grads = [m.grad.detach().cpu().clone() for m, _ in amp.zip_params(opt)]
            assert not opt._amp_stash.pending_finish
            seen.append(grads)
            rm.clip_grad_norm(1e9 if step == 0 else 1e-3)     # steps 1 and 2 clip
            opt.step()
            opt.zero_grad()
        return seen
    got, want = run(True), run(False)
    for step, (gs, ws) in enumerate(zip(got, want)):
        assert len(gs) == len(ws) > 0
        for g, w in zip(gs, ws):
            assert_bits_equal(g, w, f"master gradient read through {reader} at step {step}")


def test_amp_with_the_loss_scale_schedule_on_the_device():
    """``amp.initialize(..., device_loss_scale=True)``: the same training loop with the schedule on the device and on
    the host - an injected overflow in step 2 (skipped, scale halved and truncated by ``patch_amp_scaler``'s rule),
    a window doubling - must walk the same parameters and the same scale sequence, and the device mode must not
    read anything back unless asked."""
    from rannc_amd.fused_optim import FusedAdam

    def run(on_device):
        torch.manual_seed(3)
        model = _tiny_model()
        opt = FusedAdam(model.parameters(), lr=1e-2)
        model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 7, min_loss_scale=None,
                                    device_loss_scale=on_device)
        scaler = amp._amp_state.loss_scalers[0]
        scaler._loss_scale, scaler._scale_seq_len = 100.0, 3
        if on_device:
            scaler.to_device(torch.device(DEV))           # rewrite the device state from the edited attributes
        rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
        gen = torch.Generator().manual_seed(4)
        scales = []
        for step in range(7):
            x = torch.randn(16, 32, generator=gen).to(DEV).to(torch.float16)
            loss = rm(x).float().pow(2).mean()
            with amp.scale_loss(loss, opt) as scaled:
                scaled.backward()
                if step == 2:
                    opt._amp_stash.all_fp16_params[1].grad.view(-1)[0] = float("inf")
            rm.clip_grad_norm(1.0)
            opt.step()
            opt.zero_grad()
            scales.append(scaler.loss_scale())
        masters = [m.detach().cpu().clone() for m in opt._amp_stash.all_fp32_from_fp16_params]
        steps = float(opt.state[opt._amp_stash.all_fp32_from_fp16_params[0]]["step"])
        return scales, masters, steps

    host_scales, host_masters, host_steps = run(False)
    dev_scales, dev_masters, dev_steps = run(True)
    # 100: clean, clean, inf -> int(50) = 50, then three clean steps -> 100, one more clean
    assert host_scales == [100.0, 100.0, 50.0, 50.0, 50.0, 100.0, 100.0]
    assert dev_scales == host_scales
    assert host_steps == dev_steps == 6.0
    for a, b in zip(dev_masters, host_masters):
        torch.testing.assert_close(a, b, rtol=2e-6, atol=1e-8)


@pytest.mark.parametrize("micro_batches", [2, 4])
@pytest.mark.parametrize("fused", [False, True])
def test_amp_gradient_accumulation_then_clip(micro_batches, fused):
    """Accumulation steps {2, 4} as the reference's tests run them (``test/test_simple.py:21-46``,
    ``test/common.py:98-103``), followed by ``clip_grad_norm``: the accumulated master gradients are the oracle's
    (bit for bit) and the clip multiplies them by the coefficient of their norm.  In fused mode the norm comes from
    the sums the accumulating pass left on the device - ``clip_grad_norm`` makes no pass over the gradients unless
    it clips - in eager mode from a pass of its own; both within 1e-6 of the oracle's."""
    model = _tiny_model()
    opt = torch.optim.SGD(model.parameters(), lr=0.1)
    model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8, fused=fused)
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    want = None
    for i in range(micro_batches):
        x = torch.randn(16, 32, device=DEV, dtype=torch.float16)
        loss = rm(x).float().pow(2).mean()
        with amp.scale_loss(loss, opt) as scaled:
            scaled.backward()
            grads = [p.grad.detach().cpu().clone() for p in opt._amp_stash.all_fp16_params]
        if want is None:
            want, _ = oracle.unscale_and_check(grads, 1.0 / 256.0)
        else:
            oracle.unscale_accumulate(want, grads, 1.0 / 256.0)
    stash = opt._amp_stash
    masters = stash.all_fp32_from_fp16_params
    for m, w in zip(masters, want):
        assert_bits_equal(m.grad.cpu(), w, "accumulated master grad")
    assert stash.sums_cover_all == fused                  # the accumulating pass's sums are kept for the clip
    norm = oracle.grad_global_l2_norm(want)
    max_norm = 0.5 * norm                                 # clips
    rm.clip_grad_norm(max_norm)
    if fused:
        assert stash.clip_decided and not stash.sums_cover_all        # took the decision from the sums
        res = stash.unscale_plan.result()
        assert res.clipped == 1 and math.isclose(res.norm, norm, rel_tol=1e-6)
        coef = res.coef
    else:
        coef = None
    clipped = [w.clone() for w in want]
    _, want_coef = oracle.clip_grad_norm(clipped, float(torch.tensor(max_norm, dtype=torch.float32)))
    assert want_coef is not None
    if coef is None:
        coef = float(torch.tensor(want_coef, dtype=torch.float32))
        for m, w in zip(masters, clipped):
            torch.testing.assert_close(m.grad.cpu(), w, rtol=2e-6, atol=0)
    else:
        assert math.isclose(coef, want_coef, rel_tol=1e-6)
        for m, w in zip(masters, want):
            assert_bits_equal(m.grad.cpu(), w * torch.tensor(coef, dtype=torch.float32), "clipped with the device's coefficient")
    opt.step()
    opt.zero_grad()
