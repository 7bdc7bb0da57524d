"""The pybind11 entry points (rannc_amd._ranncgrad) over the same C ABI: they take PyTorch-ROCm
tensors directly, give the same results as the ctypes path and translate errors the way the
reference's pybind module does (ValueError / RuntimeError)."""
import math

import pytest
import torch

from oracle import gradpath as oracle
from rannc_amd import _lib, _ranncgrad
from tests.helpers import assert_bits_equal


def test_layout_and_constants_match_the_c_abi():
    assert _ranncgrad.version() == _lib.lib.rg_version()
    assert (_ranncgrad.RG_F32, _ranncgrad.RG_F16, _ranncgrad.RG_BF16) == (_lib.RG_F32, _lib.RG_F16, _lib.RG_BF16)
    for numel, es, r in [(1000, 2, 8), (100, 2, 8), (7, 4, 3), (0, 4, 2)]:
        assert tuple(_ranncgrad.segment_layout(numel, es, r)) == _lib.segment_layout(numel, es, r)
        assert _ranncgrad.aligned_numel(numel, es, r) == oracle.calc_aligned_num_elems(numel, es, r)


def test_errors_are_python_exceptions():
    with pytest.raises(ValueError):
        _ranncgrad.aligned_numel(1, 3, 1)
    with pytest.raises(ValueError):
        _ranncgrad.segment_layout(10, 4, 0)
    with pytest.raises(ValueError, match="GPU"):
        _ranncgrad.Plan([torch.zeros(4)], [torch.zeros(4)])
    with pytest.raises(ValueError, match="GPU"):
        _ranncgrad.copy_cast(torch.zeros(4), torch.zeros(4))


@pytest.mark.gpu
def test_fused_step_through_pybind_matches_oracle_and_ctypes():
    from rannc_amd.multi_tensor import TensorPlan
    dev = "cuda:0"
    g = torch.Generator().manual_seed(5)
    cpu = [(torch.randn(s, generator=g) * 1e-2 * 65536).to(torch.bfloat16) for s in [(70001,), (33,), (4096,), (0,)]]
    srcs = [t.to(dev) for t in cpu]
    out_a = [torch.zeros(t.shape, device=dev) for t in cpu]
    out_b = [torch.zeros(t.shape, device=dev) for t in cpu]
    pa = _ranncgrad.Plan(srcs, out_a)
    pa.fused_step(2.0 ** -16, 0.25)
    ra = pa.result()
    pb = TensorPlan(srcs, out_b)
    pb.fused_step(2.0 ** -16, 0.25)
    rb = pb.result()
    assert (ra["norm"], ra["coef"], ra["overflow"], ra["clipped"]) == (rb.norm, rb.coef, rb.overflow, rb.clipped)
    assert pa.tensor_norms() == pb.tensor_norms() and pa.num_tensors == 4 and pa.total_numel == pb.plan.total_numel
    want = oracle.fused_step(cpu, ["f32"] * 4, 2.0 ** -16, 0.25)
    assert math.isclose(ra["norm"], want.norm, rel_tol=1e-6) and math.isclose(ra["coef"], want.coef, rel_tol=1e-6)
    for a, b in zip(out_a, out_b):
        assert_bits_equal(a.cpu(), b.cpu(), "pybind vs ctypes")
    # the other operations and the plan-free copy
    pa.unscale_pack(2.0 ** -16)
    un, _ = oracle.unscale_and_check(cpu, 2.0 ** -16)
    for a, w in zip(out_a, un):
        assert_bits_equal(a.cpu(), w, "unscale_pack")
    pa.zero()
    torch.cuda.synchronize()
    assert all(bool((a == 0).all()) for a in out_a)
    half = torch.zeros(70001, dtype=torch.float16, device=dev)
    _ranncgrad.copy_cast(half, srcs[0])
    assert_bits_equal(half.cpu(), cpu[0].to(torch.float16), "copy_cast")
    with pytest.raises(ValueError, match="contiguous"):
        _ranncgrad.Plan([torch.zeros(4, 4, device=dev).t()], [torch.zeros(4, 4, device=dev)])
    with pytest.raises(ValueError, match="dtype"):
        _ranncgrad.Plan([torch.zeros(4, dtype=torch.float64, device=dev)], None)
    pa.close()
    with pytest.raises(RuntimeError, match="closed"):
        pa.grad_norm()


@pytest.mark.gpu
def test_optimizer_table_through_pybind_matches_ctypes():
    from rannc_amd import _lib
    from rannc_amd.multi_tensor import stream_handle
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(6)
    shapes = [(70001,), (33,), (4096,)]
    p0 = [torch.randn(s, generator=g) for s in shapes]
    grads = [(torch.randn(s, generator=g) * 1e-2).to(dev) for s in shapes]
    sets = []
    for _ in range(2):
        sets.append(dict(p=[t.to(dev) for t in p0], m=[torch.zeros(s, device=dev) for s in shapes],
                         v=[torch.zeros(s, device=dev) for s in shapes],
                         c=[torch.zeros(s, device=dev, dtype=torch.bfloat16) for s in shapes]))
    a, b = sets
    oa = _ranncgrad.Optim(a["p"], grads, a["m"], a["v"], a["c"])
    ob = _lib.OptimTable(0, [t.data_ptr() for t in b["p"]], [t.data_ptr() for t in grads], [t.data_ptr() for t in b["m"]],
                         [t.data_ptr() for t in b["v"]], [t.data_ptr() for t in b["c"]], [t.numel() for t in p0],
                         [_lib.RG_F32] * 3, [_lib.RG_BF16] * 3)
    for step in (1, 2):
        oa.adam_step(1e-3, 0.9, 0.999, 1e-8, 0.01, step)
        ob.adam_step(1e-3, 0.9, 0.999, 1e-8, 0.01, step, stream=stream_handle(dev))
    oa.sgd_step(0.1)
    ob.sgd_step(0.1, stream=stream_handle(dev))
    # the clip decision of a plan, consumed on the device by both bindings
    pl = _ranncgrad.Plan(grads, [torch.zeros_like(t) for t in grads])
    pl.step_begin(1.0)
    pl.step_decide(1e-3)
    assert pl.result()["clipped"] == 1
    oa.sgd_step(0.1, gate=pl.result_device_ptr())
    ob.sgd_step(0.1, gate=pl.result_device_ptr(), stream=stream_handle(dev))
    # the step with its count on the device: one clock per binding, both continue from step 2
    clocks = []
    for _ in range(2):
        clock = torch.zeros(8, dtype=torch.float32, device=dev)
        clock.view(torch.int64)[0] = 2
        clocks.append(clock)
    oa.adam_step_clocked(clocks[0], 1e-3, 0.9, 0.999, 1e-8, 0.01)
    _lib.adam_clock_advance(clocks[1].data_ptr(), 1e-3, 0.9, 0.999, 0, 0, stream_handle(dev))
    ob.adam_step_clocked(clocks[1].data_ptr(), 1e-3, 0.9, 0.999, 1e-8, 0.01, stream=stream_handle(dev))
    torch.cuda.synchronize()
    assert int(clocks[0].view(torch.int64)[0]) == 3 and float(clocks[0][4]) == 3.0
    assert_bits_equal(clocks[0].cpu(), clocks[1].cpu(), "clock")
    for k in "pmvc":
        for x, y in zip(a[k], b[k]):
            assert_bits_equal(x.cpu(), y.cpu(), f"pybind vs ctypes {k}")
    assert not torch.equal(a["p"][0].cpu(), p0[0])
    with pytest.raises(ValueError, match="float32"):
        _ranncgrad.Optim([torch.zeros(4, device=dev, dtype=torch.float16)], [torch.zeros(4, device=dev)])
    with pytest.raises(ValueError, match="exp_avg"):
        _ranncgrad.Optim([torch.zeros(4, device=dev)], [torch.zeros(4, device=dev)]).adam_step(1e-3, 0.9, 0.999, 1e-8, 0.0, 1)
    oa.close()
    with pytest.raises(RuntimeError, match="closed"):
        oa.sgd_step(0.1)


def test_reference_entry_point_names_are_exported():
    """The free functions of the reference's extension on this path (src/main.cpp:55-59, 78-136, 191-245)."""
    for name in ("get_rank", "get_world_size", "barrier", "allreduce_tensor", "bcast_tensor", "all_gather",
                 "register_amp_master_param", "store_dist_param", "load_dist_param", "set_dist_param",
                 "get_dist_param_segment", "set_dist_param_dtype", "get_dist_param_range", "remove_dist_param",
                 "dist_param_registered"):
        assert callable(getattr(_ranncgrad, name)), name
    assert (_ranncgrad.get_rank(), _ranncgrad.get_world_size()) == (0, 1)
    assert _ranncgrad.dist_param_registered(12345) is False
    with pytest.raises(ValueError, match="not registered"):
        _ranncgrad.get_dist_param_range(12345)
    with pytest.raises(ValueError, match="root"):
        _ranncgrad.bcast_tensor(torch.zeros(1), 1)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_dist_param_functions_of_the_compiled_module_match_the_oracle(dtype):
    dev = "cuda:0"
    g = torch.Generator().manual_seed(9)
    full = torch.randn(129, 3, generator=g).to(dtype)
    p = torch.nn.Parameter(full.to(dev))
    ora = oracle.DistParamOracle(0, 1)
    want_part = ora.store(1, full)
    part = _ranncgrad.store_dist_param(p)
    pid = id(p)
    try:
        assert _ranncgrad.dist_param_registered(pid) and part.requires_grad
        assert_bits_equal(part.detach().cpu(), want_part, "stored segment")
        assert tuple(_ranncgrad.get_dist_param_range(pid)) == ora.get_range(1)
        lo, hi = _ranncgrad.get_dist_param_range(pid)
        assert_bits_equal(part.detach().cpu(), full.flatten()[lo:hi], "segment == full.flatten()[range]")   # test/common.py:57-63
        loaded = _ranncgrad.load_dist_param(pid)
        assert not loaded.is_cuda and loaded.shape == full.shape and loaded.requires_grad
        assert_bits_equal(loaded.detach(), oracle.DistParamOracle.load(1, [ora]), "loaded tensor")
        new = torch.randn(129, 3, generator=g).to(dtype)
        _ranncgrad.set_dist_param(pid, new.to(dev))
        ora.set(1, new)
        assert_bits_equal(_ranncgrad.get_dist_param_segment(pid).detach().cpu(), ora.parts[1], "set")
        _ranncgrad.set_dist_param_dtype(pid, torch.float32)
        ora.set_scalar_type(1, torch.float32)
        seg = _ranncgrad.get_dist_param_segment(pid)
        assert seg.dtype == torch.float32 and seg.requires_grad
        assert_bits_equal(seg.detach().cpu(), ora.parts[1], "cast segment")
        assert_bits_equal(_ranncgrad.load_dist_param(pid).detach(), new.float(), "loaded after cast")
    finally:
        _ranncgrad.remove_dist_param(pid)
    assert not _ranncgrad.dist_param_registered(pid)


# ----------------------------------------------------------------------------- the compiled RaNNCModule / ParamStorage

def _named_params(dtypes, seed, dev="cuda:0"):
    g = torch.Generator().manual_seed(seed)
    shapes = [(257, 33), (1,), (4099,), (64, 64), (7,)]
    return {f"layer.{i}.w": torch.nn.Parameter(torch.randn(s, generator=g).to(dt).to(dev))
            for i, (s, dt) in enumerate(zip(shapes, dtypes))}


def test_compiled_module_has_the_reference_methods():
    """The per-step methods of the reference's bound class (src/main.cpp:333-380)."""
    for name in ("clip_grad_norm", "calc_grad_norm", "zero_grad", "align_params", "get_local_param_range",
                 "get_local_param_segment", "use_amp_master_params", "allreduce_grads", "allreduce_grads_zero",
                 "sync_param_zero", "sync_param", "sync_param_grad", "undeploy"):
        assert callable(getattr(_ranncgrad.RaNNCModule, name)), name
    m = _ranncgrad.RaNNCModule(True, False, False, True, False)
    assert m.use_amp_master_params() is True
    with pytest.raises(RuntimeError, match="not initialised"):
        m.clip_grad_norm(1.0)
    with pytest.raises(ValueError, match="not found"):
        _ranncgrad.get_param_storage().get_param_tensor(123)
    with pytest.raises(ValueError, match="not found"):
        _ranncgrad.get_amp_master_param(123)


@pytest.mark.gpu
@pytest.mark.parametrize("dtypes", [[torch.float32] * 5, [torch.float16, torch.float32, torch.bfloat16, torch.float16, torch.float32]])
def test_compiled_module_norm_clip_and_zero_match_the_python_registry(dtypes):
    """calc_grad_norm / clip_grad_norm / zero_grad of the compiled class against the registry driven from Python
    over the ctypes binding (same kernels, so the same bits) and against the oracle; one parameter without a
    gradient; max_grad_norm crossing the binding as a C float."""
    from rannc_amd.param_storage import ParamStorage
    named = _named_params(dtypes, seed=31)
    twins = {n: torch.nn.Parameter(p.detach().clone()) for n, p in named.items()}
    g = torch.Generator().manual_seed(32)
    cpu_grads = {}
    for (n, p), q in zip(named.items(), twins.values()):
        if n.endswith(".1.w"):
            continue                                   # no gradient: left out of norm, clip and zero
        cpu_grads[n] = (torch.randn(p.shape, generator=g) * 0.3).to(p.dtype)
        p.grad = cpu_grads[n].to(p.device)
        q.grad = cpu_grads[n].to(q.device)
    _ranncgrad.reset_param_storage()
    mod = _ranncgrad.RaNNCModule(False, False, False, True, False)
    ids = mod.init(named, False)
    assert list(ids) == sorted(named) and all(ids[n] == id(p) for n, p in named.items())
    st = ParamStorage()
    for n, q in twins.items():
        st.register_param(id(q), q)
    st.deploy("g", {n: id(q) for n, q in twins.items()})
    try:
        want_norm = oracle.grad_global_l2_norm([cpu_grads[n] for n in sorted(cpu_grads)])
        norm = mod.calc_grad_norm()
        assert norm == st.calc_grad_global_l2_norm("g", False)
        assert math.isclose(norm, want_norm, rel_tol=1e-6)
        mod.clip_grad_norm(0.1)                        # 0.1 is not an fp32 number: narrowed at the binding
        st.clip_grad_norm("g", float(torch.tensor(0.1, dtype=torch.float32)), False)
        clipped = [g.clone() for g in (cpu_grads[n] for n in sorted(cpu_grads))]
        _, coef = oracle.clip_grad_norm(clipped, float(torch.tensor(0.1, dtype=torch.float32)))
        assert coef is not None
        for n, p in named.items():
            if n not in cpu_grads:
                assert p.grad is None
                continue
            assert_bits_equal(p.grad.cpu(), twins[n].grad.cpu(), f"compiled vs ctypes {n}")
        for got, want in zip((named[n].grad for n in sorted(cpu_grads)), clipped):
            assert torch.allclose(got.float().cpu(), want.float(), rtol=2e-3 if want.dtype != torch.float32 else 1e-6, atol=0)
        mod.zero_grad()
        torch.cuda.synchronize()
        assert all(p.grad is None or bool((p.grad == 0).all()) for p in named.values())
    finally:
        mod.undeploy()
        st.undeploy("g")
        _ranncgrad.reset_param_storage()


@pytest.mark.gpu
def test_compiled_module_does_not_keep_gradients_alive():
    """The tables keep raw addresses; the tensors behind them are released as soon as the launch is queued, so that
    ``zero_grad(set_to_none=True)`` gives the memory back before the next backward pass allocates new gradients."""
    named = {f"layer.{i}.w": torch.nn.Parameter(torch.randn(1 << 20, device="cuda:0")) for i in range(4)}
    _ranncgrad.reset_param_storage()
    mod = _ranncgrad.RaNNCModule(False, False, False, True, False)
    mod.init(named, False)
    try:
        import gc
        gc.collect()                      # what earlier tests left in reference cycles must not be freed in mid-test
        torch.cuda.synchronize()
        base = torch.cuda.memory_allocated()
        for call in (mod.calc_grad_norm, lambda: mod.clip_grad_norm(1.0), mod.zero_grad):
            for p in named.values():
                p.grad = torch.ones_like(p)
            assert torch.cuda.memory_allocated() >= base + 4 * (4 << 20)
            call()
            for p in named.values():
                p.grad = None
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated() <= base, call
    finally:
        mod.undeploy()
        _ranncgrad.reset_param_storage()


@pytest.mark.gpu
def test_compiled_module_zero_segments_and_amp_masters():
    """enable_zero: layouts, local segments and aligned buffers of the compiled class follow the oracle's closed
    forms at one rank; with amp masters registered the norm is taken over the masters' gradients."""
    dtypes = [torch.float16] * 5
    named = _named_params(dtypes, seed=33)
    before = {n: p.detach().cpu().clone() for n, p in named.items()}
    _ranncgrad.reset_param_storage()
    mod = _ranncgrad.RaNNCModule(True, False, True, True, False)
    ids = mod.init(named, False)
    try:
        mod.align_params()
        torch.cuda.synchronize()
        masters = {}
        for n, p in named.items():
            pid = ids[n]
            assert_bits_equal(p.detach().cpu(), before[n], "values survive the re-homing")
            aligned, seg, offs, srcs = _lib.segment_layout(p.numel(), p.element_size(), 1)
            assert tuple(mod.get_local_param_range(pid)) == (offs[0], offs[0] + srcs[0]) == (0, p.numel())
            buf = _ranncgrad.get_param_storage().get_buffer(mod.native_graph_id, pid)
            assert buf.numel() == aligned == oracle.calc_aligned_num_elems(p.numel(), 2, 1)
            assert bool((buf[p.numel():] == 0).all()) and buf.data_ptr() == p.data_ptr()
            seg_t = mod.get_local_param_segment(pid)
            assert seg_t.dim() == 1 and seg_t.data_ptr() == p.data_ptr() and seg_t.requires_grad
            assert mod.get_local_param_segment(pid) is seg_t or mod.get_local_param_segment(pid).data_ptr() == seg_t.data_ptr()
            masters[n] = seg_t.detach().clone().float().requires_grad_(True)
            _ranncgrad.register_amp_master_param(pid, masters[n])
        g = torch.Generator().manual_seed(34)
        cpu = {n: torch.randn(m.shape, generator=g) * 0.01 for n, m in masters.items()}
        for n, m in masters.items():
            m.grad = cpu[n].to(m.device)
        want = oracle.grad_global_l2_norm([cpu[n] for n in sorted(cpu)])
        assert math.isclose(mod.calc_grad_norm(), want, rel_tol=1e-6)
        with pytest.raises(ValueError, match="not registered"):
            mod.get_local_param_range(12345)
    finally:
        mod.undeploy()
        _ranncgrad.reset_param_storage()
