"""Host-side logic that needs no GPU: workload definitions, the loss-scale schedule, optimizer
patching bookkeeping, registry error behaviour, argument checks that fire before any launch."""
import types

import pytest
import torch

from oracle import gradpath as oracle
from rannc_amd import _pyrannc, amp, opt, workloads
from rannc_amd.multi_tensor import TensorPlan, copy_cast_, dtype_code
from rannc_amd.param_storage import ParamStorage


def test_workload_definitions_match_the_configs():
    c1, c2, c3, c4 = (workloads.step_config(k) for k in ("c1_mlp", "c2_bert_large", "c3_bert_enlarged", "c4_resnet152x2"))
    assert (len(c1.params), c1.total_numel) == (8, 4 * (1024 * 1024 + 1024))
    assert len(c2.params) == 391 and abs(c2.total_numel - 3.35e8) < 1e6
    assert len(c3.params) == 775 and abs(c3.total_numel - 2.48e9) < 1e7
    assert len(c4.params) == 934 and abs(c4.total_numel - 2.3e8) < 1e7
    bn = [workloads.numel(s) for _, s in c4.params if len(s) == 1 and "fc" not in _]
    assert min(bn) == 64 and max(bn) == 2048
    for c in (c1, c2, c3, c4):
        names = [n for n, _ in c.params]
        assert names == sorted(names)                      # deployed in name order (ParamStorage.cpp:23-31)
    sizes = workloads.zero_segment_sizes()
    assert len(sizes) == 4096 and all(s % 2 == 1 for s in sizes) and abs(sum(sizes) - 1e10) < 1e5
    assert sizes == workloads.zero_segment_sizes()         # seeded


def test_make_grads_is_seeded_and_injects():
    cfg = workloads.step_config("c3_bert_enlarged_overflow")
    a, inj_a = workloads.make_grads(cfg, seed=3, scale_numel=0.0005)
    b, inj_b = workloads.make_grads(cfg, seed=3, scale_numel=0.0005)
    assert inj_a == inj_b and len(inj_a) >= 2
    assert all(torch.equal(x.view(torch.int16), y.view(torch.int16)) for x, y in zip(a, b))
    for j, (ti, fi) in enumerate(inj_a[:2]):
        v = a[ti].view(-1)[fi]
        assert torch.isinf(v) if j % 2 == 0 else torch.isnan(v)
    assert a[0].dtype == torch.float16


def test_loss_scaler_schedule_literal_sequence():
    """The product's scaler against hand-written literals (Apex's published schedule) and, step by
    step, against the oracle's restatement of it."""
    ours = amp.LossScaler("dynamic", min_loss_scale=1.0, max_loss_scale=2.0 ** 10, scale_window=3)
    ours._loss_scale = 2.0 ** 8
    want = oracle.LossScalerState(loss_scale=2.0 ** 8, scale_window=3, min_loss_scale=1.0, max_loss_scale=2.0 ** 10)
    seq = [False, False, True, False, False, False, True, True, False, False, False, False, False, False, False]
    scales = [256, 256, 128, 128, 128, 256, 128, 64, 64, 64, 128, 128, 128, 256, 256]
    counts = [1, 2, 0, 1, 2, 0, 0, 0, 1, 2, 0, 1, 2, 0, 1]
    for had, scale, count in zip(seq, scales, counts):
        ours._has_overflow = had
        assert ours.update_scale() == had == want.update_scale(had)
        ours.clear_overflow_state()
        assert (ours.loss_scale(), ours._unskipped) == (scale, count) == (want.loss_scale, want.unskipped)
    static = amp.LossScaler(128.0)
    static._has_overflow = True
    assert static.update_scale() is False and static.loss_scale() == 128.0


def _fake_model(params, enable_zero=False, enable_apex_amp=False):
    m = types.SimpleNamespace()
    m.used_param_ids = {id(p) for p in params}
    m.enable_zero, m.enable_apex_amp, m.offload_params = enable_zero, enable_apex_amp, False
    m.use_amp_master_params = lambda: enable_apex_amp
    m.device = torch.device("cpu")
    return m


def test_patch_optimizer_orders_and_state_dict_roundtrip():
    ps = [torch.nn.Parameter(torch.randn(3, 2)), torch.nn.Parameter(torch.randn(5)), torch.nn.Parameter(torch.randn(4))]
    unused = torch.nn.Parameter(torch.randn(2))
    o = torch.optim.Adam([{"params": [ps[0], unused]}, {"params": [ps[1], ps[2]], "lr": 0.5}], lr=0.1)
    model = _fake_model(ps)
    opt.patch_optimizer(model, o)
    # the unused parameter is dropped locally but keeps its global order (pyrannc/opt.py:222-249)
    assert [len(g["params"]) for g in o.param_groups] == [1, 2]
    assert o.order_local_to_global == {0: 0, 1: 2, 2: 3}
    assert o.global_order_to_id == {0: id(ps[0]), 1: id(unused), 2: id(ps[1]), 3: id(ps[2])}
    assert o.original_param_groups[0]["params"] == [0, 1] and o.original_param_groups[1]["params"] == [2, 3]
    for p in ps:
        p.grad = torch.ones_like(p)
    o.step()
    g = o.state_dict(from_global=True)
    assert sorted(g["state"].keys()) == [0, 2, 3] and g["param_groups"] == o.original_param_groups
    local = o.state_dict()
    assert sorted(local["state"].keys()) == [0, 1, 2]
    # load it back through the global numbering
    o2 = torch.optim.Adam([{"params": [ps[0], unused]}, {"params": [ps[1], ps[2]], "lr": 0.5}], lr=0.1)
    opt.patch_optimizer(model, o2)
    o2.load_state_dict(g, from_global=True)
    for k in (0, 1, 2):
        assert torch.equal(o2.state_dict()["state"][k]["exp_avg"], local["state"][k]["exp_avg"])


def test_slice_optimizer_state_uses_the_zero_range():
    sd = {"state": {0: {"exp_avg": torch.arange(12.0).view(3, 4), "step": 3}}, "param_groups": []}
    out = opt._slice_optimizer_state(sd, {77: slice(2, 7)}, {0: 77})
    assert out["state"][0]["exp_avg"].tolist() == [2.0, 3.0, 4.0, 5.0, 6.0] and out["state"][0]["step"] == 3


def test_registry_errors_are_value_errors():
    st = ParamStorage()
    with pytest.raises(ValueError, match="not found"):
        st.get_param_tensor(1)
    with pytest.raises(ValueError, match="master"):
        st.get_amp_master_param_tensor(1)
    with pytest.raises(ValueError, match="not registered"):
        _pyrannc.get_dist_param_range(123456)
    with pytest.raises(ValueError, match="not registered"):
        _pyrannc.load_dist_param(123456)
    assert _pyrannc.dist_param_registered(123456) is False
    assert (_pyrannc.get_rank(), _pyrannc.get_world_size()) == (0, 1)
    with pytest.raises(ValueError):
        _pyrannc.bcast_tensor(torch.zeros(1), 3)
    m = _pyrannc.RaNNCModule()
    with pytest.raises(RuntimeError, match="not initialised"):
        m.clip_grad_norm(1.0)


def test_argument_checks_fire_before_any_launch():
    with pytest.raises(ValueError, match="dtype"):
        dtype_code(torch.float64)
    with pytest.raises(ValueError, match="GPU"):
        TensorPlan([torch.zeros(4)], [torch.zeros(4)])
    with pytest.raises(ValueError, match="GPU"):
        copy_cast_(torch.zeros(4), torch.zeros(4))
    with pytest.raises(ValueError, match="neither"):
        TensorPlan([None], [None], device=torch.device("cuda", 0))


def test_module_requires_amp_for_zero():
    import rannc_amd
    with pytest.raises(ValueError, match="enable_apex_amp"):
        rannc_amd.RaNNCModule(torch.nn.Linear(2, 2), enable_zero=True)


def test_module_passes_the_wrapped_models_interface_through():
    """What ``pyrannc.RaNNCModule`` offers besides the step calls (``pyrannc/__init__.py:312-372, 510-537``): ``to`` /
    ``cuda`` are ignored, unknown attributes come from the wrapped module, parameter and buffer iterators, ``train`` /
    ``eval`` / ``enable_dropout`` reach the module.  None of it needs a GPU before the first forward call."""
    import rannc_amd

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = torch.nn.Linear(3, 2)
            self.drop = torch.nn.Dropout(0.5)
            self.register_buffer("steps", torch.zeros(1))
            self.marker = "hello"

        def forward(self, x):
            return self.drop(self.lin(x))

        def describe(self, k):
            return f"net-{k}"

    net = Net()
    rm = rannc_amd.RaNNCModule(net, None)
    assert rm.to("cpu") is rm and rm.cuda() is rm                      # ignored, as in the reference
    assert rm.marker == "hello" and rm.describe(3) == "net-3"
    with pytest.raises(AttributeError, match="no attribute"):
        rm.no_such_thing
    assert [n for n, _ in rm.named_parameters()] == ["lin.weight", "lin.bias"]
    assert len(list(rm.parameters())) == 2
    assert [n for n, _ in rm.named_buffers()] == ["steps"] and len(list(rm.buffers())) == 1
    assert rm.eval() is rm and not net.training and not net.drop.training
    rm.enable_dropout(True)
    assert net.drop.training and not net.lin.training                  # only the dropout layers change
    assert rm.train() is rm and net.training
    # once deployed the iterators keep to the parameters this process works on (all of them with one rank)
    rm.ready, rm.used_param_ids = True, {id(net.lin.weight)}
    assert [n for n, _ in rm.named_parameters()] == ["lin.weight"]
    assert [n for n, _ in rm.named_parameters(from_global=True)] == ["lin.weight", "lin.bias"]
    assert len(list(rm.parameters())) == 1
    rm.ready = False
