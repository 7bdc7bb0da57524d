"""Checkpoint round trips through ``torch.save`` / ``torch.load``, as the reference's own test drives them
(``test/common.py:256-310``): ``RaNNCModule.state_dict()`` into a fresh module, and the optimizer's
``state_dict(from_global=True)`` back through ``load_state_dict(..., from_global=True)`` - under ZeRO every state
tensor cut to the parameter's local range (``pyrannc/opt.py:186-202``) and moved to the device."""
import copy

import pytest
import torch

import rannc_amd
from rannc_amd import _pyrannc, amp
from rannc_amd.fused_optim import FusedAdam
from tests.helpers import assert_bits_equal

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _base(seed=31):
    torch.manual_seed(seed)
    return torch.nn.Sequential(torch.nn.Linear(24, 37), torch.nn.Tanh(), torch.nn.Linear(37, 5)).to(DEV)   # odd sizes


def _inputs(n, dtype, seed=32):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(8, 24, generator=g).to(DEV).to(dtype) for _ in range(n)]


def _train(rm, opt, xs, use_amp):
    for x in xs:
        loss = rm(x).float().pow(2).mean()
        if use_amp:
            with amp.scale_loss(loss, opt) as scaled:
                scaled.backward()
        else:
            loss.backward()
        rm.clip_grad_norm(0.05)
        opt.step()
        opt.zero_grad()


@pytest.mark.parametrize("opt_cls", [FusedAdam, torch.optim.Adam])
def test_fp32_checkpoint_resumes_with_identical_steps(tmp_path, opt_cls):
    """No amp: save after three steps, rebuild everything from the files, and the next two steps of the resumed
    run are bit-identical to those of the run that never stopped."""
    _pyrannc.clear()
    xs = _inputs(5, torch.float32)
    model = _base()
    opt = opt_cls(model.parameters(), lr=1e-2)
    rm = rannc_amd.RaNNCModule(model, opt)
    _train(rm, opt, xs[:3], False)
    torch.save(rm.state_dict(), tmp_path / "model.pt")
    torch.save(opt.state_dict(from_global=True), tmp_path / "opt_state.pt")
    _train(rm, opt, xs[3:], False)
    want = [p.detach().cpu().clone() for p in model.parameters()]

    _pyrannc.clear()
    ld_model = _base(seed=99)                                   # different initial values: everything must come from the files
    ld_model.load_state_dict(torch.load(tmp_path / "model.pt", map_location="cpu"))
    ld_opt = opt_cls(ld_model.parameters(), lr=1e-2)
    ld_rm = rannc_amd.RaNNCModule(ld_model, ld_opt)
    ld_rm._deploy()
    global_sd = torch.load(tmp_path / "opt_state.pt")
    assert sorted(global_sd["state"].keys()) == [0, 1, 2, 3]
    assert all(not v.is_cuda for st in global_sd["state"].values() for v in st.values() if torch.is_tensor(v))
    ld_opt.load_state_dict(global_sd, from_global=True)
    assert all(v.is_cuda for st in ld_opt.state.values() for k, v in st.items() if torch.is_tensor(v) and v.dim() > 0)
    _train(ld_rm, ld_opt, xs[3:], False)
    for p, w in zip(ld_model.parameters(), want):
        assert_bits_equal(p.detach().cpu(), w, "resumed run")


@pytest.mark.parametrize("enable_zero", [False, True])
@pytest.mark.parametrize("opt_cls", [FusedAdam, torch.optim.Adam])
def test_amp_checkpoint_round_trip(tmp_path, enable_zero, opt_cls):
    """amp O2 (+ ZeRO): the saved model state holds the fp32 masters under the parameter names; the optimizer
    state comes back in the global numbering on the host, in the parameters' shapes, and loads into a fresh
    optimizer as flattened, range-cut device tensors with the same bits."""
    _pyrannc.clear()
    xs = _inputs(4, torch.float16)
    model = _base()
    names = [n for n, _ in model.named_parameters()]
    opt = opt_cls(model.parameters(), lr=1e-2)
    model, opt = amp.initialize(model, opt, opt_level="O2", max_loss_scale=2.0 ** 8)
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True, enable_zero=enable_zero)
    _train(rm, opt, xs[:3], True)
    model_sd = rm.state_dict()
    opt_sd = opt.state_dict(from_global=True)
    torch.save(model_sd, tmp_path / "model.pt")
    torch.save(opt_sd, tmp_path / "opt_state.pt")
    masters = {n: rm.get_param(n, True).detach().cpu().clone() for n in names}
    local_state = {i: {k: (v.detach().cpu().clone() if torch.is_tensor(v) else v) for k, v in opt.state[p].items()}
                   for i, p in enumerate(p for g in opt.param_groups for p in g["params"])}

    loaded = torch.load(tmp_path / "model.pt", map_location="cpu")
    assert list(loaded.keys()) == names
    for n in names:
        assert loaded[n].dtype == torch.float32
        assert_bits_equal(loaded[n].flatten()[:masters[n].numel()], masters[n].flatten(), f"saved master {n}")
    global_sd = torch.load(tmp_path / "opt_state.pt")
    shapes = dict(model.named_parameters())
    for order, n in enumerate(names):
        st = global_sd["state"][order]
        assert sorted(st.keys()) == ["exp_avg", "exp_avg_sq", "step"]
        assert float(st["step"]) == 3.0
        for k in ("exp_avg", "exp_avg_sq"):
            assert st[k].shape == shapes[n].shape and not st[k].is_cuda      # the reference's gather returns view(shape)
            assert_bits_equal(st[k].flatten(), local_state[order][k].flatten(), f"{k} of {n}")

    ld_model = _base(seed=99)                 # a second module next to the first: both go on training below
    ld_model.load_state_dict(loaded)
    ld_opt = opt_cls(ld_model.parameters(), lr=1e-2)
    ld_model, ld_opt = amp.initialize(ld_model, ld_opt, opt_level="O2", max_loss_scale=2.0 ** 8)
    ld_rm = rannc_amd.RaNNCModule(ld_model, ld_opt, enable_apex_amp=True, enable_zero=enable_zero)
    ld_rm._deploy()
    for p, q in zip(ld_model.parameters(), model.parameters()):              # half(master) on both sides
        assert_bits_equal(p.detach().cpu().flatten()[:q.numel()], q.detach().cpu().flatten(), "model parameter")
    ld_opt.load_state_dict(global_sd, from_global=True)
    stepped = [p for g in ld_opt.param_groups for p in g["params"]]
    for i, p in enumerate(stepped):
        for k in ("exp_avg", "exp_avg_sq"):
            got = ld_opt.state[p][k]
            assert got.is_cuda
            if enable_zero:                                                  # flattened and cut to the local range
                rng = ld_opt.param_zero_range[ld_opt.global_order_to_id[i]]
                assert got.dim() == 1 and got.numel() == rng.stop - rng.start
            assert_bits_equal(got.detach().cpu().flatten(), local_state[i][k].flatten(), f"loaded {k} {i}")
        assert float(ld_opt.state[p]["step"]) == 3.0
    # both runs go on: same inputs, and masters that differ only by the half rounding of the reload
    _train(rm, opt, xs[3:], True)
    _train(ld_rm, ld_opt, xs[3:], True)
    for p, q in zip(ld_model.parameters(), model.parameters()):
        torch.testing.assert_close(p.detach().float().cpu().flatten()[:q.numel()], q.detach().float().cpu().flatten(),
                                   rtol=2e-2, atol=2e-3)
