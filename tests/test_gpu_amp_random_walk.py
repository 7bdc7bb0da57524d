"""Seeded random training loops through the mirror of the reference API - ``amp.scale_loss`` contexts (one to three per
step: gradient accumulation), injected overflows, a parameter without a gradient, ``amp.master_params`` read in
mid-step, ``RaNNCModule.clip_grad_norm`` that clips or not, ``optimizer.step``, ``zero_grad`` - checked after every
step against the oracle's restatement of the same sequence on the CPU: Apex's unscale / accumulate / flag
(``oracle.unscale_and_check``, ``unscale_accumulate``), the reference's scaler wrapper (``patched_update_scale``,
``pyrannc/amp/__init__.py:44-65``), ``ParamStorage::clipGradNorm`` (``oracle.clip_grad_norm``), ``torch.optim.Adam``
(``oracle.optim.adam_step``) and the master -> model copy.  The single-feature tests exercise each of these alone;
this one walks the state machine behind them (deferred or eager write, one- or two-pass strategy, steady-state
records, tables that are re-pointed or rebuilt) through orders nobody wrote down by hand."""
import random

import pytest
import torch

import rannc_amd
from oracle import gradpath as oracle
from oracle import optim as oracle_optim
from rannc_amd import amp
from rannc_amd.fused_optim import FusedAdam
from tests.helpers import assert_bits_equal

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SHAPES = [(64, 33), (33,), (128, 64), (7,), (1, 257), (96, 96)]
LR = 1e-2
STEPS = 24


class _Holder(torch.nn.Module):
    def __init__(self, gen):
        super().__init__()
        self.ps = torch.nn.ParameterList([torch.nn.Parameter((torch.randn(s, generator=gen) * 0.1).to(DEV)) for s in SHAPES])

    def forward(self, x):
        return x


def _walk(seed, half, fused, fused_opt, scale_mode):
    """Runs one loop; returns the masters at the end (for the comparison between configurations)."""
    rng = random.Random(seed)
    gen = torch.Generator().manual_seed(seed)
    model = _Holder(gen)
    opt_cls = FusedAdam if fused_opt else torch.optim.Adam
    opt = opt_cls(model.parameters(), lr=LR)
    dynamic = scale_mode != "static"
    model, opt = amp.initialize(model, opt, opt_level="O2", half_dtype=half, fused=fused,
                                loss_scale="dynamic" if dynamic else 512.0, max_loss_scale=2.0 ** 12,
                                device_loss_scale=scale_mode == "device")
    scaler = amp._amp_state.loss_scalers[0]
    if dynamic:
        scaler._loss_scale, scaler._scale_seq_len = 1000.0, 3        # not a power of two: the wrapper's int() matters
        if scale_mode == "device":
            scaler.to_device(torch.device(DEV))
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    rm._deploy()
    rm._setup_amp_params()                                            # patches the scaler as the reference's __call__ does
    stash = opt._amp_stash
    halves, masters = stash.all_fp16_params, stash.all_fp32_from_fp16_params
    n = len(halves)
    assert n == len(SHAPES) and all(p.dtype == half for p in halves)

    want_scaler = oracle.LossScalerState(loss_scale=1000.0 if dynamic else 512.0, unskipped=0, scale_window=3,
                                         min_loss_scale=None, max_loss_scale=2.0 ** 12, dynamic=dynamic)
    want_p = [m.detach().cpu().clone() for m in masters]
    want_m = [torch.zeros_like(p) for p in want_p]
    want_v = [torch.zeros_like(p) for p in want_p]
    counts = [0] * n
    loss = torch.zeros((), device=DEV)

    for step in range(STEPS):
        micro_batches = 1 if scale_mode == "device" else rng.choice([1, 1, 2, 3])
        missing = rng.randrange(n) if (scale_mode != "device" and rng.random() < 0.15) else None
        inject_at = rng.randrange(micro_batches) if (dynamic and rng.random() < 0.2) else None
        read_masters = rng.random() < 0.25
        clip = rng.random() < 0.7
        max_norm = rng.choice([1e-3, 1e-2, 1e6])
        tag = f"seed {seed} step {step} (mb {micro_batches}, missing {missing}, inf at {inject_at}, read {read_masters}, " \
              f"clip {clip and max_norm})"

        want_grads = [None] * n
        skip = False
        for mb in range(micro_batches):
            assert scaler.loss_scale() == float(want_scaler.loss_scale), tag
            scale = float(want_scaler.loss_scale)
            cpu_grads = []
            for i, s in enumerate(SHAPES):
                if i == missing:
                    cpu_grads.append(None)
                    continue
                g = (torch.randn(s, generator=gen) * 1e-2 * scale).to(half)
                if inject_at == mb and i == (step % n if step % n != missing else (step + 1) % n):
                    g.view(-1)[g.numel() // 2] = float("inf") if step % 2 else float("nan")
                cpu_grads.append(g)
            with amp.scale_loss(loss, opt):
                for p, g in zip(halves, cpu_grads):
                    p.grad = None if g is None else g.to(DEV)
            present = [i for i in range(n) if cpu_grads[i] is not None]
            if mb == 0:
                vals, flag = oracle.unscale_and_check([cpu_grads[i] for i in present], 1.0 / scale)
                for i, v in zip(present, vals):
                    want_grads[i] = v
            else:
                flag = oracle.unscale_accumulate([want_grads[i] for i in present], [cpu_grads[i] for i in present], 1.0 / scale)
            if scale_mode != "device":
                skip = oracle.patched_update_scale(want_scaler, bool(flag)) or skip
            else:
                skip = bool(flag)
        if read_masters:
            got = [m.grad for m in amp.master_params(opt)]
            if not skip:
                for i in range(n):
                    if want_grads[i] is None:
                        assert got[i] is None, tag
                    else:
                        assert_bits_equal(got[i].cpu(), want_grads[i], f"{tag}: master grad {i}")
        if clip:
            rm.clip_grad_norm(max_norm)
            if not skip:
                oracle.clip_grad_norm([g for g in want_grads if g is not None], float(torch.tensor(max_norm, dtype=torch.float32)))
        opt.step()
        opt.zero_grad()
        rm.zero_grad()
        if scale_mode == "device":                    # the device applies the schedule after the step
            oracle.patched_update_scale(want_scaler, skip)
        if not skip:
            for i in range(n):
                if want_grads[i] is None:
                    continue
                counts[i] += 1
                oracle_optim.adam_step([want_p[i]], [want_grads[i]], [want_m[i]], [want_v[i]], counts[i], lr=LR)
        torch.cuda.synchronize()
        assert scaler.loss_scale() == float(want_scaler.loss_scale), tag
        for i in range(n):
            got_p = masters[i].detach().cpu()
            torch.testing.assert_close(got_p, want_p[i], rtol=2e-6, atol=2e-6 * LR, msg=lambda m: f"{tag}: master {i}: {m}")
            assert_bits_equal(halves[i].detach().cpu(), oracle_optim.model_copy(got_p, half), f"{tag}: model copy {i}")
            st = opt.state.get(masters[i], {})
            if counts[i]:
                assert float(st["step"]) == counts[i], tag
                torch.testing.assert_close(st["exp_avg"].cpu(), want_m[i], rtol=2e-6, atol=1e-9, msg=lambda m: f"{tag}: exp_avg {i}: {m}")
                torch.testing.assert_close(st["exp_avg_sq"].cpu(), want_v[i], rtol=2e-6, atol=1e-12, msg=lambda m: f"{tag}: exp_avg_sq {i}: {m}")
                # the oracle follows the GPU from here: differences of the last bit must not pile up over the walk
                want_m[i], want_v[i] = st["exp_avg"].cpu().clone(), st["exp_avg_sq"].cpu().clone()
            want_p[i] = got_p.clone()
    return [m.detach().cpu().clone() for m in masters]


CONFIGS = [
    # half dtype, fused amp, fused optimizer, loss scale
    (torch.float16, True, True, "dynamic"),
    (torch.float16, False, True, "dynamic"),
    (torch.bfloat16, True, False, "dynamic"),
    (torch.bfloat16, False, False, "dynamic"),
    (torch.bfloat16, True, True, "static"),
    (torch.float16, True, True, "device"),
]


@pytest.mark.parametrize("seed", [11, 12, 13])
@pytest.mark.parametrize("half,fused,fused_opt,scale_mode", CONFIGS,
                         ids=[f"{str(h).split('.')[-1]}-{'fused' if f else 'eager'}-{'FusedAdam' if o else 'torchAdam'}-{s}"
                              for h, f, o, s in CONFIGS])
def test_random_training_loop_follows_the_oracle(seed, half, fused, fused_opt, scale_mode):
    _walk(seed, half, fused, fused_opt, scale_mode)


@pytest.mark.parametrize("seed", [21, 22])
def test_deferred_and_eager_routes_end_at_the_same_bits(seed):
    """The same loop with the write of the master gradients deferred (``fused=True``: one- or two-pass strategy, or no
    write at all because the optimizer reads the model gradients) and eager (``fused=False``): identical masters."""
    a = _walk(seed, torch.float16, True, True, "dynamic")
    b = _walk(seed, torch.float16, False, True, "dynamic")
    for i, (x, y) in enumerate(zip(a, b)):
        assert_bits_equal(x, y, f"seed {seed}: master {i}")
