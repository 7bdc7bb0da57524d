"""Pins of the optimizer oracle: the library itself (torch.optim on CPU, bit for bit), a
float64 evaluation of the textbook formulas, and closed forms of the first step."""
import math

import pytest
import torch

from oracle import optim as oracle_optim
from tests.helpers import assert_bits_equal

SHAPES = [(1,), (7,), (64, 33), (1000,), (4099,)]


def _tensors(seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(s, generator=g) * scale for s in SHAPES]


@pytest.mark.parametrize("cls,kw,decoupled", [
    (torch.optim.Adam, dict(lr=1e-3), False),
    (torch.optim.Adam, dict(lr=3e-4, betas=(0.8, 0.99), eps=1e-6, weight_decay=0.01), False),
    (torch.optim.Adam, dict(lr=1e-2, betas=(0.3, 0.9)), False),          # lerp weight >= 0.5 branch
    (torch.optim.AdamW, dict(lr=1e-3, weight_decay=0.05), True),
    (torch.optim.Adam, dict(lr=1e-3, maximize=True), False),
])
def test_adam_oracle_is_torch_optim_bit_for_bit(cls, kw, decoupled):
    params = [torch.nn.Parameter(t) for t in _tensors(1)]
    opt = cls(params, foreach=False, **kw)
    mine = [p.detach().clone() for p in params]
    ms = [torch.zeros_like(p) for p in mine]
    vs = [torch.zeros_like(p) for p in mine]
    b1, b2 = kw.get("betas", (0.9, 0.999))
    for step in range(1, 6):
        grads = _tensors(100 + step, 1e-2)
        for p, g in zip(params, grads):
            p.grad = g.clone()
        opt.step()
        oracle_optim.adam_step(mine, grads, ms, vs, step, lr=kw["lr"], beta1=b1, beta2=b2, eps=kw.get("eps", 1e-8),
                               weight_decay=kw.get("weight_decay", 0.0), decoupled=decoupled,
                               maximize=kw.get("maximize", False))
        for p, q in zip(params, mine):
            assert_bits_equal(q, p.detach(), f"param step {step}")
        for p, m, v in zip(params, ms, vs):
            assert_bits_equal(m, opt.state[p]["exp_avg"], "exp_avg")
            assert_bits_equal(v, opt.state[p]["exp_avg_sq"], "exp_avg_sq")


@pytest.mark.parametrize("kw", [
    dict(lr=0.01),
    dict(lr=0.1, momentum=0.9),
    dict(lr=0.1, momentum=0.9, dampening=0.1, weight_decay=1e-3),
    dict(lr=0.05, momentum=0.8, nesterov=True),
    dict(lr=0.05, weight_decay=0.1, maximize=True),
])
def test_sgd_oracle_is_torch_optim_bit_for_bit(kw):
    params = [torch.nn.Parameter(t) for t in _tensors(2)]
    opt = torch.optim.SGD(params, foreach=False, **kw)
    mine = [p.detach().clone() for p in params]
    bufs = [None] * len(mine)
    for step in range(1, 5):
        grads = _tensors(200 + step, 1e-1)
        for p, g in zip(params, grads):
            p.grad = g.clone()
        opt.step()
        oracle_optim.sgd_step(mine, grads, bufs, kw["lr"], kw.get("momentum", 0.0), kw.get("dampening", 0.0),
                              kw.get("weight_decay", 0.0), kw.get("nesterov", False), kw.get("maximize", False))
        for p, q in zip(params, mine):
            assert_bits_equal(q, p.detach(), f"param step {step}")


def test_adam_oracle_against_float64_and_first_step_closed_form():
    p0, g0 = _tensors(3)[4], _tensors(4, 1e-2)[4]
    p, m, v = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    p64, m64, v64 = p0.double(), m.double(), v.double()
    for step in range(1, 4):
        oracle_optim.adam_step([p], [g0], [m], [v], step, lr=1e-3)
        p64, m64, v64 = oracle_optim.adam_step_f64(p64, g0, m64, v64, step, lr=1e-3)
        assert torch.allclose(p.double(), p64, rtol=1e-6, atol=1e-9)
        assert torch.allclose(m.double(), m64, rtol=1e-6, atol=1e-12)
        assert torch.allclose(v.double(), v64, rtol=1e-6, atol=1e-16)
    # first step from zero state: m_hat = g, v_hat = g^2, so the update is lr * g / (|g| + eps) ~ lr * sign(g)
    p1, m1, v1 = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    oracle_optim.adam_step([p1], [g0], [m1], [v1], 1, lr=1e-3)
    want = p0.double() - 1e-3 * g0.double() / (g0.double().abs() + 1e-8)
    assert torch.allclose(p1.double(), want, rtol=1e-6, atol=1e-9)
    # grad_scale is a plain pre-multiplication
    pa, ma, va = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    pb, mb, vb = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    oracle_optim.adam_step([pa], [g0], [ma], [va], 1, grad_scale=0.25)
    oracle_optim.adam_step([pb], [g0 * 0.25], [mb], [vb], 1)
    assert_bits_equal(pa, pb, "grad_scale")


def test_model_copy_rounds_to_nearest_even():
    x = torch.tensor([1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8, 65520.0, -0.0])
    assert oracle_optim.model_copy(x, torch.bfloat16).tolist() == [1.0, 1.015625, 65536.0, -0.0]
    assert math.isinf(float(oracle_optim.model_copy(x, torch.float16)[2]))
