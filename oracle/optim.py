"""TEST INFRASTRUCTURE ONLY - CPU restatement of the optimizer step that follows the clip.

The reference leaves the step to ``torch.optim`` (``optim.Adam(model.parameters(), lr=lr)`` at
``test/common.py:142,165``; ``optim.SGD(model.parameters(), lr=0.01)`` at
``examples/tutorial.py:28``) on the parameters ``pyrannc/opt.py:205-312`` hands it, and under
amp Apex copies each fp32 master into its fp16 model parameter afterwards
(``pyrannc/amp/__init__.py:10-18`` keeps the pairing).  The functions below spell that
arithmetic out per tensor in fp32 ATen ops in the order ``torch/optim/adam.py`` and
``torch/optim/sgd.py`` (single-tensor forms) use, with the scalar factors computed in double
from Python floats.  Pinned in ``tests/test_oracle_optim.py`` against the library itself
(``torch.optim.Adam / AdamW / SGD`` on CPU, bit for bit over several steps), against a float64
evaluation of the textbook formulas, and against closed forms of the first step.

Only tests, ``__graft_entry__.smoke()`` and the CPU-baseline leg of ``bench.py`` may import this.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch


def adam_step(params: Sequence[torch.Tensor], grads: Sequence[torch.Tensor], exp_avgs: Sequence[torch.Tensor],
              exp_avg_sqs: Sequence[torch.Tensor], step: int, lr: float = 1e-3, beta1: float = 0.9,
              beta2: float = 0.999, eps: float = 1e-8, weight_decay: float = 0.0, decoupled: bool = False,
              maximize: bool = False, grad_scale: float = 1.0) -> None:
    """One Adam (``decoupled``: AdamW) step in place; ``step`` counts from 1 and is shared by
    the tensors given.  ``grad_scale`` multiplies every gradient first (in fp32)."""
    bias_correction1 = 1 - beta1 ** step
    bias_correction2 = 1 - beta2 ** step
    step_size = lr / bias_correction1
    bias_correction2_sqrt = bias_correction2 ** 0.5
    scale = torch.tensor(grad_scale, dtype=torch.float32)
    for p, g, m, v in zip(params, grads, exp_avgs, exp_avg_sqs):
        g = g.to(torch.float32) * scale
        if maximize:
            g = -g
        if weight_decay != 0:
            if decoupled:
                p.mul_(1 - lr * weight_decay)
            else:
                g = g.add(p, alpha=weight_decay)
        m.lerp_(g, 1 - beta1)
        v.mul_(beta2).addcmul_(g, g, value=1 - beta2)
        denom = (v.sqrt() / bias_correction2_sqrt).add_(eps)
        p.addcdiv_(m, denom, value=-step_size)


def sgd_step(params: Sequence[torch.Tensor], grads: Sequence[torch.Tensor],
             momentum_buffers: Optional[List[Optional[torch.Tensor]]], lr: float, momentum: float = 0.0,
             dampening: float = 0.0, weight_decay: float = 0.0, nesterov: bool = False, maximize: bool = False,
             grad_scale: float = 1.0) -> None:
    """One SGD step in place.  ``momentum_buffers[i] is None`` = first step of that buffer
    (it becomes a copy of the gradient); the list is updated."""
    scale = torch.tensor(grad_scale, dtype=torch.float32)
    for i, (p, g) in enumerate(zip(params, grads)):
        g = g.to(torch.float32) * scale
        if maximize:
            g = -g
        if weight_decay != 0:
            g = g.add(p, alpha=weight_decay)
        if momentum != 0:
            buf = momentum_buffers[i]
            if buf is None:
                buf = g.clone()
                momentum_buffers[i] = buf
            else:
                buf.mul_(momentum).add_(g, alpha=1 - dampening)
            g = g.add(buf, alpha=momentum) if nesterov else buf
        p.add_(g, alpha=-lr)


def adam_step_f64(p, g, m, v, step, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0, decoupled=False):
    """Textbook Adam in float64 on float64 copies; returns (p, m, v).  Yardstick only."""
    p, g, m, v = (t.to(torch.float64) for t in (p, g, m, v))
    if weight_decay != 0:
        if decoupled:
            p = p * (1 - lr * weight_decay)
        else:
            g = g + weight_decay * p
    m = beta1 * m + (1 - beta1) * g
    v = beta2 * v + (1 - beta2) * g * g
    m_hat = m / (1 - beta1 ** step)
    v_hat = v / (1 - beta2 ** step)
    p = p - lr * m_hat / (v_hat.sqrt() + eps)
    return p, m, v


def model_copy(master: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Apex's post-step ``model = half(master)``: ATen's round-to-nearest-even conversion."""
    return master.to(dtype)
