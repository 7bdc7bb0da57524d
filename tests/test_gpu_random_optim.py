"""Randomised parity of the optimizer step (fixed seeds): random tensor counts and sizes around
tile and chunk boundaries, every gradient / model-copy dtype, parameters, moments, gradients and
copies at arbitrary element offsets inside their allocations, Adam / AdamW / SGD variants.
Tolerances as in test_gpu_optim.py: 2e-6 relative for parameters and state, bit-exact model copy."""
import random

import pytest
import torch

from oracle import optim as oracle_optim
from rannc_amd import _lib
from rannc_amd.multi_tensor import stream_handle
from tests.helpers import TORCH_DTYPE, assert_bits_equal

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
SIZES = [1, 3, 31, 32, 33, 1000, 1023, 1025, 4095, 4096, 4097, 16383, 16384, 16385, 16384 + 31, 20000]


def _arena(tensors, lead, gap):
    total = lead + sum(t.numel() + gap for t in tensors) + 64
    arena = torch.zeros(total, dtype=tensors[0].dtype, device=DEV)
    views, off = [], lead
    for t in tensors:
        v = arena.narrow(0, off, t.numel())
        v.copy_(t)
        views.append(v)
        off += t.numel() + gap
    return views


@pytest.mark.parametrize("seed", range(40))
def test_random_optimizer_tables(seed):
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    n = rng.randint(1, 12)
    sizes = [rng.choice(SIZES + [rng.randint(1, 70000)]) for _ in range(n)]
    gname = rng.choice(["f32", "f16", "bf16"])
    cname = rng.choice([None, "f32", "f16", "bf16"])
    algo = rng.choice(["adam", "adamw", "sgd", "sgd_momentum", "sgd_nesterov"])
    adam, momentum = algo.startswith("adam"), algo in ("sgd_momentum", "sgd_nesterov")
    p_cpu = [torch.randn(s, generator=g) for s in sizes]
    m_cpu = [torch.randn(s, generator=g) * 1e-2 for s in sizes]
    v_cpu = [torch.rand(s, generator=g) * 1e-4 for s in sizes]
    g_cpu = [(torch.randn(s, generator=g) * 1e-2).to(TORCH_DTYPE[gname]) for s in sizes]
    p = _arena(p_cpu, rng.randint(0, 40), rng.randint(0, 3))
    m = _arena(m_cpu, rng.randint(0, 40), rng.randint(0, 3))
    v = _arena(v_cpu, rng.randint(0, 40), 1)
    gd = _arena(g_cpu, rng.randint(0, 40), rng.randint(0, 3))
    c = _arena([torch.zeros(s, dtype=TORCH_DTYPE[cname]) for s in sizes], rng.randint(0, 40), rng.randint(0, 3)) if cname else None
    table = _lib.OptimTable(0, [x.data_ptr() for x in p], [x.data_ptr() for x in gd],
                            [x.data_ptr() for x in m] if (adam or momentum) else None,
                            [x.data_ptr() for x in v] if adam else None, [x.data_ptr() for x in c] if c else None, sizes,
                            [_lib.DTYPE_CODES[gname]] * n, [_lib.DTYPE_CODES[cname]] * n if cname else None)
    stream = stream_handle(DEV)
    wd, gscale, step = rng.choice([0.0, 0.01]), rng.choice([1.0, 0.25]), rng.randint(1, 50)
    if adam:
        table.adam_step(1e-3, 0.9, 0.999, 1e-8, wd, step, decoupled=(algo == "adamw"), grad_scale=gscale, stream=stream)
        oracle_optim.adam_step(p_cpu, g_cpu, m_cpu, v_cpu, step, weight_decay=wd, decoupled=(algo == "adamw"), grad_scale=gscale)
    else:
        mom = 0.9 if momentum else 0.0
        table.sgd_step(0.05, momentum=mom, weight_decay=wd, nesterov=(algo == "sgd_nesterov"), grad_scale=gscale, stream=stream)
        oracle_optim.sgd_step(p_cpu, g_cpu, list(m_cpu) if momentum else None, 0.05, momentum=mom, weight_decay=wd,
                              nesterov=(algo == "sgd_nesterov"), grad_scale=gscale)
    what = f"seed {seed} {algo} grad {gname} copy {cname}"
    for i in range(n):
        torch.testing.assert_close(p[i].cpu(), p_cpu[i], rtol=2e-6, atol=2e-8, msg=lambda s: f"{what} param {i}: {s}")
        if adam or momentum:
            torch.testing.assert_close(m[i].cpu(), m_cpu[i], rtol=2e-6, atol=1e-12, msg=lambda s: f"{what} state1 {i}: {s}")
        if adam:
            torch.testing.assert_close(v[i].cpu(), v_cpu[i], rtol=2e-6, atol=1e-16, msg=lambda s: f"{what} state2 {i}: {s}")
        if c:
            assert_bits_equal(c[i].cpu(), p[i].cpu().to(TORCH_DTYPE[cname]), f"{what} model copy {i}")
    table.close()
