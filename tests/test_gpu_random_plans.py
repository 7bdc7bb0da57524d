"""Randomised parity (fixed seeds): tensor lists with random sizes, mixed dtypes per tensor,
missing gradients and arbitrary element offsets of sources and destinations, checked against
the CPU oracle for the fused step, the one-pass unscale+pack, casts and the norm."""
import math
import random

import pytest
import torch

from oracle import gradpath as oracle
from rannc_amd import _lib
from rannc_amd.multi_tensor import TensorPlan
from tests.helpers import assert_bits_equal

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTS = [torch.float32, torch.float16, torch.bfloat16]
NAME = {torch.float32: "f32", torch.float16: "f16", torch.bfloat16: "bf16"}


def _random_case(seed, max_tensors=40):
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    n_t = rng.randint(1, max_tensors)
    sizes = []
    for _ in range(n_t):
        kind = rng.random()
        if kind < 0.15:
            sizes.append(rng.choice([0, 1, 2, 3, 7, 8, 9]))
        elif kind < 0.6:
            sizes.append(rng.randint(10, 5000))
        elif kind < 0.9:
            sizes.append(rng.randint(5000, 60000))
        else:
            sizes.append(rng.choice([16383, 16384, 16385, 32769, 131071, 200003]))
    pairs = [(rng.choice(DTS), rng.choice(DTS)) for _ in range(n_t)]
    scale_pow = rng.choice([0, 4, 8, 12])
    srcs = [(torch.randn(n, generator=g) * 10 ** rng.uniform(-3, 1) * 2.0 ** scale_pow).to(sd) for n, (sd, _) in zip(sizes, pairs)]
    return rng, sizes, pairs, srcs, 2.0 ** -scale_pow


def _place(tensors_by_dtype_order, rng, fill=0.0):
    """One arena per dtype; every tensor at a random element offset from the previous one."""
    out = [None] * len(tensors_by_dtype_order)
    for dt in DTS:
        idx = [i for i, t in enumerate(tensors_by_dtype_order) if t.dtype == dt]
        if not idx:
            continue
        gaps = [rng.randint(0, 9) for _ in idx]
        total = sum(tensors_by_dtype_order[i].numel() + gp for i, gp in zip(idx, gaps)) + 16
        arena = torch.full((total,), fill, dtype=dt, device=DEV)
        off = 0
        for i, gp in zip(idx, gaps):
            off += gp
            n = tensors_by_dtype_order[i].numel()
            v = arena.narrow(0, off, n)
            v.copy_(tensors_by_dtype_order[i])
            out[i] = v
            off += n
    return out


@pytest.mark.parametrize("one_pass", [False, True])
@pytest.mark.parametrize("seed", range(24))
def test_random_fused_step(seed, one_pass):
    """``one_pass``: the same cases under RG_STEP_EXPECT_NO_CLIP (write while summing, in-place multiply only if the
    step clips after all) - same bits; after an overflow that strategy has written the unscaled values."""
    rng, sizes, pairs, srcs_cpu, inv_scale = _random_case(seed)
    srcs = _place(srcs_cpu, rng)
    dsts = _place([torch.full((n,), 3.0, dtype=dd) for n, (_, dd) in zip(sizes, pairs)], rng, fill=3.0)
    missing = set(i for i in range(len(sizes)) if rng.random() < 0.1)
    plan_srcs = [None if i in missing else s for i, s in enumerate(srcs)]
    max_norm = rng.choice([1e-3, 0.5, 1e6])
    plan = TensorPlan(plan_srcs, dsts, chunk_elems=rng.choice([0, 2048, 4096, 16384]))
    plan.fused_step(inv_scale, max_norm, _lib.RG_STEP_EXPECT_NO_CLIP if one_pass else _lib.RG_STEP_DEFAULT)
    res = plan.result()
    tn = plan.tensor_norms()
    # oracle, tensor by tensor (destination dtypes differ per tensor)
    unscaled, norms, flag = [], [], 0
    for i, (s, (sd, dd)) in enumerate(zip(srcs_cpu, pairs)):
        if i in missing:
            u = torch.zeros(sizes[i], dtype=dd)
        else:
            us, f = oracle.unscale_and_check([s], inv_scale, dd)
            u = us[0]
            flag |= f
        unscaled.append(u)
        norms.append(oracle.per_tensor_norms([u])[0])
    assert res.overflow == flag
    if flag:        # a source value did not fit its half type: the step is skipped, nothing is written
        assert res.skipped == 1 and res.clipped == 0
        if one_pass:
            for i, (u, d) in enumerate(zip(unscaled, dsts)):
                assert_bits_equal(d.cpu(), u, f"seed {seed} tensor {i}: unscaled values after an overflow")
        else:
            assert all(bool((d == 3.0).all()) for d in dsts)
        return
    total = math.sqrt(sum(n * n for n in norms))
    assert math.isclose(res.norm, total, rel_tol=1e-6, abs_tol=1e-30)
    for a, b in zip(tn, norms):
        assert math.isclose(a, b, rel_tol=1e-6, abs_tol=1e-30)
    coef = oracle.clip_coefficient(total, max_norm)
    assert res.clipped == (1 if coef is not None else 0)
    c32 = torch.tensor(res.coef, dtype=torch.float32)
    for i, (u, d) in enumerate(zip(unscaled, dsts)):
        want = (u.float() * c32).to(u.dtype) if res.clipped else u
        assert_bits_equal(d.cpu(), want, f"seed {seed} tensor {i} {pairs[i]}")
    plan.close()


@pytest.mark.parametrize("seed", range(100, 112))
def test_random_unscale_pack_and_cast(seed):
    rng, sizes, pairs, srcs_cpu, inv_scale = _random_case(seed, max_tensors=25)
    srcs = _place(srcs_cpu, rng)
    dsts = _place([torch.zeros(n, dtype=dd) for n, (_, dd) in zip(sizes, pairs)], rng)
    plan = TensorPlan(srcs, dsts)
    plan.unscale_pack(inv_scale)
    res = plan.result()
    norms, flag = [], 0
    for s, d, (_, dd) in zip(srcs_cpu, dsts, pairs):
        us, f = oracle.unscale_and_check([s], inv_scale, dd)
        flag |= f
        assert_bits_equal(d.cpu(), us[0], f"seed {seed} unscale_pack")
        norms.append(oracle.per_tensor_norms([us[0]])[0])
    assert res.overflow == flag
    total = math.sqrt(sum(n * n for n in norms))
    if math.isfinite(total):
        assert math.isclose(res.norm, total, rel_tol=1e-6, abs_tol=1e-30)
    else:
        assert not math.isfinite(res.norm)
    plan.scale_cast(1.0)
    for s, d, (_, dd) in zip(srcs_cpu, dsts, pairs):
        assert_bits_equal(d.cpu(), oracle.cast(s, dd), f"seed {seed} cast")
    plan.grad_norm()
    want_norm = oracle.grad_global_l2_norm(srcs_cpu)
    if math.isfinite(want_norm):
        assert math.isclose(plan.result().norm, want_norm, rel_tol=1e-6, abs_tol=1e-30)
    plan.zero()
    torch.cuda.synchronize()
    assert all(bool((d == 0).all()) for d in dsts)
    plan.close()


@pytest.mark.parametrize("seed", range(200, 206))
def test_random_overflow_positions(seed):
    rng, sizes, pairs, srcs_cpu, inv_scale = _random_case(seed, max_tensors=12)
    nonempty = [i for i, n in enumerate(sizes) if n > 0]
    if not nonempty:
        pytest.skip("all tensors empty")
    ti = rng.choice(nonempty)
    srcs_cpu[ti].view(-1)[rng.randrange(sizes[ti])] = rng.choice([float("inf"), float("-inf"), float("nan")])
    srcs = _place(srcs_cpu, rng)
    dsts = _place([torch.full((n,), 3.0, dtype=dd) for n, (_, dd) in zip(sizes, pairs)], rng, fill=3.0)
    plan = TensorPlan(srcs, dsts)
    plan.fused_step(inv_scale, 1.0)
    res = plan.result()
    assert res.overflow == 1 and res.skipped == 1 and res.clipped == 0
    assert all(bool((d == 3.0).all()) for d in dsts)
    plan.fused_step(inv_scale, 1.0, _lib.RG_STEP_WRITE_ON_OVERFLOW)
    for s, d, (_, dd) in zip(srcs_cpu, dsts, pairs):
        assert_bits_equal(d.cpu(), oracle.unscale_and_check([s], inv_scale, dd)[0][0], "written on overflow")
    plan.close()


@pytest.mark.parametrize("one_pass", [False, True])
def test_thousands_of_tiny_tensors(one_pass):
    """3000 tensors of 0 to 40 elements (biases, layer-norm vectors), mixed dtypes, packed into one fp32 bucket at
    running-sum offsets: nearly every chunk is a ragged sliver and most write tiles are empty."""
    rng = random.Random(77)
    g = torch.Generator().manual_seed(77)
    sizes = [rng.randint(0, 40) for _ in range(3000)]
    srcs_cpu = [(torch.randn(n, generator=g) * 0.05 * 256.0).to(rng.choice(DTS)) for n in sizes]
    srcs = _place(srcs_cpu, rng)
    total = sum(sizes)
    bucket = torch.full((total + 3,), 5.0, dtype=torch.float32, device=DEV)[3:]
    dsts, off = [], 0
    for n in sizes:
        dsts.append(bucket.narrow(0, off, n))
        off += n
    plan = TensorPlan(srcs, dsts)
    plan.fused_step(1.0 / 256.0, 0.5, _lib.RG_STEP_EXPECT_NO_CLIP if one_pass else _lib.RG_STEP_DEFAULT)
    res, tn = plan.result(), plan.tensor_norms()
    want = oracle.fused_step(srcs_cpu, ["f32"] * len(srcs_cpu), 1.0 / 256.0, 0.5)
    assert res.overflow == want.overflow == 0 and res.clipped == 1
    assert math.isclose(res.norm, want.norm, rel_tol=1e-6)
    for a, b in zip(tn, want.tensor_norms):
        assert math.isclose(a, b, rel_tol=1e-6, abs_tol=1e-30)
    unscaled = oracle.fused_step(srcs_cpu, ["f32"] * len(srcs_cpu), 1.0 / 256.0, math.inf).buckets["f32"]
    unscaled.mul_(float(res.coef))
    assert_bits_equal(bucket.cpu(), unscaled, "bucket of tiny tensors")
    plan.close()
