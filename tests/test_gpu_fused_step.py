"""GPU parity of the fused unscale + flag + norm + clip + pack step against the CPU oracle.

Bars: bucket contents, overflow flag and the clip decision bit-exact; global norm, per-tensor
norms and the clip coefficient within 1e-6 relative (fp32 accumulation order differs).
The clipped values are compared bit-for-bit against the oracle's unscaled bucket multiplied,
on the CPU, by the coefficient the GPU reported (the coefficient itself is held to 1e-6).
"""
import math

import pytest
import torch

from oracle import gradpath as oracle
from rannc_amd import _lib
from rannc_amd.multi_tensor import TensorPlan
from tests.helpers import TORCH_DTYPE, assert_bits_equal, place_in_arena

pytestmark = pytest.mark.gpu
REL = 1e-6
DEV = "cuda:0"


def _grads(shapes, dtype, std, scale, seed):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(s, generator=g) * std * scale).to(dtype) for s in shapes]


def _run_fused(grads_cpu, dst_dtype, inv_scale, max_norm, flags=_lib.RG_STEP_DEFAULT, chunk_elems=0,
               lead=1, gap=1, dst_lead=3, prefill=7.0):
    srcs = place_in_arena(grads_cpu, DEV, lead, gap)
    numels = [g.numel() for g in grads_cpu]
    total = sum(numels)
    bucket_all = torch.full((total + dst_lead + 5,), prefill, dtype=dst_dtype, device=DEV)
    bucket = bucket_all.narrow(0, dst_lead, total)
    offs, _ = oracle.bucket_layout(numels, ["f32"] * len(numels))
    dsts = [bucket.narrow(0, o, n) for o, n in zip(offs, numels)]
    plan = TensorPlan(srcs, dsts, chunk_elems=chunk_elems)
    plan.fused_step(inv_scale, max_norm, flags)
    res = plan.result()
    tnorms = plan.tensor_norms()
    torch.cuda.synchronize()
    out = bucket.cpu()
    guard = torch.cat([bucket_all[:dst_lead], bucket_all[dst_lead + total:]]).cpu()
    assert bool((guard == prefill).all()), "wrote outside the bucket"
    plan.close()
    return res, tnorms, out


def _check_against_oracle(grads_cpu, dst_name, inv_scale, max_norm, res, tnorms, out, prefill=7.0):
    n = len(grads_cpu)
    want = oracle.fused_step(grads_cpu, [dst_name] * n, inv_scale, max_norm)
    assert res.overflow == want.overflow
    if want.overflow:
        assert res.skipped == 1 and res.clipped == 0
        return want
    assert math.isclose(res.norm, want.norm, rel_tol=REL, abs_tol=1e-30), (res.norm, want.norm)
    for i, (a, b) in enumerate(zip(tnorms, want.tensor_norms)):
        assert math.isclose(a, b, rel_tol=REL, abs_tol=1e-30), (i, a, b)
    assert res.clipped == (1 if want.coef is not None else 0)
    # unscaled bucket from the oracle, then the GPU's own coefficient applied on the CPU
    unscaled = oracle.fused_step(grads_cpu, [dst_name] * n, inv_scale, math.inf).buckets.get(dst_name)
    if unscaled is None:
        unscaled = torch.zeros(0, dtype=TORCH_DTYPE[dst_name])
    if want.coef is not None:
        assert math.isclose(res.coef, want.coef, rel_tol=REL), (res.coef, want.coef)
        unscaled.mul_(float(res.coef))
    else:
        assert res.coef == 1.0
    assert_bits_equal(out, unscaled, "bucket")
    return want


SHAPES_SMALL = [(0,), (1,), (3,), (7,), (8,), (9,), (63,), (64,), (65,), (1000,), (33, 31), (2049,), (4096,), (12345,)]


@pytest.mark.parametrize("src_name,dst_name", [("f32", "f32"), ("f16", "f32"), ("bf16", "f32"), ("f16", "f16"),
                                               ("bf16", "bf16"), ("f32", "bf16"), ("f32", "f16"), ("bf16", "f16"),
                                               ("f16", "bf16")])
@pytest.mark.parametrize("max_norm", [1.0, 1e9])
def test_small_shapes_all_dtype_pairs(src_name, dst_name, max_norm):
    scale = 1.0 if src_name == "f32" else 256.0
    grads = _grads(SHAPES_SMALL, TORCH_DTYPE[src_name], 1e-1, scale, seed=1)
    res, tn, out = _run_fused(grads, TORCH_DTYPE[dst_name], 1.0 / scale, max_norm)
    _check_against_oracle(grads, dst_name, 1.0 / scale, max_norm, res, tn, out)


@pytest.mark.parametrize("lead,gap,dst_lead", [(0, 0, 0), (1, 1, 1), (3, 2, 5), (7, 5, 2), (4, 4, 4)])
@pytest.mark.parametrize("src_name", ["f32", "f16", "bf16"])
def test_alignment_sweep(lead, gap, dst_lead, src_name):
    shapes = [(5000,), (17,), (8191,), (8192,), (8193,), (40000,)]
    grads = _grads(shapes, TORCH_DTYPE[src_name], 1e-2, 64.0, seed=2)
    res, tn, out = _run_fused(grads, torch.float32, 1 / 64.0, 0.5, chunk_elems=2048, lead=lead, gap=gap, dst_lead=dst_lead)
    _check_against_oracle(grads, "f32", 1 / 64.0, 0.5, res, tn, out)


@pytest.mark.parametrize("chunk", [2048, 4096, 16384, 0])
def test_chunk_sizes_multi_chunk_tensor(chunk):
    shapes = [(300001,), (5,), (70000,), (2048 * 3,)]
    grads = _grads(shapes, torch.bfloat16, 1e-2, 65536.0, seed=3)
    res, tn, out = _run_fused(grads, torch.float32, 1 / 65536.0, 1.0, chunk_elems=chunk)
    _check_against_oracle(grads, "f32", 1 / 65536.0, 1.0, res, tn, out)


@pytest.mark.parametrize("src_name", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("where", ["first", "last", "odd", "every_tensor"])
@pytest.mark.parametrize("value", [float("inf"), float("-inf"), float("nan")])
def test_overflow_flag(src_name, where, value):
    shapes = [(129,), (5000,), (1,), (20000,)]
    grads = _grads(shapes, TORCH_DTYPE[src_name], 1e-2, 16.0, seed=4)
    if where == "first":
        grads[0].view(-1)[0] = value
    elif where == "last":
        grads[-1].view(-1)[-1] = value
    elif where == "odd":
        grads[1].view(-1)[2501] = value
    else:
        for g in grads:
            g.view(-1)[g.numel() // 2] = value
    res, tn, out = _run_fused(grads, torch.float32, 1 / 16.0, 1.0, chunk_elems=2048)
    assert res.overflow == 1 and res.skipped == 1 and res.clipped == 0
    assert bool((out == 7.0).all()), "write pass must be skipped on overflow"
    # Apex-identical contents on request: unscaled, unclipped
    res2, _, out2 = _run_fused(grads, torch.float32, 1 / 16.0, 1.0, flags=_lib.RG_STEP_WRITE_ON_OVERFLOW, chunk_elems=2048)
    assert res2.overflow == 1 and res2.clipped == 0
    want, flag = oracle.unscale_and_check(grads, 1 / 16.0)
    assert flag == 1
    assert_bits_equal(out2, torch.cat([w.flatten() for w in want]), "unscaled on overflow")


def test_no_false_overflow_at_dtype_max():
    g16 = torch.full((4099,), 65504.0, dtype=torch.float16)
    gb = torch.full((4099,), 3.3895e38, dtype=torch.bfloat16)
    for g in (g16, gb):
        res, tn, out = _run_fused([g], torch.float32, 1.0, 0.0)
        assert res.overflow == 0
    # finite fp32 inputs whose squares overflow fp32: norm is inf but the flag stays 0
    big = torch.full((5000,), 1e30, dtype=torch.float32)
    res, tn, out = _run_fused([big], torch.float32, 1.0, 0.0)
    assert res.overflow == 0 and math.isinf(res.norm)
    assert_bits_equal(out, big, "values pass through")


def test_zero_grads_do_not_clip():
    grads = [torch.zeros(1000), torch.zeros(3)]
    res, tn, out = _run_fused(grads, torch.float32, 1.0, 1e-9)
    # norm 0 -> 0 + 1e-6 > 1e-9 is TRUE in the reference (ParamStorage.cpp:723-725): it clips with coef 1e-9/1e-6
    want = oracle.fused_step(grads, ["f32", "f32"], 1.0, 1e-9)
    assert (want.coef is not None) == bool(res.clipped)
    res, tn, out = _run_fused(grads, torch.float32, 1.0, 1.0)
    assert res.clipped == 0 and res.norm == 0.0 and bool((out == 0).all())


def test_threshold_is_strict_and_eps_added_before_compare():
    g = torch.zeros(16)
    g[0] = 3.0
    g[1] = 4.0           # norm exactly 5
    for max_norm, clipped in [(5.0, 1), (5.000002, 0), (4.9999, 1), (5.5, 0)]:
        res, _, out = _run_fused([g], torch.float32, 1.0, max_norm)
        want = oracle.fused_step([g], ["f32"], 1.0, max_norm)
        assert res.clipped == clipped == (1 if want.coef is not None else 0), max_norm
        if clipped:
            assert math.isclose(res.coef, want.coef, rel_tol=REL)


def test_subnormal_products_are_kept():
    # bf16 values whose product with 2^-16 is an fp32 subnormal: must not be flushed
    g = torch.tensor([1e-36, -3e-37, 2e-38, 1.0], dtype=torch.bfloat16).repeat(600)
    res, tn, out = _run_fused([g], torch.float32, 2.0 ** -16, 0.0)
    want, _ = oracle.unscale_and_check([g], 2.0 ** -16)
    assert bool((want[0] != 0).all())
    assert_bits_equal(out, want[0], "subnormal unscale")


def test_missing_gradient_reads_as_zero():
    a = torch.randn(3000)
    dst = torch.full((3000 + 517,), 5.0, device=DEV)
    plan = TensorPlan([a.to(DEV), None], [dst[:3000], dst[3000:]])
    plan.fused_step(1.0, 0.0)
    res = plan.result()
    out = dst.cpu()
    assert_bits_equal(out[:3000], a, "copied")
    assert bool((out[3000:] == 0).all())
    assert math.isclose(res.norm, float(a.double().norm()), rel_tol=REL)


def test_in_place_clip_matches_clip_grad_norm():
    grads = _grads([(1023,), (50000,), (7,)], torch.float32, 1.0, 1.0, seed=5)
    dev = place_in_arena(grads, DEV, 1, 3)
    plan = TensorPlan(dev, dev)
    plan.fused_step(1.0, 2.0, _lib.RG_STEP_IGNORE_OVERFLOW)
    res = plan.result()
    ref = [g.clone() for g in grads]
    norm, coef = oracle.clip_grad_norm(ref, 2.0)
    assert math.isclose(res.norm, norm, rel_tol=REL) and math.isclose(res.coef, coef, rel_tol=REL)
    for d, g in zip(dev, grads):
        assert_bits_equal(d.cpu(), g * torch.tensor(res.coef), "in-place clip")


def test_repeatable_bits():
    grads = _grads([(100003,), (4097,)], torch.float16, 1e-2, 1024.0, seed=6)
    a = _run_fused(grads, torch.float32, 1 / 1024.0, 0.1)
    b = _run_fused(grads, torch.float32, 1 / 1024.0, 0.1)
    assert a[0].norm == b[0].norm and a[0].coef == b[0].coef and a[1] == b[1]
    assert_bits_equal(a[2], b[2], "run-to-run")


@pytest.mark.parametrize("order", [0, 3, 64, 256, -1])
def test_every_write_order_gives_the_oracles_bits(order):
    """The order in which a writing pass hands its tiles to the XCDs (``rg_plan_set_write_order``, what
    ``rg_plan_tune`` chooses between) only reorders the work: with each order the two-pass step and the one-pass
    ``unscale_pack`` are held to the CPU oracle - bucket bit-exact, norms and coefficient to 1e-6."""
    g = torch.Generator().manual_seed(77)
    grads = [(torch.randn(n, generator=g) * 8).to(torch.bfloat16) for n in (100003, 5, 16384, 40000, 1, 262147)]
    srcs = place_in_arena(grads, DEV, 1, 3)
    total = sum(t.numel() for t in grads)
    offs, _ = oracle.bucket_layout([t.numel() for t in grads], ["f32"] * len(grads))
    bucket = torch.full((total + 1,), 3.0, device=DEV)[1:]
    dsts = [bucket.narrow(0, o, t.numel()) for o, t in zip(offs, grads)]
    plan = TensorPlan(srcs, dsts, chunk_elems=4096)
    plan.set_write_order(order)
    assert plan.write_order() == order
    plan.fused_step(0.125, 0.5)
    res, tn = plan.result(), plan.tensor_norms()
    want = _check_against_oracle(grads, "f32", 0.125, 0.5, res, tn, bucket.cpu())
    assert want.coef is not None
    bucket.fill_(3.0)
    plan.unscale_pack(0.125)
    res, tn = plan.result(), plan.tensor_norms()
    _check_against_oracle(grads, "f32", 0.125, math.inf, res, tn, bucket.cpu())
    plan.close()


def test_set_write_order_rejects_values_outside_its_range():
    t = torch.zeros(4096, device=DEV)
    plan = TensorPlan([t], [torch.zeros_like(t)])
    with pytest.raises(ValueError, match="order"):
        plan.set_write_order(-2)
    with pytest.raises(ValueError, match="order"):
        plan.set_write_order(1 << 20)
    plan.close()


# ----------------------------------------------------------------------------- one-pass strategy

@pytest.mark.parametrize("src_name,dst_name", [("bf16", "f32"), ("f16", "f32"), ("f32", "f32"), ("f16", "f16"), ("f32", "bf16")])
@pytest.mark.parametrize("max_norm", [0.5, 1e9])
def test_expect_no_clip_strategy_matches_the_oracle(src_name, dst_name, max_norm):
    """RG_STEP_EXPECT_NO_CLIP: one writing pass plus, only when the step clips after all, an in-place
    scale - same flag, norm (1e-6), decision and written bits as the oracle, whether or not it clips."""
    scale = 1.0 if src_name == "f32" else 256.0
    shapes = SHAPES_SMALL + [(300001,), (70000,)]
    grads = _grads(shapes, TORCH_DTYPE[src_name], 1e-1, scale, seed=21)
    for lead, gap, dst_lead in ((0, 0, 0), (1, 1, 3)):
        res, tn, out = _run_fused(grads, TORCH_DTYPE[dst_name], 1.0 / scale, max_norm, flags=_lib.RG_STEP_EXPECT_NO_CLIP,
                                  lead=lead, gap=gap, dst_lead=dst_lead)
        _check_against_oracle(grads, dst_name, 1.0 / scale, max_norm, res, tn, out)
        assert res.clipped == (1 if max_norm == 0.5 else 0)


@pytest.mark.parametrize("in_place", [False, True])
def test_gated_scale_with_several_chunks_per_block(in_place):
    """More than 16384 chunks: the in-place multiply behind a one-pass write hands each of its blocks several
    consecutive chunks.  A step that clips against expectation must still write the bits of the two-pass step,
    ragged tensor ends and the last, partly filled block of chunks included."""
    shapes = [(17_000_001,), (1023,), (20_500_003,), (1,), (2_000_000,)]     # 19,000+ chunks of 2048 elements
    grads = _grads(shapes, torch.float32, 1e-2, 1.0, seed=26)
    if in_place:
        dev = place_in_arena(grads, DEV, 1, 1)
        plan = TensorPlan(dev, dev, chunk_elems=2048)
        assert plan.plan.num_chunks > 16384 + 3
        plan.fused_step(1.0, 0.25, _lib.RG_STEP_IGNORE_OVERFLOW | _lib.RG_STEP_EXPECT_NO_CLIP)
        res = plan.result()
        assert res.clipped == 1
        coef = torch.tensor(res.coef, dtype=torch.float32)
        for g, d in zip(grads, dev):
            assert_bits_equal(d, g * coef, "clipped in place")
        plan.close()
        return
    res, tn, out = _run_fused(grads, torch.float32, 1.0, 0.25, flags=_lib.RG_STEP_EXPECT_NO_CLIP, chunk_elems=2048)
    assert res.clipped == 1
    _check_against_oracle(grads, "f32", 1.0, 0.25, res, tn, out)


def test_expect_no_clip_on_overflow_leaves_the_unscaled_values():
    grads = _grads([(5000,), (17,), (40000,)], torch.float16, 1e-2, 64.0, seed=22)
    grads[2].view(-1)[12345] = float("inf")
    res, tn, out = _run_fused(grads, torch.float32, 1 / 64.0, 0.5, flags=_lib.RG_STEP_EXPECT_NO_CLIP)
    assert res.overflow == 1 and res.skipped == 1 and res.clipped == 0 and res.coef == 1.0
    want, flag = oracle.unscale_and_check(grads, 1 / 64.0)        # written as Apex's multi_tensor_scale writes them
    assert flag == 1
    assert_bits_equal(out, torch.cat([w.flatten() for w in want]), "unscaled values on overflow")


@pytest.mark.parametrize("flags", [_lib.RG_STEP_IGNORE_OVERFLOW, _lib.RG_STEP_IGNORE_OVERFLOW | _lib.RG_STEP_EXPECT_NO_CLIP])
@pytest.mark.parametrize("max_norm", [0.25, 1e9])
def test_in_place_clip_writes_only_when_it_clips(flags, max_norm):
    """clip_grad_norm on existing gradients (dst == src, inv_scale == 1): bits as the oracle's in-place clip;
    below the bound nothing is written at all under either strategy."""
    cpu = _grads([(300001,), (5,), (70000,), (6144,)], torch.float32, 1e-2, 1.0, seed=23)
    dev = place_in_arena(cpu, DEV, 1, 1)
    plan = TensorPlan(dev, dev)
    plan.fused_step(1.0, max_norm, flags)
    res = plan.result()
    want = [g.clone() for g in cpu]
    norm, coef = oracle.clip_grad_norm(want, max_norm)
    assert math.isclose(res.norm, norm, rel_tol=REL)
    assert res.clipped == (1 if coef is not None else 0)
    for g, c, d in zip(cpu, want, dev):
        if coef is None:
            assert_bits_equal(d, g, "untouched")
        else:
            assert math.isclose(res.coef, coef, rel_tol=REL)
            assert_bits_equal(d, g * torch.tensor(res.coef, dtype=torch.float32), "clipped in place")
    plan.close()


def test_max_norm_crosses_the_boundary_as_a_c_float():
    """max_grad_norm = 0.1 is not an fp32 number: the reference narrows it at the binding
    (``src/main.cpp:339-342``) and divides in double (``src/comp/ParamStorage.cpp:723-740``)."""
    grads = _grads([(4097,), (33,)], torch.float32, 1.0, 1.0, seed=24)
    res, tn, out = _run_fused(grads, torch.float32, 1.0, 0.1)
    want = _check_against_oracle(grads, "f32", 1.0, 0.1, res, tn, out)
    import numpy as np
    assert want.coef == float(np.float32(0.1)) / (want.norm + 1e-6) and want.coef != 0.1 / (want.norm + 1e-6)
    assert math.isclose(res.coef, float(np.float32(want.coef)), rel_tol=REL)


@pytest.mark.parametrize("max_norm", [0.5, 1e9])
def test_unscale_pack_then_apply_clip_writes_the_bits_of_the_fused_step(max_norm):
    grads = _grads([(300001,), (5,), (70000,), (6144,)], torch.bfloat16, 1e-2, 65536.0, seed=25)
    srcs = place_in_arena(grads, DEV, 1, 1)
    total = sum(g.numel() for g in grads)
    bucket = torch.full((total + 3,), 7.0, dtype=torch.float32, device=DEV)[3:]
    offs, _ = oracle.bucket_layout([g.numel() for g in grads], ["f32"] * len(grads))
    dsts = [bucket.narrow(0, o, g.numel()) for o, g in zip(offs, grads)]
    plan = TensorPlan(srcs, dsts)
    with pytest.raises(ValueError, match="rg_unscale_pack"):
        plan.step_apply_clip(max_norm)                      # nothing has left sums of the destinations yet
    plan.unscale_pack(1 / 65536.0)
    plan.step_apply_clip(max_norm)
    res, tn = plan.result(), plan.tensor_norms()
    _check_against_oracle(grads, "f32", 1 / 65536.0, max_norm, res, tn, bucket.cpu())
    with pytest.raises(ValueError, match="rg_unscale_pack"):
        plan.step_apply_clip(max_norm)                      # the sums no longer describe the destinations
    plan.close()
