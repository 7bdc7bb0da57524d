"""Pins for the CPU oracle.

The reference ships no golden vectors, known-answer tests or fixtures for this path
(its tests compare two live runs at rtol 1e-2), so every oracle function is pinned here by
evidence that does not retype its formula: IEEE closed forms evaluated with numpy integer
arithmetic, library routines (numpy ``astype(float16)``, ``np.ldexp``, torch's own
``_amp_foreach_non_finite_check_and_unscale_``), float64 brute force, exact special cases
(3-4-5, constant tensors of 4^k elements) and the reference test's one structural invariant,
``segment == full.flatten()[range]`` (``test/common.py:57-63``).
"""
import math

import numpy as np
import pytest
import torch

from oracle import gradpath as oracle


# ----------------------------------------------------------------------------- helpers

def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def f32_bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int32).numpy().view(np.uint32)


def np_bf16_to_f32(bits_u16: np.ndarray) -> np.ndarray:
    return (bits_u16.astype(np.uint32) << 16).view(np.float32)


def np_f32_to_bf16_rne(x_f32: np.ndarray) -> np.ndarray:
    """Integer-arithmetic round-to-nearest-even to the top 16 bits."""
    u = x_f32.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = np.isnan(x_f32)
    r[nan] = 0x7FC0
    return r


def interesting_f32() -> torch.Tensor:
    g = torch.Generator().manual_seed(7)
    rnd = torch.randn(4000, generator=g) * torch.logspace(-30, 30, 4000)
    special = torch.tensor([0.0, -0.0, 1.0, -1.0, 65504.0, 65519.99, 65520.0, 1e-8, 6e-8, 5.96e-8, 2.98e-8,
                            6.1e-5, 6.0e-5, 3.4e38, -3.4e38, 1e-40, -1e-45, float("inf"), float("-inf"),
                            1.0 + 2 ** -8, 1.0 + 2 ** -9, 1.0 + 3 * 2 ** -9, 1.0 + 2 ** -11, 1.0 + 3 * 2 ** -11])
    return torch.cat([rnd, special])


# ----------------------------------------------------------------------------- pack

def test_consolidate_is_concatenation_per_dtype():
    g = torch.Generator().manual_seed(0)
    shapes = [(3, 5), (7,), (0,), (2, 2, 2), (1,)]
    dts = ["f32", "bf16", "f32", "bf16", "f16"]
    grads = [torch.randn(s, generator=g).to(oracle.DTYPES[d]) for s, d in zip(shapes, dts)]
    grads_with_hole = list(grads)
    grads_with_hole[3] = None           # undefined grad -> its view stays zero
    b = oracle.consolidate(grads_with_hole, [x.numel() for x in grads], dts)
    assert torch.equal(b["f32"], torch.cat([grads[0].flatten(), grads[2].flatten()]))
    assert torch.equal(b["bf16"], torch.cat([grads[1].flatten(), torch.zeros(8, dtype=torch.bfloat16)]))
    assert torch.equal(b["f16"], grads[4].flatten())


def test_zero_staging_pack_pads_with_zero_and_widens_half_only():
    x = torch.arange(1, 11, dtype=torch.float16)
    buf = oracle.zero_staging_pack(x, 4, to_fp32=True)       # unit = 8 * 4 = 32
    assert buf.dtype == torch.float32 and buf.numel() == 32
    assert torch.equal(buf[:10], x.float()) and bool((buf[10:] == 0).all())
    assert oracle.zero_staging_pack(x, 4, to_fp32=False).dtype == torch.float16
    # the reference widens Half only (ParamStorage.cpp:485-488), bf16 stays bf16
    assert oracle.zero_staging_pack(x.to(torch.bfloat16), 2, to_fp32=True).dtype == torch.bfloat16
    g = torch.zeros(10)
    oracle.zero_copy_back(g, torch.full((8,), 2.0), 8)        # last rank: min(8, 10 - 8) = 2 elements
    assert g.tolist() == [0.0] * 8 + [2.0, 2.0]
    oracle.zero_copy_back(g, torch.full((8,), 3.0), 16)       # nothing left: no-op
    assert g.tolist() == [0.0] * 8 + [2.0, 2.0]


# ----------------------------------------------------------------------------- unscale + flag

@pytest.mark.parametrize("k", [16, 12, 0, 3])
def test_unscale_by_power_of_two_is_exponent_shift(k):
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(5000, generator=g) * 1e-2 * 2.0 ** k).to(torch.bfloat16)
    x[:4] = torch.tensor([1e-36, -3e-37, 2e-38, 0.0]).to(torch.bfloat16)   # products become fp32 subnormals
    out, flag = oracle.unscale_and_check([x], 2.0 ** -k)
    want = np.ldexp(np_bf16_to_f32(bf16_bits(x)), -k).astype(np.float32)
    assert flag == 0
    assert np.array_equal(f32_bits(out[0]), want.view(np.uint32))
    assert (want[:3] != 0).all()


@pytest.mark.parametrize("inv_scale", [1.0 / 65536.0, 1.0 / 3.0, 0.7])
def test_unscale_matches_torch_amp_foreach(inv_scale):
    g = torch.Generator().manual_seed(2)
    xs = [torch.randn(n, generator=g) * 100.0 for n in (1, 17, 4096)]
    want = [x.clone() for x in xs]
    found = torch.zeros(1)
    torch._amp_foreach_non_finite_check_and_unscale_(want, found, torch.tensor(inv_scale))
    out, flag = oracle.unscale_and_check(xs, inv_scale)
    assert flag == 0 and found.item() == 0.0
    for a, b in zip(out, want):
        assert np.array_equal(f32_bits(a), f32_bits(b))
    xs[1][3] = float("inf")
    found.zero_()
    torch._amp_foreach_non_finite_check_and_unscale_([x.clone() for x in xs], found, torch.tensor(inv_scale))
    assert found.item() == 1.0 and oracle.unscale_and_check(xs, inv_scale)[1] == 1


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_overflow_flag_special_cases(dtype):
    base = [torch.ones(5, dtype=dtype), torch.ones(64, dtype=dtype), torch.zeros(0, dtype=dtype)]
    assert oracle.unscale_and_check(base, 0.5)[1] == 0
    for bad in (float("inf"), float("-inf"), float("nan")):
        for ti, idx in ((0, 0), (1, 63), (1, 31)):
            xs = [b.clone() for b in base]
            xs[ti][idx] = bad
            assert oracle.unscale_and_check(xs, 0.5)[1] == 1, (bad, ti, idx)
    fmax = torch.finfo(dtype).max
    assert oracle.unscale_and_check([torch.full((3,), fmax, dtype=dtype)], 1.0)[1] == 0
    # the flag looks at the input: a finite input stays unflagged whatever the product does
    assert oracle.unscale_and_check([torch.full((3,), 3e38)], 4.0)[1] == 0


# ----------------------------------------------------------------------------- casts

def test_cast_f32_to_f16_is_ieee_rne():
    x = interesting_f32()
    got = oracle.cast(x, torch.float16).view(torch.int16).numpy().view(np.uint16)
    with np.errstate(over="ignore"):
        want = x.numpy().astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)
    assert got[list(x).index(65520.0)] == 0x7C00 and got[list(x).index(65504.0)] == 0x7BFF


def test_cast_f32_to_bf16_is_rne_on_the_top_16_bits():
    x = interesting_f32()
    assert np.array_equal(bf16_bits(oracle.cast(x, torch.bfloat16)), np_f32_to_bf16_rne(x.numpy()))
    ties = torch.tensor([0x3F808000, 0x3F818000, 0x3F80FFFF, 0x3F808001], dtype=torch.int64).to(torch.int32).view(torch.float32)
    assert bf16_bits(oracle.cast(ties, torch.bfloat16)).tolist() == [0x3F80, 0x3F82, 0x3F81, 0x3F81]
    assert torch.isnan(oracle.cast(torch.tensor([float("nan")]), torch.bfloat16)).all()


def test_widening_is_exact():
    h = torch.arange(-2 ** 15, 2 ** 15, dtype=torch.int32).to(torch.int16)          # every bit pattern
    f16 = h.view(torch.float16)
    want = f16.numpy().astype(np.float32)
    got = oracle.cast(f16, torch.float32).numpy()
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    b = h.view(torch.bfloat16)
    got = oracle.cast(b, torch.float32)
    want = np_bf16_to_f32(bf16_bits(b))
    ok = ~np.isnan(want)
    assert np.array_equal(f32_bits(got)[ok], want.view(np.uint32)[ok])


def test_master_copy_back_roundtrip():
    g = torch.Generator().manual_seed(3)
    model = [torch.randn(100, generator=g).to(torch.bfloat16), torch.randn(7, generator=g).to(torch.bfloat16)]
    masters = oracle.master_from_model(model)
    assert all(m.dtype == torch.float32 for m in masters)
    masters[0].add_(1e-3)
    want0 = np_f32_to_bf16_rne(masters[0].numpy())
    keep1 = bf16_bits(model[1]).copy()
    oracle.master_copy_back(masters, model)
    assert np.array_equal(bf16_bits(model[0]), want0) and np.array_equal(bf16_bits(model[1]), keep1)


# ----------------------------------------------------------------------------- norm + clip

def test_norm_closed_forms():
    # constant tensors of 4^k elements: norm = |c| * 2^k exactly
    assert oracle.grad_global_l2_norm([torch.full((4096,), 0.5)]) == 32.0
    assert oracle.grad_global_l2_norm([torch.full((64, 64), -0.25, dtype=torch.bfloat16)]) == 16.0
    # 3-4-5 over two tensors, an undefined grad and an empty tensor in between
    a = torch.zeros(10); a[3] = 3.0
    b = torch.zeros(1000, dtype=torch.float16); b[999] = -4.0
    assert oracle.grad_global_l2_norm([a, None, torch.zeros(0), b]) == 5.0
    assert oracle.per_tensor_norms([a, None, b]) == [3.0, None, 4.0]


def test_norm_against_float64_brute_force_and_fp32_rounding_point():
    g = torch.Generator().manual_seed(4)
    xs = [torch.randn(n, generator=g) * s for n, s in ((100003, 1e-3), (17, 5.0), (2 ** 20, 1e-2))]
    per = oracle.per_tensor_norms(xs)
    for x, n in zip(xs, per):
        exact = float(np.linalg.norm(x.numpy().astype(np.float64)))
        assert n == float(np.float32(exact))                       # rounded to fp32 exactly once
    total = oracle.grad_global_l2_norm(xs)
    exact_total = math.sqrt(sum(float(np.linalg.norm(x.numpy().astype(np.float64))) ** 2 for x in xs))
    assert math.isclose(total, exact_total, rel_tol=1e-7)
    # the literal ATen CPU op agrees only loosely (its fp32 accumulation drifts with size)
    for a, b in zip(oracle.per_tensor_norms_aten(xs), per):
        assert math.isclose(a, b, rel_tol=1e-4)


def test_clip_threshold_eps_and_float_narrowing():
    # eps is added before the strict compare (ParamStorage.cpp:723-725)
    assert oracle.clip_coefficient(5.0, 5.0) == 5.0 / (5.0 + 1e-6)
    assert oracle.clip_coefficient(5.0, 5.5) is None
    assert oracle.clip_coefficient(0.0, 1.0) is None
    assert oracle.clip_coefficient(float("nan"), 1.0) is None
    assert oracle.clip_coefficient(float("inf"), 1.0) == 0.0
    # max_norm crosses the binding as a C float (src/main.cpp:339-342)
    assert oracle.clip_coefficient(1.0, 0.1) == float(np.float32(0.1)) / (1.0 + 1e-6)
    assert oracle.clip_coefficient(1.0, 0.1) != 0.1 / (1.0 + 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_clip_multiplies_by_the_coefficient_narrowed_to_fp32(dtype):
    g = torch.Generator().manual_seed(5)
    xs = [(torch.randn(n, generator=g)).to(dtype) for n in (1000, 3)]
    before = [x.clone() for x in xs]
    norm, coef = oracle.clip_grad_norm(xs, 0.25)
    assert coef is not None and math.isclose(norm, math.sqrt(sum(float(b.double().square().sum()) for b in before)), rel_tol=1e-6)
    c32 = np.float32(coef)
    for x, b in zip(xs, before):
        prod = (b.float().numpy() * c32).astype(np.float32)
        if dtype == torch.float32:
            assert np.array_equal(f32_bits(x), prod.view(np.uint32))
        elif dtype == torch.bfloat16:
            assert np.array_equal(bf16_bits(x), np_f32_to_bf16_rne(prod))
        else:
            assert np.array_equal(x.view(torch.int16).numpy().view(np.uint16), prod.astype(np.float16).view(np.uint16))
    # below the bound nothing is touched
    ys = [b.clone() for b in before]
    assert oracle.clip_grad_norm(ys, 1e6)[1] is None and all(torch.equal(y, b) for y, b in zip(ys, before))


def test_fused_step_known_answer():
    # bf16 gradients scaled by 2^16: four 2s (norm 4) and one 3 (norm 3) -> global norm 5
    S = 65536.0
    g = [torch.full((4,), 2.0 * S, dtype=torch.bfloat16), torch.full((1,), 3.0 * S, dtype=torch.bfloat16)]
    r = oracle.fused_step(g, ["f32", "f32"], 2.0 ** -16, 1.0)
    assert r.overflow == 0 and r.tensor_norms == [4.0, 3.0] and r.norm == 5.0 and r.coef == 1.0 / (5.0 + 1e-6)
    c = np.float32(r.coef)
    assert r.buckets["f32"].tolist() == [float(np.float32(2.0) * c)] * 4 + [float(np.float32(3.0) * c)]
    r = oracle.fused_step(g, ["f32", "f32"], 2.0 ** -16, 8.0)
    assert r.coef is None and r.buckets["f32"].tolist() == [2.0] * 4 + [3.0]
    # sqrt(12) is not an fp32 number: the per-tensor rounding to fp32 is visible in the total
    r = oracle.fused_step([torch.full((3,), 2.0), torch.full((1,), 2.0)], ["f32", "f32"], 1.0, 100.0)
    assert r.norm != 4.0 and math.isclose(r.norm, 4.0, rel_tol=1e-7)
    g[0][1] = float("nan")
    r = oracle.fused_step(g, ["f32", "f32"], 2.0 ** -16, 1.0)
    assert r.overflow == 1 and r.coef is None           # skipped: no clip


# ----------------------------------------------------------------------------- dist params

@pytest.mark.parametrize("nranks", [1, 2, 4, 8])
@pytest.mark.parametrize("shape,dtype", [((10,), torch.float32), ((3, 7), torch.float16), ((5,), torch.bfloat16),
                                         ((1000,), torch.float16), ((0,), torch.float32), ((129, 3), torch.float32)])
def test_dist_param_segments_tile_the_tensor_and_load_restores_it(nranks, shape, dtype):
    g = torch.Generator().manual_seed(6)
    full = torch.randn(shape, generator=g).to(dtype)
    ranks = [oracle.DistParamOracle(r, nranks) for r in range(nranks)]
    parts = [o.store(11, full) for o in ranks]
    flat = full.flatten()
    for o, part in zip(ranks, parts):
        lo, hi = o.get_range(11)
        assert torch.equal(part, flat[lo:hi])                       # test/common.py:57-63
    assert torch.equal(torch.cat(parts), flat)
    assert torch.equal(oracle.DistParamOracle.load(11, ranks), full)
    # set(): every rank takes its own slice of a new full tensor
    new = torch.randn(shape, generator=g).to(dtype)
    for o in ranks:
        o.set(11, new)
    assert torch.equal(oracle.DistParamOracle.load(11, ranks), new)
    # dtype change keeps the layout (segment sizes in elements)
    for o in ranks:
        o.set_scalar_type(11, torch.float32)
    assert torch.equal(oracle.DistParamOracle.load(11, ranks), new.float())


def test_align_buffer_keeps_values_and_zero_pads():
    p = torch.arange(1, 11, dtype=torch.float16).view(2, 5)
    buf = oracle.align_buffer(p, 8)                                  # unit 64
    assert buf.numel() == 64 and torch.equal(buf[:10], p.flatten()) and bool((buf[10:] == 0).all())


# ----------------------------------------------------------------------------- loss scaler wrapper

def test_patched_update_scale_cases():
    # no overflow anywhere: nothing changes, step is not skipped
    s = oracle.LossScalerState(loss_scale=1024.0, unskipped=5)
    assert oracle.patched_update_scale(s, False) is False and s.loss_scale == 1024.0 and s.unskipped == 6
    # local overflow: own update halves, wrapper stores int(min) and zeroes the counter
    s = oracle.LossScalerState(loss_scale=1024.0, unskipped=5)
    assert oracle.patched_update_scale(s, True) is True and s.loss_scale == 512 and s.unskipped == 0
    # overflow on another rank only: this rank adopts the smaller scale and skips too
    s = oracle.LossScalerState(loss_scale=1024.0, unskipped=5)
    assert oracle.patched_update_scale(s, False, other_flags=[1], other_scales=[256]) is True
    assert s.loss_scale == 256 and s.unskipped == 0
    # the minimum wins even when the local scale is smaller
    s = oracle.LossScalerState(loss_scale=128.0)
    assert oracle.patched_update_scale(s, False, other_flags=[1], other_scales=[512]) is True and s.loss_scale == 128


def test_update_scale_hand_written_sequences():
    """Apex's published schedule, pinned by literals worked out by hand (not by a second typing
    of the formula): (had_overflow) -> (skip, loss_scale, unskipped) after the call."""
    s = oracle.LossScalerState(loss_scale=256.0, scale_window=3, min_loss_scale=None, max_loss_scale=512.0)
    steps = [
        (True,  (True, 128.0, 0)),    # overflow: halve, counter to zero, skip
        (False, (False, 128.0, 1)),
        (False, (False, 128.0, 2)),
        (False, (False, 256.0, 0)),   # third clean step in a row: double, counter to zero
        (False, (False, 256.0, 1)),
        (True,  (True, 128.0, 0)),    # an overflow forgets the clean steps counted so far
        (True,  (True, 64.0, 0)),
        (False, (False, 64.0, 1)),
        (False, (False, 64.0, 2)),
        (False, (False, 128.0, 0)),
        (False, (False, 128.0, 1)),
        (False, (False, 128.0, 2)),
        (False, (False, 256.0, 0)),
        (False, (False, 256.0, 1)),
        (False, (False, 256.0, 2)),
        (False, (False, 512.0, 0)),
        (False, (False, 512.0, 1)),
        (False, (False, 512.0, 2)),
        (False, (False, 512.0, 0)),   # capped at max_loss_scale; the counter still restarts
    ]
    for i, (had, want) in enumerate(steps):
        assert (s.update_scale(had), s.loss_scale, s.unskipped) == want, i
    # floor: with min_loss_scale the scale stops there, without one it keeps halving below 1
    s = oracle.LossScalerState(loss_scale=4.0, min_loss_scale=2.0)
    assert [(s.update_scale(True), s.loss_scale) for _ in range(3)] == [(True, 2.0), (True, 2.0), (True, 2.0)]
    s = oracle.LossScalerState(loss_scale=2.0, min_loss_scale=None)
    assert [(s.update_scale(True), s.loss_scale) for _ in range(3)] == [(True, 1.0), (True, 0.5), (True, 0.25)]
    # defaults of amp.initialize: 2^16 start, 2000-step window, 2^24 cap
    s = oracle.LossScalerState()
    assert (s.loss_scale, s.scale_window, s.max_loss_scale, s.min_loss_scale) == (65536.0, 2000, 16777216.0, None)
    for _ in range(1999):
        assert s.update_scale(False) is False
    assert (s.loss_scale, s.unskipped) == (65536.0, 1999)
    assert s.update_scale(False) is False and (s.loss_scale, s.unskipped) == (131072.0, 0)
    # a static scale neither moves nor skips, overflow or not
    s = oracle.LossScalerState(loss_scale=128.0, dynamic=False, scale_window=2)
    assert [s.update_scale(h) for h in (True, False, True, False)] == [False] * 4 and s.loss_scale == 128.0


# ----------------------------------------------------------------------------- timed CPU baseline

def _bucket_views(grads, dtype):
    n = sum(g.numel() for g in grads)
    bucket = torch.full((n,), 7.0, dtype=dtype)        # stale values: every element must be overwritten
    views, off = [], 0
    for g in grads:
        views.append(bucket.narrow(0, off, g.numel()).view(g.shape))
        off += g.numel()
    return bucket, views


@pytest.mark.parametrize("src_dtype,inv_scale", [(torch.bfloat16, 2.0 ** -16), (torch.float16, 2.0 ** -12),
                                                 (torch.float32, 1.0)])
def test_reference_step_cpu_does_the_work_of_fused_step(src_dtype, inv_scale):
    """The timed CPU leg against the oracle's fused step on the same mixed list: flag exact,
    norm within 1e-4 (ATen's fp32 accumulation), coefficient consistent with its own norm, and
    the bucket it leaves bit-exact given that coefficient."""
    gen = torch.Generator().manual_seed(11)
    shapes = [(257, 33), (1,), (4096,), (3, 5, 7), (0,), (63,), (1000, 17)]
    grads = [(torch.randn(s, generator=gen) * 1e-2 / inv_scale).to(src_dtype) for s in shapes]
    for max_norm in (1.0, 1e6):                        # clips / does not clip
        bucket, views = _bucket_views(grads, torch.float32)
        ovf, norm, coef = oracle.reference_step_cpu(grads, views, inv_scale, max_norm)
        want = oracle.fused_step(grads, ["f32"] * len(grads), inv_scale, max_norm)
        assert ovf == want.overflow == 0
        assert math.isclose(norm, want.norm, rel_tol=1e-4)
        assert (coef is None) == (want.coef is None) == (max_norm == 1e6)
        unscaled = oracle.fused_step(grads, ["f32"] * len(grads), inv_scale, math.inf).buckets["f32"]
        if coef is not None:
            assert math.isclose(coef, want.coef, rel_tol=1e-4)
            assert coef == float(np.float32(max_norm)) / (norm + 1e-6)
            unscaled = (unscaled.numpy() * np.float32(coef)).astype(np.float32)
            assert np.array_equal(f32_bits(bucket), unscaled.view(np.uint32))
        else:
            assert np.array_equal(f32_bits(bucket), f32_bits(unscaled))
    # overflow: flagged, nothing clipped (the step is skipped)
    bad = [g.clone() for g in grads]
    bad[3].view(-1)[104] = float("inf")
    bad[6].view(-1)[0] = float("nan")
    bucket, views = _bucket_views(bad, torch.float32)
    ovf, norm, coef = oracle.reference_step_cpu(bad, views, inv_scale, 1.0)
    want = oracle.fused_step(bad, ["f32"] * len(bad), inv_scale, 1.0)
    assert ovf == want.overflow == 1 and coef is None and want.coef is None
    finite = torch.isfinite(bucket)
    assert int((~finite).sum()) == 2
    assert torch.equal(bucket[finite], want.buckets["f32"][finite])     # written unscaled, unclipped


# ----------------------------------------------------------------------------- accumulation

def test_unscale_accumulate_is_two_roundings():
    g = torch.Generator().manual_seed(8)
    master = torch.randn(3000, generator=g)
    model = (torch.randn(3000, generator=g) * 100).to(torch.float16)
    want = (master.numpy().astype(np.float32)
            + (model.numpy().astype(np.float32) * np.float32(0.37)).astype(np.float32)).astype(np.float32)
    m = master.clone()
    assert oracle.unscale_accumulate([m, torch.zeros(2)], [model, None], 0.37) == 0
    assert np.array_equal(f32_bits(m), want.view(np.uint32))
    # exact case: accumulating x/2 twice onto zero gives x
    z = torch.zeros(3000)
    oracle.unscale_accumulate([z], [model], 0.5)
    oracle.unscale_accumulate([z], [model], 0.5)
    assert torch.equal(z, model.float())
    model[5] = float("nan")
    assert oracle.unscale_accumulate([master.clone()], [model], 0.5) == 1


def test_sum_clone_grads_order_and_rounding():
    # fp16: (a + b) + c is rounded after every addition, in clone order
    a = torch.tensor([2048.0, 1.0], dtype=torch.float16)
    b = torch.tensor([1.0, 1.0], dtype=torch.float16)
    c = torch.tensor([1.0, -2.0], dtype=torch.float16)
    grads = [None]
    clones = [[a.clone(), b.clone(), c.clone()]]
    oracle.sum_clone_grads(grads, clones)
    # 2048 + 1 = 2049 -> rounds to 2048 (ulp 2), again + 1 -> 2048; a sum in higher precision would give 2050
    assert grads[0].tolist() == [2048.0, 0.0]
    assert all(float(g.abs().sum()) == 0.0 for g in clones[0])           # clone grads are cleared
    have = [torch.tensor([10.0, 10.0], dtype=torch.float16)]
    oracle.sum_clone_grads(have, [[a.clone(), None, c.clone()]])
    assert have[0].tolist() == [2058.0, 9.0]                              # grad_sum = [2048, -1] is added to the existing gradient
