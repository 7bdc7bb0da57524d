"""rg_fused_step_static - the fused step over one tensor pair with no plan and no allocation -
through the C ABI, against rg_fused_step on a one-tensor plan: result block and every written
bit equal, on two calls in a row, the second with a smaller input (the library's fixed working
array still holds the first call's partial sums then).  Collected last on purpose."""
import ctypes as C

import pytest
import torch

from rannc_amd import _lib
from rannc_amd.multi_tensor import TensorPlan, stream_handle

from .helpers import assert_bits_equal

pytestmark = pytest.mark.gpu

CODES = {torch.float32: _lib.RG_F32, torch.float16: _lib.RG_F16, torch.bfloat16: _lib.RG_BF16}


def _static_step(src, dst, inv_scale, max_norm, flags=_lib.RG_STEP_DEFAULT):
    """-> rg_step_result read back from the caller's device memory."""
    dev = src.device
    res_dev = torch.full((3,), -1, dtype=torch.int64, device=dev)           # 24 bytes, 8-byte aligned
    _lib.fused_step_static(src.data_ptr(), dst.data_ptr(), src.numel(), CODES[src.dtype], CODES[dst.dtype],
                           inv_scale, max_norm, flags, res_dev.data_ptr(), dev.index, stream_handle(dev))
    raw = res_dev.cpu().numpy().tobytes()
    return _lib.StepResult.from_buffer_copy(raw)


def _plan_step(src, dst, inv_scale, max_norm, flags=_lib.RG_STEP_DEFAULT):
    plan = TensorPlan([src], [dst])
    plan.fused_step(inv_scale, max_norm, flags)
    res = plan.result()
    plan.close()
    return res


def _same_result(a, b):
    assert (a.overflow, a.clipped, a.skipped) == (b.overflow, b.clipped, b.skipped)
    if a.norm == a.norm or b.norm == b.norm:
        assert C.c_double(a.norm).value == C.c_double(b.norm).value, (a.norm, b.norm)
    assert a.coef == b.coef, (a.coef, b.coef)


def _case(n, sdt, ddt, lead, inv_scale, max_norm, dev, gen, poison=None, flags=_lib.RG_STEP_DEFAULT):
    src = (torch.randn(n + lead, generator=gen, device=dev) * (1e-2 / inv_scale)).to(sdt)[lead:]
    if poison is not None:
        src[poison] = float("inf")
    want_dst = torch.full((n + 3,), 5.0, dtype=ddt, device=dev)[3:]
    got_dst = torch.full((n + 3,), 5.0, dtype=ddt, device=dev)[3:]
    want = _plan_step(src, want_dst, inv_scale, max_norm, flags)
    got = _static_step(src, got_dst, inv_scale, max_norm, flags)
    torch.cuda.synchronize()
    _same_result(got, want)
    assert_bits_equal(got_dst, want_dst, f"static vs plan, n={n} {sdt}->{ddt}")
    return got


def test_static_step_matches_the_plan_twice_in_a_row_second_call_smaller():
    dev = torch.device("cuda", 0)
    gen = torch.Generator(device=dev).manual_seed(5)
    big = _case(40_000_003, torch.bfloat16, torch.float32, 1, 2.0 ** -16, 1.0, dev, gen)
    assert big.clipped == 1 and big.overflow == 0 and big.norm > 1.0
    small = _case(70_001, torch.bfloat16, torch.float32, 3, 2.0 ** -16, 1.0, dev, gen)
    assert small.clipped == 1 and small.norm < big.norm
    # further shapes on the same array: in place fp32, fp16 -> fp16 without clipping, one element, nothing
    _case(5_000_000, torch.float16, torch.float16, 0, 2.0 ** -12, 1e9, dev, gen)
    _case(1, torch.float32, torch.float32, 0, 1.0, 1.0, dev, gen)
    _case(0, torch.float32, torch.float32, 0, 1.0, 1.0, dev, gen)
    # overflow: flagged and skipped (destination untouched), or written when asked to
    r = _case(1_000_000, torch.float16, torch.float32, 1, 2.0 ** -12, 1.0, dev, gen, poison=777_777)
    assert r.overflow == 1 and r.skipped == 1
    r = _case(1_000_000, torch.float16, torch.float32, 1, 2.0 ** -12, 1.0, dev, gen, poison=0,
              flags=_lib.RG_STEP_WRITE_ON_OVERFLOW)
    assert r.overflow == 1


def test_static_step_fp32_sources_large_enough_for_the_largest_chunks():
    """fp32 sources switch to chunks of 8192 elements (32 KiB of source, as for 16-bit types) once the tensor is
    large enough for the cap to bind - above about 16.8 M elements; the one-tensor plan does the same, and norm,
    coefficient and every written bit must still agree."""
    dev = torch.device("cuda", 0)
    gen = torch.Generator(device=dev).manual_seed(7)
    r = _case(35_000_003, torch.float32, torch.float32, 1, 2.0 ** -8, 1.0, dev, gen)
    assert r.clipped == 1
    r = _case(20_000_001, torch.float32, torch.float16, 0, 2.0 ** -8, 1.0, dev, gen)
    assert r.clipped == 1
    _case(9_000_000, torch.float32, torch.bfloat16, 2, 2.0 ** -8, 1e9, dev, gen)     # smaller again, no clip


def test_static_step_in_place_clip():
    dev = torch.device("cuda", 0)
    gen = torch.Generator(device=dev).manual_seed(6)
    g = torch.randn(3_000_001, generator=gen, device=dev)
    want = g.clone()
    w = _plan_step(want, want, 1.0, 0.5, _lib.RG_STEP_IGNORE_OVERFLOW)
    r = _static_step(g, g, 1.0, 0.5, _lib.RG_STEP_IGNORE_OVERFLOW)
    torch.cuda.synchronize()
    _same_result(r, w)
    assert_bits_equal(g, want, "in-place clip")


def test_static_step_rejects_what_it_cannot_hold():
    dev = torch.device("cuda", 0)
    t = torch.zeros(8, device=dev)
    # the limit is 8 GiB of source: 2^32 elements of a 16-bit type, 2^31 of fp32
    with pytest.raises(ValueError, match="exceed the limit"):
        _lib.fused_step_static(t.data_ptr(), t.data_ptr(), _lib.RG_STATIC_MAX_NUMEL + 1, _lib.RG_F16, _lib.RG_F16,
                               1.0, 1.0, 0, None, 0, 0)
    with pytest.raises(ValueError, match="exceed the limit"):
        _lib.fused_step_static(t.data_ptr(), t.data_ptr(), _lib.RG_STATIC_MAX_NUMEL // 2 + 1, _lib.RG_F32, _lib.RG_F32,
                               1.0, 1.0, 0, None, 0, 0)
    with pytest.raises(ValueError, match="inv_scale"):
        _lib.fused_step_static(t.data_ptr(), t.data_ptr(), 8, _lib.RG_F32, _lib.RG_F32, 0.0, 1.0, 0, None, 0, 0)
    with pytest.raises(ValueError, match="changes dtype"):
        _lib.fused_step_static(t.data_ptr(), t.data_ptr(), 8, _lib.RG_F32, _lib.RG_F16, 1.0, 1.0, 0, None, 0, 0)
