"""The five benchmark configurations on the GPU.

* against the CPU oracle at sizes it finishes in seconds (``c1_mlp`` in full, the others with every
  tensor's dim 0 scaled down, same tensor list and dtypes);
* at full size through properties that do not depend on size: the unscale by a power of two is
  an exact exponent shift, so the packed bucket must equal ``(x.float() * inv) * coef``
  evaluated by torch on the device bit for bit; the norm must match a float64 accumulation;
  the flag must follow the injected non-finite values; a second run must give the same bits;
  unflatten -> cast -> repack of the ZeRO flat buffer must be the identity.
torch-on-GPU is used here only as a checker of the HIP library's output.
"""
import math

import pytest
import torch

from oracle import gradpath as oracle
from rannc_amd import _lib
from rannc_amd.multi_tensor import TensorPlan
from rannc_amd.workloads import make_grads, step_config, zero_segment_sizes
from tests.helpers import TORCH_DTYPE, assert_bits_equal

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
REL = 1e-6


def _bucket_views(grads, dtype):
    n = sum(g.numel() for g in grads)
    bucket = torch.zeros(n, dtype=dtype, device=DEV)
    views, off = [], 0
    for g in grads:
        views.append(bucket.narrow(0, off, g.numel()))
        off += g.numel()
    return bucket, views


@pytest.mark.parametrize("key,scale", [("c1_mlp", 1.0), ("c2_bert_large", 0.01), ("c3_bert_enlarged", 0.002),
                                       ("c3_bert_enlarged_overflow", 0.002), ("c4_resnet152x2", 0.02)])
def test_config_against_oracle(key, scale):
    cfg = step_config(key)
    grads_cpu, injected = make_grads(cfg, seed=0, device="cpu", scale_numel=scale)
    ddt = TORCH_DTYPE[cfg.bucket_dtype]
    dev = [g.to(DEV) for g in grads_cpu]
    bucket, views = _bucket_views(dev, ddt)
    bucket.fill_(7.0)
    plan = TensorPlan(dev, views)
    plan.fused_step(cfg.inv_scale, cfg.max_norm)
    res = plan.result()
    tn = plan.tensor_norms()
    want = oracle.fused_step(grads_cpu, [cfg.bucket_dtype] * len(grads_cpu), cfg.inv_scale, cfg.max_norm)
    assert res.overflow == want.overflow == (1 if injected else 0)
    if want.overflow:
        assert res.skipped == 1 and bool((bucket == 7.0).all())
        return
    assert math.isclose(res.norm, want.norm, rel_tol=REL)
    for a, b in zip(tn, want.tensor_norms):
        assert math.isclose(a, b, rel_tol=REL, abs_tol=1e-30)
    assert res.clipped == 1 and want.coef is not None and math.isclose(res.coef, want.coef, rel_tol=REL)
    unscaled = oracle.fused_step(grads_cpu, [cfg.bucket_dtype] * len(grads_cpu), cfg.inv_scale, math.inf).buckets[cfg.bucket_dtype]
    unscaled.mul_(float(res.coef))
    assert_bits_equal(bucket.cpu(), unscaled, key)
    plan.close()


def test_c1_pack_then_unflatten_back():
    """Configuration 1 end to end: the eight MLP gradients packed into one fp32 bucket by the fused step, then the
    bucket unflattened back into one separately allocated tensor per parameter - each must hold exactly the slice
    of the oracle's bucket that belongs to it."""
    cfg = step_config("c1_mlp")
    grads_cpu, _ = make_grads(cfg, seed=0, device="cpu")
    ddt = TORCH_DTYPE[cfg.bucket_dtype]
    dev = [g.to(DEV) for g in grads_cpu]
    bucket, views = _bucket_views(dev, ddt)
    pack = TensorPlan(dev, views)
    pack.fused_step(cfg.inv_scale, cfg.max_norm)
    res = pack.result()
    outs = [torch.full(g.shape, 7.0, dtype=ddt, device=DEV) for g in dev]
    back = TensorPlan(views, outs)
    back.scale_cast(1.0)
    want = oracle.fused_step(grads_cpu, [cfg.bucket_dtype] * len(grads_cpu), cfg.inv_scale, math.inf).buckets[cfg.bucket_dtype]
    want.mul_(float(res.coef))
    off = 0
    for g, o in zip(grads_cpu, outs):
        assert o.shape == g.shape
        assert_bits_equal(o.cpu().view(-1), want.narrow(0, off, g.numel()), "unflattened")
        off += g.numel()
    assert off == want.numel()
    pack.close()
    back.close()


def _full_size_check(key):
    cfg = step_config(key)
    grads, injected = make_grads(cfg, seed=0, device=DEV)
    ddt = TORCH_DTYPE[cfg.bucket_dtype]
    bucket, views = _bucket_views(grads, ddt)
    plan = TensorPlan(grads, views)
    plan.fused_step(cfg.inv_scale, cfg.max_norm)
    res = plan.result()
    tn = torch.tensor(plan.tensor_norms(), dtype=torch.float64)
    assert res.overflow == (1 if injected else 0)
    if injected:
        assert res.skipped == 1 and res.clipped == 0
        plan.fused_step(cfg.inv_scale, cfg.max_norm, _lib.RG_STEP_WRITE_ON_OVERFLOW)
        assert plan.result().overflow == 1
        for g, v in zip(grads, views):
            want = (g.float() * cfg.inv_scale).view(-1)
            assert torch.equal(torch.nan_to_num(v, nan=1.5, posinf=2.5, neginf=-2.5),
                               torch.nan_to_num(want, nan=1.5, posinf=2.5, neginf=-2.5))
        return
    # norm against a float64 accumulation on the device
    sq = torch.stack([torch.linalg.vector_norm(g.float() * cfg.inv_scale, dtype=torch.float64) for g in grads]).cpu()
    assert torch.allclose(tn, sq.float().double(), rtol=REL, atol=0)
    total = math.sqrt(float((sq.float().double() ** 2).sum()))
    assert math.isclose(res.norm, total, rel_tol=REL)
    g = res.norm + 1e-6
    assert res.clipped == (1 if g > cfg.max_norm else 0)
    if res.clipped:
        assert math.isclose(res.coef, cfg.max_norm / g, rel_tol=REL)
    coef = torch.tensor(res.coef, dtype=torch.float32, device=DEV)
    inv = torch.tensor(cfg.inv_scale, dtype=torch.float32, device=DEV)
    for gr, v in zip(grads, views):
        want_v = ((gr.float() * inv) * coef).to(ddt).view(-1)
        assert bool(torch.equal(v, want_v)), "bucket differs from (x * inv) * coef"
    # same bits on a second run
    first = bucket.clone()
    plan.fused_step(cfg.inv_scale, cfg.max_norm)
    r2 = plan.result()
    assert torch.equal(first, bucket) and r2.norm == res.norm and r2.coef == res.coef
    plan.close()


@pytest.mark.parametrize("key", ["c2_bert_large", "c4_resnet152x2", "c3_bert_enlarged", "c3_bert_enlarged_overflow"])
def test_config_full_size_properties(key):
    _full_size_check(key)
    torch.cuda.empty_cache()


def test_c2_master_copy_back_full_size():
    cfg = step_config("c2_bert_large")
    g = torch.Generator(device=DEV).manual_seed(1)
    masters = [torch.randn(s, generator=g, device=DEV) for _, s in cfg.params]
    models = [torch.zeros(m.shape, dtype=torch.bfloat16, device=DEV) for m in masters]
    TensorPlan(masters, models).scale_cast(1.0)
    for m, p in zip(masters, models):
        assert bool(torch.equal(p, m.to(torch.bfloat16)))


@pytest.mark.parametrize("total,nseg", [(3_000_001, 64), (10_000_000_000, 4096)])
def test_c5_zero_flat_buffer_roundtrip(total, nseg):
    """Flat fp16 buffer -> parameter segments (unflatten) -> fp32 masters (cast) -> fp16 -> flat (repack):
    bit-exact identity, at a small size and at the full 10 B elements (20 GB flat + 20 GB params + 40 GB masters)."""
    free, _ = torch.cuda.mem_get_info()
    if total * 10 > free * 0.9:
        pytest.skip(f"needs {total * 10 / 1e9:.0f} GB of device memory")
    sizes = zero_segment_sizes(nseg, total, seed=0)
    n = sum(sizes)
    assert all(s % 2 == 1 for s in sizes)
    flat = torch.empty(n, dtype=torch.float16, device=DEV)
    # cheap on-device pattern covering every fp16 bit pattern except NaNs (exponent 31 masked out)
    step = 1 << 28
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        idx = torch.arange(lo, hi, device=DEV, dtype=torch.int64)
        bits = ((idx * 2654435761) >> 7) & 0xFFFF
        bits = torch.where((bits & 0x7C00) == 0x7C00, bits & 0x83FF, bits)
        flat[lo:hi] = bits.to(torch.int16).view(torch.float16)
        del idx, bits
    offs = [0]
    for s in sizes:
        offs.append(offs[-1] + s)
    flat_views = [flat.narrow(0, o, s) for o, s in zip(offs, sizes)]
    params = [torch.empty(s, dtype=torch.float16, device=DEV) for s in sizes]
    unflatten = TensorPlan(flat_views, params)
    unflatten.scale_cast(1.0)
    torch.cuda.synchronize()
    for i in (0, 1, nseg // 2, nseg - 1):
        assert torch.equal(params[i].view(torch.int16), flat_views[i].view(torch.int16))
    masters = [torch.empty(s, dtype=torch.float32, device=DEV) for s in sizes]
    TensorPlan(params, masters).scale_cast(1.0)
    for i in (0, nseg - 1):
        assert torch.equal(masters[i], params[i].float())
    back = torch.zeros_like(flat)
    back_views = [back.narrow(0, o, s) for o, s in zip(offs, sizes)]
    halves = [torch.empty(s, dtype=torch.float16, device=DEV) for s in sizes] if total < 10 ** 9 else params
    TensorPlan(masters, halves).scale_cast(1.0)          # fp32 -> fp16 (exact: the values came from fp16)
    TensorPlan(halves, back_views).scale_cast(1.0)       # repack
    torch.cuda.synchronize()
    assert torch.equal(back.view(torch.int16), flat.view(torch.int16)), "round trip is not the identity"
    unflatten.close()


def test_single_tensor_beyond_two_to_the_31_elements():
    """One tensor of 2^31 + 4099 fp16 elements: chunk and tile offsets inside a tensor are 64-bit.  The fused step
    through a plan and through the allocation-free entry point, and the plan-free cast copy, are checked against
    torch on the device element for element (the unscale by a power of two is exact, the clip is one fp32 multiply)."""
    n = 2 ** 31 + 4099
    gen = torch.Generator(device=DEV).manual_seed(7)
    x = torch.empty(n, dtype=torch.float16, device=DEV)
    step = 2 ** 28
    for lo in range(0, n, step):                         # filled in pieces: no fp32 temporary of the full size
        hi = min(n, lo + step)
        x[lo:hi] = (torch.randn(hi - lo, generator=gen, device=DEV) * 1e-3 * 4096.0).to(torch.float16)
    out = torch.zeros(n, dtype=torch.float32, device=DEV)
    inv, max_norm = 1.0 / 4096.0, 1.0
    plan = TensorPlan([x], [out])
    plan.fused_step(inv, max_norm)
    res = plan.result()
    assert res.overflow == 0 and res.clipped == 1
    sq = 0.0
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        sq += float(((x[lo:hi].float() * inv).double() ** 2).sum())
    assert math.isclose(res.norm, float(torch.tensor(math.sqrt(sq), dtype=torch.float32)), rel_tol=REL)
    coef = torch.tensor(res.coef, dtype=torch.float32, device=DEV)
    inv_t = torch.tensor(inv, dtype=torch.float32, device=DEV)
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        assert bool(torch.equal(out[lo:hi], (x[lo:hi].float() * inv_t) * coef)), f"elements {lo}..{hi}"
    first = out[-8192:].clone()
    # the allocation-free entry point: same decision, same bits
    out.zero_()
    res_dev = torch.zeros(8, dtype=torch.int32, device=DEV)
    _lib.fused_step_static(x.data_ptr(), out.data_ptr(), n, _lib.RG_F16, _lib.RG_F32, inv, max_norm, 0, res_dev.data_ptr(), 0,
                           torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert bool(torch.equal(out[-8192:], first)) and bool(torch.equal(out[:8192], (x[:8192].float() * inv_t) * coef))
    # plan-free cast copy across the 2^31 boundary
    _lib.scale_cast_single(x.data_ptr(), out.data_ptr(), n, _lib.RG_F16, _lib.RG_F32, 1.0, 0, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for lo in (0, 2 ** 31 - 5000, n - 9000):
        assert bool(torch.equal(out[lo:lo + 9000], x[lo:lo + 9000].float()))
    plan.close()
