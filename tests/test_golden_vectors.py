"""Committed golden vectors (tests/golden/fused_step_vectors.json): the oracle must keep
reproducing them on the CPU, and the HIP path must reproduce them on the GPU."""
import json
import math
import os

import pytest
import torch

from oracle import gradpath as oracle
from rannc_amd import _lib
from tests.helpers import TORCH_DTYPE, assert_bits_equal

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fused_step_vectors.json")
GOLDEN = json.load(open(PATH))
INT = {"f32": torch.int32, "f16": torch.int16, "bf16": torch.int16}


def _tensor(bits, shape, name):
    return torch.tensor(bits, dtype=INT[name]).view(TORCH_DTYPE[name]).view(shape)


def _inputs(c):
    return [_tensor(b, s, c["src_dtype"]) for b, s in zip(c["src_bits"], c["shapes"])]


@pytest.mark.parametrize("c", GOLDEN["fused_step"], ids=lambda c: c["name"])
def test_oracle_reproduces_golden(c):
    grads = _inputs(c)
    r = oracle.fused_step(grads, [c["dst_dtype"]] * len(grads), c["inv_scale"], c["max_norm"])
    assert r.overflow == c["overflow"]
    if not c["overflow"]:
        assert r.norm == c["norm"] and r.coef == c["coef"] and r.tensor_norms == c["tensor_norms"]
    else:
        assert r.coef is None
    want = _tensor(c["bucket_bits"], (len(c["bucket_bits"]),), c["dst_dtype"])
    assert_bits_equal(r.buckets[c["dst_dtype"]], want, c["name"])


@pytest.mark.parametrize("lay", GOLDEN["segment_layout"], ids=lambda l: f"{l['numel']}x{l['elem_size']}r{l['nranks']}")
def test_layout_golden(lay):
    got = _lib.segment_layout(lay["numel"], lay["elem_size"], lay["nranks"])
    assert got == (lay["aligned"], lay["segment"], lay["offsets"], lay["src_sizes"])
    o = oracle.segment_layout(lay["numel"], lay["elem_size"], lay["nranks"])
    assert (o.aligned_size, o.segment_size, list(o.offsets), list(o.src_sizes)) == got


@pytest.mark.gpu
@pytest.mark.parametrize("c", GOLDEN["fused_step"], ids=lambda c: c["name"])
def test_gpu_reproduces_golden(c):
    from rannc_amd.multi_tensor import TensorPlan
    dev = "cuda:0"
    grads = _inputs(c)
    n = sum(g.numel() for g in grads)
    bucket = torch.full((n + 3,), 7.0, dtype=TORCH_DTYPE[c["dst_dtype"]], device=dev)[3:]
    views, off = [], 0
    for g in grads:
        views.append(bucket.narrow(0, off, g.numel()))
        off += g.numel()
    plan = TensorPlan([g.to(dev) for g in grads], views)
    plan.fused_step(c["inv_scale"], c["max_norm"], _lib.RG_STEP_WRITE_ON_OVERFLOW)
    res = plan.result()
    assert res.overflow == c["overflow"]
    unclipped = _tensor(c["unclipped_bits"], (n,), c["dst_dtype"])
    if c["overflow"]:
        assert res.clipped == 0 and res.skipped == 1
        assert_bits_equal(bucket.cpu(), unclipped, c["name"])      # Apex-identical: unscaled, unclipped
        return
    assert math.isclose(res.norm, c["norm"], rel_tol=1e-6)
    for a, b in zip(plan.tensor_norms(), c["tensor_norms"]):
        assert math.isclose(a, b, rel_tol=1e-6, abs_tol=1e-30)
    assert res.clipped == (1 if c["coef"] is not None else 0)
    if c["coef"] is not None:
        assert math.isclose(res.coef, c["coef"], rel_tol=1e-6)
        if float(torch.tensor(c["coef"]).float()) == res.coef:       # same coefficient -> same bits as the golden bucket
            assert_bits_equal(bucket.cpu(), _tensor(c["bucket_bits"], (n,), c["dst_dtype"]), c["name"])
        want = unclipped.clone()
        want.mul_(float(res.coef))
        assert_bits_equal(bucket.cpu(), want, c["name"])
    else:
        assert_bits_equal(bucket.cpu(), unclipped, c["name"])
