#!/usr/bin/env python3
"""Writes tests/golden/fused_step_vectors.json: small fused-step cases with explicit input and
expected output bit patterns.

The reference holds no golden vectors for this path (its tests compare two live runs), and its
Python cannot be imported without its compiled extension, MPI and Apex, so these vectors are
produced by the CPU oracle (oracle/gradpath.py), whose functions are pinned independently in
tests/test_oracle_pins.py.  They freeze the oracle's behaviour (a regression guard for it) and
give the GPU tests inputs that do not depend on any random-number generator's version.

Run from the repository root:  python tests/golden/make_golden.py
"""
import json
import math
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import gradpath as oracle  # noqa: E402

INT = {torch.float32: torch.int32, torch.float16: torch.int16, torch.bfloat16: torch.int16}
NAME = {torch.float32: "f32", torch.float16: "f16", torch.bfloat16: "bf16"}


def bits(t):
    return t.contiguous().view(INT[t.dtype]).flatten().tolist()


def case(name, grads, dst, inv_scale, max_norm):
    r = oracle.fused_step(grads, [dst] * len(grads), inv_scale, max_norm)
    unclipped = oracle.fused_step(grads, [dst] * len(grads), inv_scale, math.inf).buckets.get(dst)
    return {
        "name": name, "src_dtype": NAME[grads[0].dtype], "dst_dtype": dst, "inv_scale": inv_scale, "max_norm": max_norm,
        "shapes": [list(g.shape) for g in grads], "src_bits": [bits(g) for g in grads],
        "overflow": r.overflow, "norm": r.norm, "coef": r.coef, "tensor_norms": r.tensor_norms,
        "bucket_bits": bits(r.buckets[dst]) if dst in r.buckets else [],
        "unclipped_bits": bits(unclipped) if unclipped is not None else [],
    }


def main():
    g = torch.Generator().manual_seed(20240)
    cases = []
    mk = lambda shapes, dt, std, scale: [(torch.randn(s, generator=g) * std * scale).to(dt) for s in shapes]  # noqa: E731
    cases.append(case("bf16_to_f32_clip", mk([(37,), (3, 5), (1,), (0,), (64,)], torch.bfloat16, 1e-2, 65536.0), "f32", 2.0 ** -16, 0.05))
    cases.append(case("f16_to_f32_noclip", mk([(33,), (8,), (129,)], torch.float16, 1e-3, 4096.0), "f32", 2.0 ** -12, 10.0))
    cases.append(case("f32_to_f32_clip", mk([(40,), (7, 3)], torch.float32, 1e-3, 1.0), "f32", 1.0, 1e-3))
    cases.append(case("bf16_to_bf16_clip", mk([(50,), (9,)], torch.bfloat16, 1.0, 1.0), "bf16", 1.0, 0.5))
    cases.append(case("f32_to_f16_nonpow2_scale", mk([(65,)], torch.float32, 1.0, 3.0), "f16", 1.0 / 3.0, 2.0))
    ovf = mk([(20,), (31,)], torch.float16, 1e-3, 4096.0)
    ovf[1][30] = float("inf")
    cases.append(case("f16_overflow_last", ovf, "f32", 2.0 ** -12, 1.0))
    nan = mk([(5,), (12,)], torch.bfloat16, 1e-2, 256.0)
    nan[0][0] = float("nan")
    cases.append(case("bf16_nan_first", nan, "f32", 2.0 ** -8, 1.0))
    edge = [torch.tensor([0.0, -0.0, 65504.0, -65504.0, 6.1e-5, 5.96e-8, -5.96e-8, 1.0, 0.333251953125], dtype=torch.float16)]
    cases.append(case("f16_edge_values", edge, "f32", 2.0 ** -12, 1e9))
    layouts = []
    for numel, es, r in [(1000, 2, 8), (100, 2, 8), (1001, 2, 1), (10, 4, 4), (0, 4, 2), (2 ** 24 + 1, 2, 8), (7, 4, 3)]:
        lay = oracle.segment_layout(numel, es, r)
        layouts.append({"numel": numel, "elem_size": es, "nranks": r, "aligned": lay.aligned_size,
                        "segment": lay.segment_size, "offsets": list(lay.offsets), "src_sizes": list(lay.src_sizes)})
    out = {"generator": "tests/golden/make_golden.py", "torch": torch.__version__, "fused_step": cases, "segment_layout": layouts}
    path = os.path.join(ROOT, "tests", "golden", "fused_step_vectors.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=None, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
