#!/usr/bin/env python3
"""Benchmark of the per-step parameter/gradient path on one MI355X.

A "step" is one pass of the measured operation over one batch of synthetic tensors that are already
resident in HBM.  The headline operation is the fused step - pass 1 reads the gradients (inf/NaN
flag + per-tensor sums of squares), a small kernel derives the global norm and the clip coefficient
on the device, pass 2 re-reads the gradients and writes the unscaled, clipped values into the packed
bucket - on the largest configuration that fits one GPU, ``c3_bert_enlarged``.

Prints ONE JSON line.  ``value`` is algorithmic GB/s over the whole step: the bytes the operation must
move (``(2s + d) N`` for a fused step that clips; s, d = source / destination bytes per element) divided
by the wall time per step.  With no ``--workload`` / ``--op`` the line also carries ``configs``: the same
measurement for every other configuration and operation of the path (each can be run alone with
``--workload`` / ``--op``, which is how the profiles under ``profiles/`` are made).
"""
from __future__ import annotations

import argparse
import json
import os
import platform
import re
import sys
import time

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E
ROOT = os.path.dirname(os.path.abspath(__file__))
HEADLINE = "c3_bert_enlarged"

FUSED_OPS = ("fused_step", "fused_step_noclip", "fused_step_noclip_2pass", "overflow_host_gate", "unscale_pack",
             "copy_back", "unflatten_back", "grad_norm", "zero", "zero_bucket", "accumulate", "unscale_accumulate", "clip_in_place",
             "consolidate", "zero_staging_pack")
C5_OPS = ("c5_unflatten", "c5_master_cast", "c5_copy_back", "c5_repack")
OPTIM_OPS = ("adam", "sgd", "adam_from_model_grads")
ALL_OPS = ("all",) + FUSED_OPS + C5_OPS + OPTIM_OPS + ("api_step", "graph_step", "ceilings")


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default=None,
                    help="c1_mlp | c2_bert_large | c3_bert_enlarged | c3_bert_enlarged_overflow | c4_resnet152x2 | c5_zero_flat")
    ap.add_argument("--op", default=None, choices=ALL_OPS,
                    help="all (default: headline + every configuration), or one operation to run alone")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--chunk-elems", type=int, default=0)
    ap.add_argument("--c5-elements", type=int, default=10_000_000_000, help="total elements of the ZeRO flat buffer")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--loss-scale", default="static", choices=("static", "dynamic", "dynamic_device"),
                    help="--op api_step: where the loss scale lives")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three plain elementwise kernels over 1 GiB of fp32 first (out = in * 1.5: 1 GiB read, "
                         "1 GiB written; known traffic for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--cpu-seconds", type=float, default=20.0, help="budget for the CPU baseline leg")
    return ap.parse_args()


def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return platform.processor() or "unknown"


def gpu_clocks() -> dict:
    """Clock and power state of GPU 0 as sysfs shows it (the current level of each clock domain is the line
    marked ``*``), read once before the first kernel so that runs on different boxes can be told apart."""
    import glob
    out = {}
    cards = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_mclk"))
    if not cards:
        return {"note": "no sysfs clock files visible"}
    base = os.path.dirname(cards[0])
    for name in ("pp_dpm_sclk", "pp_dpm_mclk", "pp_dpm_fclk", "pp_dpm_socclk"):
        try:
            lines = [l.strip() for l in open(os.path.join(base, name)) if l.strip()]
            out[name[len("pp_dpm_"):] + "_levels"] = [l.split(":", 1)[1].strip() for l in lines]
            cur = [l for l in lines if l.endswith("*")]
            if cur:
                out[name[len("pp_dpm_"):]] = cur[0].split(":", 1)[1].replace("*", "").strip()
        except OSError:
            pass
    try:
        out["perf_level"] = open(os.path.join(base, "power_dpm_force_performance_level")).read().strip()
    except OSError:
        pass
    for hw in glob.glob(os.path.join(base, "hwmon", "hwmon*")):
        for key, fn in (("power_cap_w", "power1_cap"), ("power_avg_w", "power1_average"), ("power_input_w", "power1_input")):
            try:
                out[key] = round(int(open(os.path.join(hw, fn)).read()) / 1e6, 1)
            except (OSError, ValueError):
                pass
    return out


# ----------------------------------------------------------------------------- measured traffic

def measured_traffic(op: str, workload: str, kernel: str):
    """HBM bytes per launch of ``kernel`` from the committed rocprofv3 --pmc summary of this operation and
    workload (``profiles/<op>_<workload>_hbm_traffic.txt``, lines ``traffic_bytes_per_launch: <kernel> = <bytes>``),
    or None when that summary does not exist."""
    path = os.path.join(ROOT, "profiles", f"{op}_{workload}_hbm_traffic.txt")
    try:
        with open(path) as f:
            for line in f:
                m = re.match(r"traffic_bytes_per_launch:\s*(.+?)\s*=\s*([0-9]+)\s*$", line)
                if m and m.group(1) == kernel:
                    return int(m.group(2))
    except OSError:
        pass
    return None


# ----------------------------------------------------------------------------- timing

def timed(fn, steps: int, warmup: int, min_untimed: int = 0):
    """warm-up (at least ``min_untimed`` untimed calls so the clocks have ramped), then exactly ``steps`` calls
    between two synchronisations.  Returns (wall seconds per step, device seconds per step from events on the
    launch stream, which is torch's current stream for every kernel of the library)."""
    import torch
    for _ in range(max(min_untimed, warmup)):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    while not e1.query():             # poll: a blocking wait adds its wake-up latency to the last step
        pass
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    return wall, e0.elapsed_time(e1) * 1e-3 / steps


def roofline(kernel: str, bytes_per_launch: int, launch_s: float, traffic, **extra) -> dict:
    achieved = bytes_per_launch / launch_s / 1e9
    out = {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
           "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
           "algorithmic_bytes_per_launch": int(bytes_per_launch), "avg_launch_ms": round(launch_s * 1e3, 4)}
    out.update(extra)
    return out


def entry(workload: str, op: str, step_s: float, step_bytes: int, roof: dict, **extra) -> dict:
    gbps = step_bytes / step_s / 1e9
    out = {"workload": workload, "op": op, "ms_per_step": round(step_s * 1e3, 4), "algorithmic_bytes_per_step": int(step_bytes),
           "GB/s": round(gbps, 1), "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2), "roofline": roof}
    out.update(extra)
    return out


# ----------------------------------------------------------------------------- fused-step workloads

class StepWorkload:
    """Gradients of one configuration on the device, with the packed destination bucket and its views."""

    def __init__(self, key: str, seed: int, chunk_elems: int = 0):
        import torch
        from rannc_amd.multi_tensor import TensorPlan
        from rannc_amd.workloads import make_grads, step_config
        self.torch, self.key = torch, key
        self.cfg = step_config(key)
        self.dev = torch.device("cuda", 0)
        self.grads, _ = make_grads(self.cfg, seed, device=str(self.dev))
        self.n = sum(g.numel() for g in self.grads)
        self.ddt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[self.cfg.bucket_dtype]
        self.bucket = torch.zeros(self.n, dtype=self.ddt, device=self.dev)
        self.views, off = [], 0
        for g in self.grads:
            self.views.append(self.bucket.narrow(0, off, g.numel()))
            off += g.numel()
        self.s, self.d = self.grads[0].element_size(), self.bucket.element_size()
        self.plan = TensorPlan(self.grads, self.views, chunk_elems=chunk_elems)
        # as a caller does once per plan: the library times its block -> XCD orders on this plan's own tensors
        # (destinations hold zeros here; a real caller tunes before the first step, when they are dead too)
        self.write_order = self.plan.tune()

    def close(self):
        self.plan.close()
        self.grads = self.views = self.bucket = None
        self.torch.cuda.empty_cache()

    def describe(self) -> dict:
        return {"workload": self.key, "description": self.cfg.description, "tensors": len(self.grads), "elements": self.n,
                "src_bytes_per_elem": self.s, "dst_bytes_per_elem": self.d,
                "chunk_elems": self.plan.plan.chunk_elems, "chunks": self.plan.plan.num_chunks,
                "tuned_write_order": self.write_order}


def run_fused_step(w: StepWorkload, steps: int, warmup: int, op: str = "fused_step") -> dict:
    """The fused step.  ``op`` selects the strategy: the default two passes, ``fused_step_noclip`` = a bound the norm
    stays under with the one-pass strategy asked for (RG_STEP_EXPECT_NO_CLIP), ``fused_step_noclip_2pass`` = the same
    bound with the default two passes."""
    from rannc_amd import _lib
    torch, cfg, plan = w.torch, w.cfg, w.plan
    max_norm = cfg.max_norm if op == "fused_step" else 1e30
    flags = _lib.RG_STEP_EXPECT_NO_CLIP if op == "fused_step_noclip" else _lib.RG_STEP_DEFAULT

    def step():
        plan.fused_step(cfg.inv_scale, max_norm, flags)

    # Untimed: the warm-up steps asked for, preceded by enough further steps that the GPU has left its idle clocks.
    for _ in range(max(60, warmup)):
        step()
    torch.cuda.synchronize()
    # Timed region: HIP events (recorded by the library on the launch stream) bracket only the last kernel of the
    # step - the dominant one - and only on every fifth step: each record costs a few microseconds of stream time.
    stride = min(5, max(1, steps))
    sampled = (steps + stride - 1) // stride
    plan.plan.enable_timing(-sampled)
    plan.plan.timing_stride(stride)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    done = torch.cuda.Event()
    done.record()
    while not done.query():
        pass
    torch.cuda.synchronize()
    step_s = (time.perf_counter() - t0) / steps
    res = plan.result()
    last_only = [plan.plan.read_timing(i) for i in range(sampled)]
    plan.plan.timing_stride(1)
    # A second, untimed loop brackets all stages for the breakdown.
    k = min(steps, 50)
    plan.plan.enable_timing(k)
    for _ in range(k):
        step()
    torch.cuda.synchronize()
    per_kernel = [plan.plan.read_timing(i) for i in range(k)]
    plan.plan.enable_timing(0)

    n, s, d = w.n, w.s, w.d
    clipped, overflow = bool(res.clipped), int(res.overflow)
    last_ms = sum(x[2] for x in last_only) / len(last_only)
    first_ms = sum(x[0] for x in per_kernel) / len(per_kernel)
    mid_ms = sum(x[1] for x in per_kernel) / len(per_kernel)
    extra = {}
    if op == "fused_step_noclip":
        # one pass (read s, write d) + decision + a gated in-place scale kernel that finds nothing to do
        step_bytes = (s + d) * n
        roof = roofline("pass_kernel<reduce+write, streaming>", (s + d) * n, first_ms * 1e-3,
                        measured_traffic(op, w.key, "pass_kernel<reduce+write>"),
                        note="dominant kernel timed in a second, untimed loop with every stage bracketed",
                        other_kernels={"reduce_segments+decide": {"avg_launch_ms": round(mid_ms, 4)},
                                       "pass_kernel<write> gated on the decision (idle)": {"avg_launch_ms": round(last_ms, 4)}})
    else:
        step_bytes = (2 * s + d) * n if clipped else (s + d) * n
        if res.skipped:
            # the write pass is launched and finds the step skipped: the step moves the read pass's bytes only, and
            # is scored against them
            step_bytes = s * n
            extra["note"] = ("skipped on the device: scored against s*N, the bytes the step moves; the write pass's "
                             "blocks all start, read the decision and exit")
            roof = roofline("pass_kernel<reduce, streaming>", s * n, first_ms * 1e-3,
                            measured_traffic(op, w.key, "pass_kernel<reduce>"),
                            note="the write pass found the step skipped; its idle launch took %.1f us" % (last_ms * 1e3),
                            other_kernels={"pass_kernel<write> (skipped on the device)": {"avg_launch_ms": round(last_ms, 4)},
                                           "reduce_segments+decide": {"avg_launch_ms": round(mid_ms, 4)}})
        else:
            roof = roofline("pass_kernel<write, streaming>", (s + d) * n, last_ms * 1e-3,
                            measured_traffic(op, w.key, "pass_kernel<write>"), launches_timed=len(last_only),
                            other_kernels={
                                "pass_kernel<reduce>": {"avg_launch_ms": round(first_ms, 4), "algorithmic_bytes_per_launch": s * n,
                                                        "achieved": round(s * n / (first_ms * 1e-3) / 1e9, 1),
                                                        "traffic": measured_traffic(op, w.key, "pass_kernel<reduce>")},
                                "reduce_segments+decide": {"avg_launch_ms": round(mid_ms, 4)},
                                "note": "from a second, untimed loop of the same steps with all stages bracketed"})
    return entry(w.key, op, step_s, step_bytes, roof, clipped=clipped, overflow=overflow, skipped=int(res.skipped),
                 norm=res.norm, coef=res.coef, steps=steps, elements_per_s=round(n / step_s, 1), **extra)


def run_overflow_host_gate(w: StepWorkload, steps: int, warmup: int) -> dict:
    """The two-call form a loss scaler uses: read pass, flag read on the host (it decides the loss scale there,
    ``pyrannc/amp/__init__.py:44-65``), and the write pass only launched when the step is not skipped."""
    cfg, plan = w.cfg, w.plan
    state = {"res": None}

    def step():
        plan.step_begin(cfg.inv_scale)
        state["res"] = plan.result()          # waits for the read pass
        if not state["res"].overflow:
            plan.step_finish(cfg.max_norm)

    wall, dev_s = timed(step, steps, warmup, 20)
    res = state["res"]
    n, s, d = w.n, w.s, w.d
    moved = s * n if res.overflow else (2 * s + d) * n
    roof = roofline("pass_kernel<reduce, streaming>", s * n, dev_s, measured_traffic("overflow_host_gate", w.key, "pass_kernel<reduce>"),
                    note="launch time = whole step from device events (read pass + reduce + decide + the host's read of the flag)")
    return entry(w.key, "overflow_host_gate", wall, moved, roof, overflow=int(res.overflow), steps=steps,
                 note="bytes = what the step moves: s*N when it is skipped")


def run_plan_op(w: StepWorkload, op: str, steps: int, warmup: int) -> dict:
    """Single-kernel operations over the workload's tensor list."""
    import torch
    from rannc_amd.multi_tensor import TensorPlan
    n, s, d = w.n, w.s, w.d
    cleanup = []
    if op == "unscale_pack":
        fn, nbytes, kernel = (lambda: w.plan.unscale_pack(w.cfg.inv_scale)), (s + d) * n, "pass_kernel<reduce+write>"
    elif op == "grad_norm":
        fn, nbytes, kernel = w.plan.grad_norm, s * n, "pass_kernel<reduce>"
    elif op == "zero":
        # clearParamGrads without consolidation: one separately allocated tensor per gradient, each cleared where it lies
        # (rg_zero takes the table-driven pass unless the tensors happen to lie back to back: those it clears as one range)
        outs = [torch.empty_like(g) for g in w.grads]     # stand-ins: the workload's gradients feed the other operations
        plan = TensorPlan([None] * len(outs), outs)
        cleanup.append(plan)
        end, flat = None, True
        for g in outs:
            if g.numel():
                flat = flat and end in (None, g.data_ptr())
                end = g.data_ptr() + g.numel() * g.element_size()
        fn, nbytes, kernel = plan.zero, s * n, "fill_zero_kernel" if flat else "pass_kernel<write> (zero fill)"
    elif op == "zero_bucket":
        # clearParamGrads on consolidated gradients: the bucket itself is cleared, as one flat range (rg_fill_zero)
        from rannc_amd.multi_tensor import fill_zero_
        fn, nbytes, kernel = (lambda: fill_zero_(w.bucket)), d * n, "fill_zero_kernel"
    elif op in ("accumulate", "unscale_accumulate"):
        # dst += src * scale: the destination is read and written; the second form also reports flag and norm
        w.bucket.zero_()
        if op == "accumulate":
            fn, kernel = (lambda: w.plan.accumulate(w.cfg.inv_scale)), "pass_kernel<write+accumulate>"
        else:
            fn, kernel = (lambda: w.plan.unscale_accumulate(w.cfg.inv_scale)), "pass_kernel<reduce+write+accumulate>"
        nbytes = (s + 2 * d) * n
    elif op == "clip_in_place":
        # RaNNCModule.clip_grad_norm on gradients that are already unscaled: read pass over the bucket, decision,
        # in-place multiply
        plan = TensorPlan(w.views, w.views)
        cleanup.append(plan)
        w.plan.scale_cast(w.cfg.inv_scale)
        fn, nbytes, kernel = (lambda: plan.fused_step(1.0, 1e-30)), 3 * d * n, "pass_kernel<reduce> + pass_kernel<write>"
    elif op == "copy_back":
        # fp32 masters (the packed bucket holds fp32 values after a step) -> model parameters in the gradient dtype
        mdt = w.grads[0].dtype if w.grads[0].dtype != torch.float32 else torch.bfloat16
        masters = torch.randn(n, device=w.dev, dtype=torch.float32)
        mviews, off = [], 0
        for g in w.grads:
            mviews.append(masters.narrow(0, off, g.numel()))
            off += g.numel()
        models = [torch.empty(g.shape, dtype=mdt, device=w.dev) for g in w.grads]
        plan = TensorPlan(mviews, models)
        cleanup.append(plan)
        fn, nbytes, kernel = (lambda: plan.scale_cast(1.0)), (4 + models[0].element_size()) * n, "pass_kernel<write>"
    elif op == "unflatten_back":
        # packed bucket -> one separately allocated tensor per parameter, same dtype
        outs = [torch.empty(g.shape, dtype=w.ddt, device=w.dev) for g in w.grads]
        plan = TensorPlan(w.views, outs)
        cleanup.append(plan)
        fn, nbytes, kernel = (lambda: plan.scale_cast(1.0)), 2 * d * n, "pass_kernel<write>"
    else:
        raise ValueError(op)
    wall, dev_s = timed(fn, steps, warmup, 20)
    for p in cleanup:
        p.close()
    extra = {}
    if op in ("unscale_pack", "unscale_accumulate"):
        extra["note"] = "launch time = pass + reduce_segments + decide kernels (whole operation, device events)"
    if op == "clip_in_place":
        extra["note"] = ("every step clips (max_norm 1e-30: the values shrink towards zero, the traffic is the same): "
                         "read d, then read d + write d")
    return entry(w.key, op, wall, nbytes, roofline(kernel, nbytes, dev_s, measured_traffic(op, w.key, kernel), **extra), steps=steps)


def run_host_layer_op(w: StepWorkload, op: str, steps: int, warmup: int) -> dict:
    """Two per-step operations of the registry, driven through the mirror of the reference's classes on parameters
    shaped like the workload: ``consolidate`` = ``GradConsolidation::consolidate`` (``src/comp/ParamStorage.cpp:118-179``:
    every gradient copied into its bucket view), ``zero_staging_pack`` = ``allReduceParamGradsZero`` at one rank
    (``:440-520``: gradients packed into zero-padded staging buffers, fp16/bf16 widened to fp32, and copied back)."""
    import torch
    from rannc_amd.param_storage import GradConsolidation, ParamStorage
    n, s = w.n, w.s
    params = [torch.nn.Parameter(torch.empty(g.shape, dtype=g.dtype, device=w.dev)) for g in w.grads]
    st = ParamStorage()
    ids = {}
    for i, p in enumerate(params):
        st.register_param(id(p), p)
        ids[f"p{i:05d}"] = id(p)
    try:
        from rannc_amd import _ranncgrad
        owners, fresh = _ranncgrad.TensorList(params), _ranncgrad.TensorList(w.grads)
        hand_out = lambda: owners.set_grads(fresh)        # as backward does: from C++
    except ImportError:
        def hand_out():
            for p, g in zip(params, w.grads):
                p.grad = g
    if op == "consolidate":
        con = GradConsolidation(st, [id(p) for p in params], False, False)

        def fn():
            hand_out()                             # backward left fresh gradients outside the buckets
            con.consolidate()
        nbytes, kernel = 2 * s * n, "pass_kernel<write> (raw copy)"
    else:
        from rannc_amd import _pyrannc
        mod = _pyrannc.RaNNCModule(True, True, True)       # amp masters reduced in fp32, ZeRO: the product's path
        mod.init({k: params[i] for i, k in enumerate(ids)}, False)
        for p, g in zip(params, w.grads):
            p.grad = g
        wide = 4 if w.grads[0].dtype == torch.float16 else s       # the reference widens fp16 only (ParamStorage.cpp:483-486)

        def fn():
            mod.allreduce_grads_zero()
        nbytes, kernel = 2 * (s + wide) * n, "pass_kernel<write> x2 (pack into staging, copy back)"
    wall, dev_s = timed(fn, steps, warmup, 10)
    if op != "consolidate":
        mod.undeploy()
    return entry(w.key, op, wall, nbytes, roofline(kernel, nbytes, dev_s, None,
                 note="launch time = all launches of the operation (device events); ms_per_step is wall time including "
                      "the host's per-parameter bookkeeping"), steps=steps, tensors=len(params))


# ----------------------------------------------------------------------------- yardsticks

def run_ceilings(steps: int, warmup: int, nbytes: int = 1 << 30) -> list:
    """The library's yardstick kernels (``rg_ceiling_kernel``): the passes' access patterns over flat 1 GiB arrays."""
    import torch
    from rannc_amd import _lib
    from rannc_amd.multi_tensor import stream_handle
    dev = torch.device("cuda", 0)
    arrays = [torch.empty(nbytes // 4, dtype=torch.float32, device=dev).fill_(1.0) for _ in range(5)]
    ptrs = [a.data_ptr() for a in arrays]
    out = []
    for name, kind, moved in (("read", 0, 1.0), ("fill", 1, 1.0), ("fill_paced", 8, 1.0), ("copy_f32", 2, 2.0), ("copy_f32_nt", 5, 2.0),
                              ("widen_bf16_f32", 3, 1.5), ("adam_streams", 4, 7.0), ("adam_streams_bf16_copy", 6, 7.5),
                              ("adam_streams_bf16_copy_step_shape", 7, 7.5)):
        def fn():
            _lib.ceiling_kernel(kind, ptrs, nbytes, 0, stream_handle(dev))
        wall, dev_s = timed(fn, steps, warmup, 20)
        b = int(moved * nbytes)
        out.append({"workload": "flat_1GiB", "op": "ceiling_" + name, "ms_per_step": round(dev_s * 1e3, 4),
                    "algorithmic_bytes_per_step": b, "GB/s": round(b / dev_s / 1e9, 1),
                    "pct_of_hbm_peak": round(100.0 * b / dev_s / 1e9 / HBM_PEAK_GBPS, 2), "steps": steps})
        if name.startswith("adam_streams"):
            for a in arrays[:4]:
                a.fill_(1.0)
    del arrays
    torch.cuda.empty_cache()
    return out


# ----------------------------------------------------------------------------- ZeRO flat buffer (config 5)

class ZeroFlat:
    """fp16 flat buffer cut into 4096 odd-sized segments at odd offsets, separately allocated fp16 parameters and
    fp32 masters (``DistributedParamLocator`` store / setScalarType / load at one rank)."""

    def __init__(self, total: int, seed: int):
        import torch
        from rannc_amd.workloads import zero_segment_sizes
        self.torch = torch
        dev = torch.device("cuda", 0)
        self.sizes = zero_segment_sizes(4096, total, seed=seed)
        self.n = n = sum(self.sizes)
        self.flat = torch.empty(n, dtype=torch.float16, device=dev)
        step = 1 << 28
        for lo in range(0, n, step):      # cheap on-device pattern: every fp16 bit pattern except inf / NaN
            hi = min(n, lo + step)
            idx = torch.arange(lo, hi, device=dev, dtype=torch.int64)
            bits = ((idx * 2654435761) >> 7) & 0xFFFF
            bits = torch.where((bits & 0x7C00) == 0x7C00, bits & 0x83FF, bits)
            self.flat[lo:hi] = bits.to(torch.int16).view(torch.float16)
            del idx, bits
        offs = [0]
        for sz in self.sizes:
            offs.append(offs[-1] + sz)
        self.flat_views = [self.flat.narrow(0, o, sz) for o, sz in zip(offs, self.sizes)]
        self.params = [torch.empty(sz, dtype=torch.float16, device=dev) for sz in self.sizes]
        self.masters = [torch.empty(sz, dtype=torch.float32, device=dev) for sz in self.sizes]

    def close(self):
        self.flat = self.flat_views = self.params = self.masters = None
        self.torch.cuda.empty_cache()


def run_c5(z: ZeroFlat, op: str, steps: int, warmup: int) -> dict:
    from rannc_amd.multi_tensor import TensorPlan
    src, dst, bpe = {"c5_unflatten": (z.flat_views, z.params, 4), "c5_master_cast": (z.params, z.masters, 6),
                     "c5_copy_back": (z.masters, z.params, 6), "c5_repack": (z.params, z.flat_views, 4)}[op]
    plan = TensorPlan(src, dst)
    order = plan.tune()                       # as a caller does once per plan: measured block -> XCD order
    wall, dev_s = timed(lambda: plan.scale_cast(1.0), steps, warmup, 5)
    plan.close()
    nbytes = bpe * z.n
    return entry("c5_zero_flat", op, wall, nbytes,
                 roofline("pass_kernel<write, streaming>", nbytes, dev_s, measured_traffic(op, "c5_zero_flat", "pass_kernel<write>")),
                 steps=steps, elements=z.n, segments=len(z.sizes), tuned_write_order=order)


# ----------------------------------------------------------------------------- CPU baseline

def cpu_baseline(key: str, seed: int, budget_s: float):
    """The reference's op sequence on the host cores (oracle.reference_step_cpu), on a bounded sample of the same
    workload: the same tensor list with dim 0 of every tensor scaled so that one CPU step fits the budget."""
    import torch
    from oracle import gradpath as oracle
    from rannc_amd.workloads import make_grads, step_config

    cfg = step_config(key)
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)
    torch.set_num_threads(threads)
    frac = 1.0
    est = cfg.total_numel * 8 / (0.3e9 * threads)      # ~0.3 GB/s per thread is a safe lower bound for the op chain
    if est > budget_s / 5:
        frac = max(0.01, (budget_s / 5) / est)
    grads, _ = make_grads(cfg, seed, device="cpu", scale_numel=frac)
    n = sum(g.numel() for g in grads)
    ddt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[cfg.bucket_dtype]
    bucket = torch.zeros(n, dtype=ddt)
    views, off = [], 0
    for g in grads:
        views.append(bucket.narrow(0, off, g.numel()).view(g.shape))
        off += g.numel()
    s, d = grads[0].element_size(), bucket.element_size()
    oracle.reference_step_cpu(grads, views, cfg.inv_scale, cfg.max_norm)      # warm-up
    best, reps, t_start = float("inf"), 0, time.perf_counter()
    coef = None
    while reps < 5 and (reps < 1 or time.perf_counter() - t_start < budget_s):
        t0 = time.perf_counter()
        ovf, norm, coef = oracle.reference_step_cpu(grads, views, cfg.inv_scale, cfg.max_norm)
        best = min(best, time.perf_counter() - t0)
        reps += 1
    nbytes = ((2 * s + d) if coef is not None else (s + d)) * n
    return {
        "value": round(nbytes / best / 1e9, 3), "unit": "GB/s", "cores": threads, "host_cpus": os.cpu_count(),
        "kind": "port",
        "sample": f"{cfg.key}: same {len(grads)}-tensor list, {n} of {cfg.total_numel} elements "
                  f"(dim-0 fraction {frac:.3f}), 1 warm-up + best of {reps} steps of {best * 1e3:.1f} ms, "
                  f"torch {torch.__version__} CPU ops on {threads} threads of {os.cpu_count()} host CPUs, {cpu_model()}",
        "elements_per_s": round(n / best, 1),
    }


# ----------------------------------------------------------------------------- optimizer step

def bench_optimizer(args, key, torch, dev) -> dict:
    """Adam (+ bf16/fp16 model copy) or plain SGD over the workload's tensors: fp32 masters, fp32
    master gradients laid out as views of one packed bucket, separately allocated moments."""
    from rannc_amd import _lib
    from rannc_amd.multi_tensor import TensorPlan, stream_handle
    from rannc_amd.workloads import make_grads, step_config

    cfg = step_config(key)
    grads, _ = make_grads(cfg, args.seed, device=str(dev))
    shapes = [g.shape for g in grads]
    copy_dt = grads[0].dtype if grads[0].dtype != torch.float32 else torch.bfloat16
    direct = args.op == "adam_from_model_grads"
    if not direct:
        del grads
    n = sum(torch.Size(sh).numel() for sh in shapes)
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    bucket = torch.randn(n, device=dev, generator=gen) * 1e-2
    gviews, off = [], 0
    for sh in shapes:
        k = torch.Size(sh).numel()
        gviews.append(bucket.narrow(0, off, k))
        off += k
    params = [torch.randn(sh, device=dev, generator=gen) for sh in shapes]
    adam = args.op in ("adam", "adam_from_model_grads")
    m = [torch.zeros_like(p) for p in params] if adam else None
    v = [torch.zeros_like(p) for p in params] if adam else None
    copies = [torch.zeros(sh, device=dev, dtype=copy_dt) for sh in shapes]
    code = {torch.float16: _lib.RG_F16, torch.bfloat16: _lib.RG_BF16}[copy_dt]
    gsrc = grads if direct else gviews
    gcode = {torch.float32: _lib.RG_F32, torch.float16: _lib.RG_F16, torch.bfloat16: _lib.RG_BF16}[gsrc[0].dtype]
    table = _lib.OptimTable(0, [t.data_ptr() for t in params], [t.data_ptr() for t in gsrc],
                            [t.data_ptr() for t in m] if adam else None, [t.data_ptr() for t in v] if adam else None,
                            [t.data_ptr() for t in copies], [t.numel() for t in params], [gcode] * len(params),
                            [code] * len(params))
    st = stream_handle(dev)
    count = [0]
    plan = TensorPlan(grads, gviews) if direct else None
    gate = plan.plan.result_device_ptr() if direct else 0

    def step():
        count[0] += 1
        if direct:       # read pass (flag + norm), clip decision, Adam on the scaled gradients: nothing else is written
            plan.step_begin(cfg.inv_scale)
            plan.step_decide(cfg.max_norm)
            table.adam_step(1e-3, 0.9, 0.999, 1e-8, 0.0, count[0], grad_scale=cfg.inv_scale, gate=gate, stream=st)
        elif adam:
            table.adam_step(1e-3, 0.9, 0.999, 1e-8, 0.0, count[0], stream=st)
        else:
            table.sgd_step(0.01, stream=st)

    step_s, launch_s = timed(step, args.steps, args.warmup, 20)
    gs = gsrc[0].element_size()
    if direct:
        bytes_per_elem = gs + (gs + 12) + 12 + 2      # read pass + Adam (grad, p, m, v in; p, m, v, copy out)
    else:
        bytes_per_elem = (16 + 12 + 2) if adam else (8 + 4 + 2)
    step_bytes = bytes_per_elem * n
    kernel = ("pass_kernel<reduce> + reduce + decide + optim_kernel<adam>, all launches of a step" if direct
              else f"optim_kernel<{args.op}, streaming>")
    out = {
        "metric": f"achieved HBM GB/s for the multi-tensor {args.op} step with model copy-back",
        "value": round(step_bytes / step_s / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": cfg.key, "op": args.op, "tensors": len(params), "elements": n,
                   "bytes_per_elem": bytes_per_elem, "model_copy_dtype": str(copy_dt), "seed": args.seed},
        "pct_of_hbm_peak": round(100.0 * step_bytes / step_s / 1e9 / HBM_PEAK_GBPS, 2),
        "roofline": roofline(kernel, step_bytes, launch_s, measured_traffic(args.op, cfg.key, "optim_kernel")),
    }
    table.close()
    if plan is not None:
        res = plan.result()
        out["config"].update({"clipped": bool(res.clipped), "overflow": int(res.overflow), "norm": res.norm})
        plan.close()
    del params, m, v, copies, bucket, gviews
    torch.cuda.empty_cache()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline_optimizer("adam" if adam else "sgd", shapes, args.seed, args.cpu_seconds,
                                                     bytes_per_elem)
    return out


def cpu_baseline_optimizer(op: str, shapes, seed: int, budget_s: float, bytes_per_elem: int) -> dict:
    """torch.optim's op sequence (the oracle restates it; bit-identical to the library) on the
    host cores, over as many leading tensors of the workload as fit the time budget."""
    import torch
    from oracle import optim as oracle_optim
    torch.set_num_threads(os.cpu_count() or 1)
    gen = torch.Generator().manual_seed(seed)
    take, total = [], 0
    for sh in shapes:
        take.append(sh)
        total += torch.Size(sh).numel()
        if total >= 64_000_000:
            break
    p = [torch.randn(sh, generator=gen) for sh in take]
    g = [torch.randn(sh, generator=gen) * 1e-2 for sh in take]
    m = [torch.zeros_like(t) for t in p]
    v = [torch.zeros_like(t) for t in p]
    best, reps, t_start = float("inf"), 0, time.perf_counter()
    while reps < 5 and (reps == 0 or time.perf_counter() - t_start < budget_s):
        t0 = time.perf_counter()
        if op == "adam":
            oracle_optim.adam_step(p, g, m, v, reps + 1)
        else:
            oracle_optim.sgd_step(p, g, None, 0.01)
        copies = [oracle_optim.model_copy(t, torch.bfloat16) for t in p]
        best = min(best, time.perf_counter() - t0)
        reps += 1
        del copies
    return {"value": round(bytes_per_elem * total / best / 1e9, 2), "unit": "GB/s", "cores": torch.get_num_threads(),
            "host_cpus": os.cpu_count(), "kind": "port", "cpu": cpu_model(),
            "sample": f"first {len(take)} tensors ({total} elements) of the workload, best of {reps} passes of "
                      f"torch.optim's per-tensor op sequence + master->bf16 copy"}


# ----------------------------------------------------------------------------- the drop-in API path

def bench_api_step(args, key: str, scale_mode: str = "static") -> dict:
    """``scale_mode``: "static" (a fixed loss scale: nothing is read back), "dynamic" (the schedule on the host: one
    read of the overflow flag per step, as the reference does) or "dynamic_device" (the schedule on the device)."""
    full = _api_step_leg(args, key, 1.0, scale_mode)
    # the same tensor list with every tensor cut to one row: the kernels have next to nothing to do, so the wall
    # time of a step is the host's own cost of driving the API (including its one wait for the flag per step)
    tiny = _api_step_leg(args, key, 0.0, scale_mode)
    full["host_only"] = {"what": "same calls on the same tensor list with every tensor cut to one row of dim 0",
                         "elements": tiny["config"]["elements"], "us_per_step": tiny["value"],
                         "device_us_per_step": tiny["device_us_per_step"], "us_per_call": tiny["host_us_per_call"]}
    full["host_us_per_step"] = tiny["value"]
    full["host_fraction_of_device_time"] = round(tiny["value"] / full["device_us_per_step"], 3)
    return full


def _api_step_leg(args, key: str, scale_numel: float, scale_mode: str = "static") -> dict:
    """Host time of the path a training script drives, on a parameter list shaped like ``key``: the exit of
    ``amp.scale_loss`` (unscale + flag), ``RaNNCModule.clip_grad_norm``, ``FusedAdam.step`` and ``zero_grad``.
    Backward is replaced by handing every half parameter a ready gradient tensor.  Reports wall microseconds per
    call (host + device, the host waits for the flag at the scale_loss exit as the reference does) next to the
    device time of the same step, and the host time alone of every call (measured with the device idle-waiting
    excluded: time until the call returns)."""
    import torch
    import rannc_amd
    from rannc_amd import amp
    from rannc_amd.fused_optim import FusedAdam
    from rannc_amd.workloads import step_config

    cfg = step_config(key)
    dev = torch.device("cuda", 0)
    half = torch.bfloat16

    class Holder(torch.nn.Module):
        def __init__(self):
            super().__init__()
            shapes = [sh if scale_numel >= 1.0 else (max(1, int(sh[0] * scale_numel)),) + tuple(sh[1:]) for _, sh in cfg.params]
            self.ps = torch.nn.ParameterList([torch.nn.Parameter(torch.randn(sh, device=dev) * 0.02) for sh in shapes])

        def forward(self, x):
            return x

    model = Holder()
    opt = FusedAdam(model.parameters(), lr=1e-4)
    model, opt = amp.initialize(model, opt, opt_level="O2", half_dtype=half,
                                loss_scale=65536.0 if scale_mode == "static" else "dynamic",
                                device_loss_scale=scale_mode == "dynamic_device")
    rm = rannc_amd.RaNNCModule(model, opt, enable_apex_amp=True)
    rm._deploy()
    params = list(model.parameters())
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    grads = [(torch.randn(p.shape, device=dev, generator=gen) * 1e-2 * 65536.0).to(half) for p in params]
    n = sum(p.numel() for p in params)
    loss = torch.zeros((), device=dev)
    names = ("assign_grads", "scale_loss_exit", "clip_grad_norm", "optimizer_step", "zero_grad")
    host = {k: 0.0 for k in names}
    try:
        # backward hands gradients out from C++; its stand-in does the same (a Python loop over 934 parameters
        # would cost more than the calls this entry is about)
        from rannc_amd import _ranncgrad
        owners, ready = _ranncgrad.TensorList(params), _ranncgrad.TensorList(grads)

        def hand_out_grads():
            owners.set_grads(ready)
    except ImportError:
        def hand_out_grads():
            for p, g in zip(params, grads):
                p.grad = g

    def one_step(record: bool):
        t = [time.perf_counter()]
        ctx = amp.scale_loss(loss, opt)
        ctx.__enter__()
        hand_out_grads()
        t.append(time.perf_counter())
        ctx.__exit__(None, None, None)
        t.append(time.perf_counter())
        rm.clip_grad_norm(1.0)
        t.append(time.perf_counter())
        opt.step()
        t.append(time.perf_counter())
        opt.zero_grad()
        rm.zero_grad()
        t.append(time.perf_counter())
        if record:
            for k, a, b in zip(names, t[:-1], t[1:]):
                host[k] += b - a

    for _ in range(max(args.warmup, 10)):
        one_step(False)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        one_step(True)
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / args.steps
    dev_s = e0.elapsed_time(e1) * 1e-3 / args.steps
    # device time of the kernels alone: the same launches back to back, nothing read on the host in between
    stash = opt._amp_stash
    bytes_per_elem = 2 + (2 + 12) + (12 + 2)     # read pass; Adam reading the scaled gradient; p, m, v and the model copy out
    out = {
        "metric": "host microseconds per training step through the RaNNCModule / amp / FusedAdam API",
        "value": round(wall * 1e6, 1), "unit": "us", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 model / f32 masters", "data": "synthetic",
        "config": {"workload": key, "op": "api_step", "tensors": len(params), "elements": n, "seed": args.seed,
                   "deferred_write": bool(stash.fused), "optimizer": "FusedAdam", "loss_scale": scale_mode},
        "device_us_per_step": round(dev_s * 1e6, 1),
        "host_us_per_call": {k: round(v / args.steps * 1e6, 1) for k, v in host.items()},
        "host_us_per_step_without_assign": round(sum(v for k, v in host.items() if k != "assign_grads") / args.steps * 1e6, 1),
        "algorithmic_bytes_per_step": bytes_per_elem * n,
        "GB/s": round(bytes_per_elem * n / wall / 1e9, 1),
        "note": "with loss_scale 'dynamic' scale_loss_exit includes the wait for the overflow flag (one host read per step, "
                "as the reference's .item()); 'static' and 'dynamic_device' read nothing back",
    }
    rm.undeploy()
    del model, opt, rm, params, grads
    torch.cuda.empty_cache()
    return out


# ----------------------------------------------------------------------------- optimizer phase decided on the device

def bench_device_decided_phase(args, key: str) -> dict:
    """Unscale + flag + norm + clip decision (``rg_step_begin`` + ``rg_step_decide``), the device-side Adam step count
    and the Adam step that reads the scaled bf16 gradients through the gate: nothing is read back by the host, so the
    phase can also be recorded in a HIP graph.  Reports microseconds per phase for the eager calls and for replays."""
    import torch
    from rannc_amd.fused_optim import FusedAdam
    from rannc_amd.multi_tensor import TensorPlan, stream_handle
    from rannc_amd.workloads import step_config
    cfg = step_config(key)
    dev = torch.device("cuda", 0)
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    shapes = [sh for _, sh in cfg.params]
    masters = [torch.nn.Parameter(torch.randn(sh, device=dev, generator=gen) * 0.02) for sh in shapes]
    models = [m.detach().to(torch.bfloat16) for m in masters]
    grads = [(torch.randn(sh, device=dev, generator=gen) * 1e-2 * 256.0).to(torch.bfloat16) for sh in shapes]
    n = sum(m.numel() for m in masters)
    flat = torch.zeros(n, device=dev)                    # master-gradient bucket: part of the plan, never written here
    views, off = [], 0
    for m in masters:
        views.append(flat.narrow(0, off, m.numel()))
        off += m.numel()
    plan = TensorPlan(grads, views)
    opt = FusedAdam(masters, lr=1e-4, capturable=True)
    opt.set_model_copies(masters, models)
    opt.set_grad_sources(masters, grads)
    opt.grad_scale, opt.gate = 1.0 / 256.0, plan.plan.result_device_ptr()

    def phase():
        s = stream_handle(dev)
        plan.plan.step_begin(1.0 / 256.0, s)
        plan.plan.step_decide(1.0, 0, s)
        opt.step()

    def per_call(fn, k):
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(k):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / k * 1e6

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        phase()                                          # allocates the optimizer state: outside any capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    k = max(args.steps, 100)
    eager = per_call(phase, k)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        phase()
    replay = per_call(graph.replay, k)
    res = plan.result()
    out = {"workload": key, "op": "optimizer_phase_device_decided",
           "what": "rg_step_begin + rg_step_decide + rg_adam_clock_advance + rg_adam_step_clocked (gated, reads the scaled "
                   "bf16 gradients, writes the bf16 model copy); no host read-back",
           "tensors": len(shapes), "elements": n, "eager_us_per_phase": round(eager, 1),
           "graph_replay_us_per_phase": round(replay, 1), "steps": k, "clipped": bool(res.clipped), "overflow": int(res.overflow)}
    plan.close()
    del opt, masters, models, grads, flat, views
    torch.cuda.empty_cache()
    return out


# ----------------------------------------------------------------------------- main

def headline_line(args, e: dict, w_desc: dict, dtype: str) -> dict:
    out = {
        "metric": "achieved HBM GB/s (% of roofline) for fused unscale+norm+clip+pack per step",
        "value": e["GB/s"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": e["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": dict(w_desc, op=e["op"], algorithmic_bytes_per_step=e["algorithmic_bytes_per_step"], seed=args.seed,
                       **{k: e[k] for k in ("clipped", "overflow", "skipped", "norm", "coef") if k in e}),
        "pct_of_hbm_peak": e["pct_of_hbm_peak"],
        "roofline": e["roofline"],
    }
    for k in ("elements_per_s", "bytes_moved_per_step", "GB/s_on_bytes_moved", "pct_of_hbm_peak_on_bytes_moved", "note"):
        if k in e:
            out[k] = e[k]
    return out


def run_one(args, key: str, op: str, steps: int, warmup: int) -> tuple:
    """One (workload, operation) measurement -> (entry, workload description, dtype string)."""
    if op in C5_OPS:
        z = ZeroFlat(args.c5_elements, args.seed)
        e = run_c5(z, op, steps, warmup)
        z.close()
        return e, {"workload": "c5_zero_flat", "description": "ZeRO flat fp16 buffer, 4096 odd-sized segments at odd offsets",
                   "elements": e["elements"]}, "f16 / f32 copies"
    w = StepWorkload(key, args.seed, args.chunk_elems)
    if op in ("fused_step", "fused_step_noclip", "fused_step_noclip_2pass"):
        e = run_fused_step(w, steps, warmup, op)
    elif op == "overflow_host_gate":
        e = run_overflow_host_gate(w, steps, warmup)
    elif op in ("consolidate", "zero_staging_pack"):
        e = run_host_layer_op(w, op, steps, warmup)
    else:
        e = run_plan_op(w, op, steps, warmup)
    if op not in ("copy_back", "unflatten_back", "consolidate", "zero_staging_pack"):
        e.setdefault("tuned_write_order", w.write_order)
    desc = w.describe()
    dtype = f"{w.cfg.grad_dtype}->{w.cfg.bucket_dtype} (fp32 arithmetic)"
    w.close()
    return e, desc, dtype


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU only (got --gpus {args.gpus}); "
              "the path has no collectives and shards by running the same kernels per rank",
              file=sys.stderr)
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if args.calibrate_copy:
        # one elementwise kernel that reads 1 GiB and writes 1 GiB (a device-to-device copy_ may be split
        # into several dispatches): the yardstick for what FETCH_SIZE / WRITE_SIZE report per byte moved
        a = torch.empty(256 << 20, dtype=torch.float32, device=dev).fill_(1.0)
        b = torch.empty_like(a)
        for _ in range(3):
            torch.mul(a, 1.5, out=b)
        torch.cuda.synchronize()
        del a, b
        torch.cuda.empty_cache()

    everything = args.op in (None, "all") and args.workload is None
    if args.op in OPTIM_OPS:
        print(json.dumps(bench_optimizer(args, args.workload or "c2_bert_large", torch, dev)), flush=True)
        return 0

    if args.op == "graph_step":
        print(json.dumps(bench_device_decided_phase(args, args.workload or "c1_mlp")), flush=True)
        return 0

    if args.op == "ceilings":
        print(json.dumps({"metric": "achieved HBM GB/s of the yardstick kernels", "unit": "GB/s", "clocks": gpu_clocks(),
                          "configs": run_ceilings(max(args.steps, 20), args.warmup)}), flush=True)
        return 0

    if args.op == "api_step":
        print(json.dumps(bench_api_step(args, args.workload or "c4_resnet152x2", args.loss_scale)), flush=True)
        return 0

    clocks = gpu_clocks()
    key = args.workload or HEADLINE
    op = args.op if args.op not in (None, "all") else ("c5_unflatten" if key == "c5_zero_flat" else "fused_step")
    e, desc, dtype = run_one(args, key, op, args.steps, args.warmup)
    out = headline_line(args, e, desc, dtype)
    out["clocks"] = clocks

    if everything:
        # every other configuration and operation of the path, each measured like the headline (their own step
        # counts: sub-millisecond steps need more of them for the first launch not to weigh)
        sub = max(args.steps, 50)
        plan = [
            ("c3_bert_enlarged_overflow", "fused_step", args.steps), ("c3_bert_enlarged_overflow", "overflow_host_gate", args.steps),
            ("c3_bert_enlarged", "fused_step_noclip", args.steps), ("c3_bert_enlarged", "unscale_pack", args.steps),
            ("c2_bert_large", "fused_step", sub), ("c2_bert_large", "fused_step_noclip", sub),
            ("c2_bert_large", "fused_step_noclip_2pass", sub), ("c2_bert_large", "unscale_pack", sub),
            ("c2_bert_large", "copy_back", sub), ("c2_bert_large", "zero", sub), ("c2_bert_large", "zero_bucket", sub), ("c2_bert_large", "grad_norm", sub),
            ("c2_bert_large", "accumulate", sub), ("c2_bert_large", "unscale_accumulate", sub),
            ("c2_bert_large", "clip_in_place", sub), ("c2_bert_large", "consolidate", sub),
            ("c2_bert_large", "zero_staging_pack", sub),
            ("c4_resnet152x2", "fused_step", sub), ("c4_resnet152x2", "fused_step_noclip", sub),
            ("c4_resnet152x2", "unscale_pack", sub), ("c4_resnet152x2", "zero", sub), ("c4_resnet152x2", "zero_bucket", sub), ("c4_resnet152x2", "grad_norm", sub),
            ("c4_resnet152x2", "accumulate", sub), ("c4_resnet152x2", "unscale_accumulate", sub),
            ("c4_resnet152x2", "clip_in_place", sub), ("c4_resnet152x2", "consolidate", sub),
            ("c4_resnet152x2", "zero_staging_pack", sub),
            ("c1_mlp", "fused_step", 4 * sub), ("c1_mlp", "fused_step_noclip", 4 * sub), ("c1_mlp", "unflatten_back", 4 * sub),
        ]
        configs = []
        cur_key, w = None, None
        for k2, op2, st in plan:
            if k2 != cur_key:
                if w is not None:
                    w.close()
                w, cur_key = StepWorkload(k2, args.seed, args.chunk_elems), k2
            if op2 in ("fused_step", "fused_step_noclip", "fused_step_noclip_2pass"):
                configs.append(run_fused_step(w, st, args.warmup, op2))
            elif op2 == "overflow_host_gate":
                configs.append(run_overflow_host_gate(w, st, args.warmup))
            elif op2 in ("consolidate", "zero_staging_pack"):
                configs.append(run_host_layer_op(w, op2, st, args.warmup))
            else:
                configs.append(run_plan_op(w, op2, st, args.warmup))
            if op2 not in ("copy_back", "unflatten_back", "consolidate", "zero_staging_pack"):      # those run on plans of their own, not tuned
                configs[-1].setdefault("tuned_write_order", w.write_order)
        if w is not None:
            w.close()
        free, _ = torch.cuda.mem_get_info()
        if args.c5_elements * 8 < free * 0.9:
            z = ZeroFlat(args.c5_elements, args.seed)
            for op5 in C5_OPS:
                configs.append(run_c5(z, op5, max(5, min(args.steps, 10)), 2))
            z.close()
        else:
            configs.append({"workload": "c5_zero_flat", "skipped": f"needs {args.c5_elements * 8 / 1e9:.0f} GB of device memory"})
        # the optimizer step behind the clip and the host cost of the drop-in API, one compact row each
        import argparse
        for op3 in ("adam", "adam_from_model_grads", "sgd"):
            sub_args = argparse.Namespace(**dict(vars(args), op=op3, steps=sub, no_cpu_baseline=True))
            r = bench_optimizer(sub_args, "c2_bert_large", torch, dev)
            configs.append({"workload": "c2_bert_large", "op": op3, "ms_per_step": r["ms_per_step"], "GB/s": r["value"],
                            "pct_of_hbm_peak": r["pct_of_hbm_peak"], "bytes_per_elem": r["config"]["bytes_per_elem"],
                            "roofline": r["roofline"], "steps": sub})
        for k3, mode in (("c4_resnet152x2", "static"), ("c2_bert_large", "static"), ("c1_mlp", "static"),
                         ("c4_resnet152x2", "dynamic"), ("c4_resnet152x2", "dynamic_device"),
                         ("c1_mlp", "dynamic"), ("c1_mlp", "dynamic_device")):
            sub_args = argparse.Namespace(**dict(vars(args), op="api_step", steps=max(args.steps, 30)))
            r = bench_api_step(sub_args, k3, mode)
            configs.append({"workload": k3, "op": "api_step", "loss_scale": mode,
                            "what": "scale_loss exit + clip_grad_norm + FusedAdam.step + zero_grad "
                            "through RaNNCModule / amp, wall time per training step",
                            "us_per_step": r["value"], "device_us_per_step": r["device_us_per_step"],
                            "host_only_us_per_step": r["host_us_per_step"], "host_us_per_call": r["host_only"]["us_per_call"],
                            "tensors": r["config"]["tensors"], "steps": sub_args.steps})
        for k3 in ("c1_mlp", "c4_resnet152x2"):
            configs.append(bench_device_decided_phase(args, k3))
        configs.extend(run_ceilings(sub, args.warmup))
        out["configs"] = configs

    if not args.no_cpu_baseline and key != "c5_zero_flat":
        out["cpu_baseline"] = cpu_baseline(key, args.seed, args.cpu_seconds)
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
