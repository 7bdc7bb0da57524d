#!/usr/bin/env python3
"""Benchmark of the fused unscale + overflow-check + norm + clip + pack step on one MI355X.

A "step" is one pass of the fused step over one batch of synthetic gradients that are already
resident in HBM: pass 1 reads the gradients (flag + per-tensor sums of squares), a small
kernel derives the global norm and the clip coefficient on the device, pass 2 re-reads the
gradients and writes the unscaled, clipped values into the packed fp32 bucket.

Prints ONE JSON line.  `value` is algorithmic GB/s over the whole step: (2*s + d) * N bytes
(s, d = source / destination bytes per element) divided by the measured time per step.
"""
from __future__ import annotations

import argparse
import json
import os
import platform
import sys
import time

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E

# HBM traffic per launch of the dominant kernel (the write pass), from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs of this same command, each scaled by what the counter reads for
# a plain 1 GiB copy (profiles/fused_step_c2_bert_large_hbm_traffic.txt).  Missing = not measured.
MEASURED_TRAFFIC_BYTES = {"c2_bert_large": 2021548222}
# the Adam step with bf16 model copy, same method (profiles/adam_step_c2_bert_large_kernel_stats.txt)
MEASURED_TRAFFIC_BYTES_ADAM = {"c2_bert_large": 10075311450}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2_bert_large")
    ap.add_argument("--op", default="fused_step", choices=["fused_step", "adam", "sgd", "adam_from_model_grads"],
                    help="fused_step (default: the graded metric), the optimizer step that follows it, or both "
                         "without ever writing the unscaled gradients (read pass + clip decision + Adam reading the scaled grads)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--chunk-elems", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three plain 1 GiB fp32 tensor copies first (known traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
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


def cpu_baseline(cfg, seed: int, budget_s: float):
    """The reference's op sequence on the host cores (oracle.reference_step_cpu), on a bounded
    sample of the same workload: the same tensor list with dim 0 of every tensor scaled so
    that one CPU step fits the budget several times."""
    import torch
    from oracle import gradpath as oracle
    from rannc_amd.workloads import make_grads

    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)
    torch.set_num_threads(threads)
    frac = 1.0
    # ~0.3 GB/s per thread is a safe lower bound for the per-tensor op chain
    est = cfg.total_numel * 8 / (0.3e9 * threads)
    if est > budget_s / 4:
        frac = max(0.02, (budget_s / 4) / est)
    grads, _ = make_grads(cfg, seed, device="cpu", scale_numel=frac)
    n = sum(g.numel() for g in grads)
    ddt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[cfg.bucket_dtype]
    bucket = torch.zeros(n, dtype=ddt)
    views, off = [], 0
    for g in grads:
        views.append(bucket.narrow(0, off, g.numel()).view(g.shape))
        off += g.numel()
    s, d = grads[0].element_size(), bucket.element_size()
    best = float("inf")
    t_start = time.perf_counter()
    reps = 0
    while reps < 5 and (reps < 2 or time.perf_counter() - t_start < budget_s):
        t0 = time.perf_counter()
        ovf, norm, coef = oracle.reference_step_cpu(grads, views, cfg.inv_scale, cfg.max_norm)
        dt = time.perf_counter() - t0
        if reps > 0 or dt > budget_s / 2:
            best = min(best, dt)
        reps += 1
    nbytes = ((2 * s + d) if coef is not None else (s + d)) * n
    return {
        "value": round(nbytes / best / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": f"{cfg.key}: same {len(grads)}-tensor list, {n} of {cfg.total_numel} elements "
                  f"(dim-0 fraction {frac:.3f}), best of {max(1, reps - 1)} steps of {best * 1e3:.1f} ms, "
                  f"torch {torch.__version__} CPU ops, {cpu_model()}",
        "elements_per_s": round(n / best, 1),
    }


def bench_optimizer(args, cfg, torch, dev) -> dict:
    """Adam (+ bf16/fp16 model copy) or plain SGD over the workload's tensors: fp32 masters, fp32
    master gradients laid out as views of one packed bucket, separately allocated moments."""
    from rannc_amd import _lib
    from rannc_amd.multi_tensor import stream_handle
    from rannc_amd.workloads import make_grads

    from rannc_amd.multi_tensor import TensorPlan
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

    for _ in range(max(0, 20 - args.warmup) + args.warmup):      # warm-up, at least 20 steps so the clocks have ramped
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()                       # the kernel is launched on torch's current stream, where these events sit
    for _ in range(args.steps):
        step()
    e1.record()
    while not e1.query():             # poll: a blocking wait adds its wake-up latency to the last step
        pass
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    launch_ms = e0.elapsed_time(e1) / args.steps
    gs = gsrc[0].element_size()
    if direct:
        bytes_per_elem = gs + (gs + 12) + 12 + 2      # read pass + Adam (grad, p, m, v in; p, m, v, copy out)
    else:
        bytes_per_elem = (16 + 12 + 2) if adam else (8 + 4 + 2)
    step_bytes = bytes_per_elem * n
    step_s = elapsed / args.steps
    achieved = step_bytes / (launch_ms * 1e-3) / 1e9
    out = {
        "metric": f"achieved HBM GB/s for the multi-tensor {args.op} step with model copy-back",
        "value": round(step_bytes / step_s / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": cfg.key, "op": args.op, "tensors": len(params), "elements": n,
                   "bytes_per_elem": bytes_per_elem, "model_copy_dtype": str(copy_dt), "seed": args.seed},
        "pct_of_hbm_peak": round(100.0 * step_bytes / step_s / 1e9 / HBM_PEAK_GBPS, 2),
        "roofline": {"bound": "hbm", "kernel": ("pass_kernel<reduce> + finalize + optim_kernel<adam>, all launches of a step"
                                                 if direct else f"optim_kernel<{args.op}, streaming>"),
                     "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES_ADAM.get(cfg.key) if args.op == "adam" else None,
                     "algorithmic_bytes_per_launch": step_bytes, "avg_launch_ms": round(launch_ms, 4)},
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
            "kind": "port", "cpu": cpu_model(),
            "sample": f"first {len(take)} tensors ({total} elements) of the workload, best of {reps} passes of "
                      f"torch.optim's per-tensor op sequence + master->bf16 copy"}


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU only (got --gpus {args.gpus}); "
              "the path has no collectives and shards by running the same kernels per rank",
              file=sys.stderr)
        return 2

    import torch
    from rannc_amd.multi_tensor import TensorPlan
    from rannc_amd.workloads import make_grads, step_config

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    cfg = step_config(args.workload)
    if args.op != "fused_step":
        print(json.dumps(bench_optimizer(args, cfg, torch, dev)), flush=True)
        return 0
    if args.calibrate_copy:
        a = torch.empty(256 << 20, dtype=torch.float32, device=dev).fill_(1.0)
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b
        torch.cuda.empty_cache()
    grads, _ = make_grads(cfg, args.seed, device=str(dev))
    n = sum(g.numel() for g in grads)
    ddt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[cfg.bucket_dtype]
    bucket = torch.zeros(n, dtype=ddt, device=dev)
    dsts, off = [], 0
    for g in grads:
        dsts.append(bucket.narrow(0, off, g.numel()))
        off += g.numel()
    s, d = grads[0].element_size(), bucket.element_size()

    plan = TensorPlan(grads, dsts, chunk_elems=args.chunk_elems)
    # Untimed: the W warm-up steps asked for, preceded by enough further steps (about 25 ms of work)
    # that the GPU has left its idle clocks before anything is timed.
    for _ in range(max(0, 60 - args.warmup) + args.warmup):
        plan.fused_step(cfg.inv_scale, cfg.max_norm)
    torch.cuda.synchronize()
    # Timed region: HIP events (recorded by the library on the launch stream) bracket only the
    # dominant kernel, the write pass, and only on every fifth step: each record costs a few
    # microseconds of stream time, which would otherwise be part of every step measured here.
    stride = min(5, max(1, args.steps))
    sampled = (args.steps + stride - 1) // stride
    plan.plan.enable_timing(-sampled)
    plan.plan.timing_stride(stride)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        plan.fused_step(cfg.inv_scale, cfg.max_norm)
    done = torch.cuda.Event()
    done.record()
    while not done.query():       # poll: a blocking wait adds its wake-up latency to the last step
        pass
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    res = plan.result()
    write_only = [plan.plan.read_timing(i) for i in range(sampled)]
    plan.plan.timing_stride(1)
    # A second, untimed loop brackets all three stages for the breakdown.
    plan.plan.enable_timing(args.steps)
    for _ in range(args.steps):
        plan.fused_step(cfg.inv_scale, cfg.max_norm)
    torch.cuda.synchronize()
    per_kernel = [plan.plan.read_timing(i) for i in range(args.steps)]
    plan.plan.enable_timing(0)

    step_s = elapsed / args.steps
    clipped = bool(res.clipped)
    step_bytes = ((2 * s + d) if clipped else (s + d)) * n
    value = step_bytes / step_s / 1e9

    # dominant kernel: the write pass (re-read s*N, write d*N)
    write_ms = sum(k[2] for k in write_only) / len(write_only)
    reduce_ms = sum(k[0] for k in per_kernel) / len(per_kernel)
    final_ms = sum(k[1] for k in per_kernel) / len(per_kernel)
    write_bytes = (s + d) * n
    achieved = write_bytes / (write_ms * 1e-3) / 1e9
    roofline = {
        "bound": "hbm", "kernel": "pass_kernel<write, streaming>", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
        "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
        "traffic": MEASURED_TRAFFIC_BYTES.get(cfg.key),
        "algorithmic_bytes_per_launch": write_bytes, "avg_launch_ms": round(write_ms, 4),
        "launches_timed": len(write_only),
        "other_kernels": {
            "pass_kernel<reduce>": {"avg_launch_ms": round(reduce_ms, 4), "algorithmic_bytes_per_launch": s * n,
                                    "achieved": round(s * n / (reduce_ms * 1e-3) / 1e9, 1)},
            "finalize_tensors_kernel+finalize_total_kernel": {"avg_launch_ms": round(final_ms, 4)},
            "note": "from a second, untimed loop of the same steps with all stages bracketed",
        },
    }

    out = {
        "metric": "achieved HBM GB/s (% of roofline) for fused unscale+norm+clip+pack per step",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": f"{cfg.grad_dtype}->{cfg.bucket_dtype} (fp32 arithmetic)",
        "data": "synthetic",
        "config": {"workload": cfg.key, "description": cfg.description, "tensors": len(grads), "elements": n,
                   "src_bytes_per_elem": s, "dst_bytes_per_elem": d,
                   "algorithmic_bytes_per_step": step_bytes, "clipped": clipped, "overflow": int(res.overflow),
                   "norm": res.norm, "coef": res.coef, "seed": args.seed,
                   "chunk_elems": plan.plan.chunk_elems, "chunks": plan.plan.num_chunks,
                   "untimed_steps_before_timing": max(0, 60 - args.warmup) + args.warmup},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "elements_per_s": round(n / step_s, 1),
        "roofline": roofline,
    }
    plan.close()
    del grads, bucket, dsts
    torch.cuda.empty_cache()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, args.seed, args.cpu_seconds)
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
