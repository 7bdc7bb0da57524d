"""CPU oracle for the per-step parameter/gradient path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module;
it exists so that tests, the smoke check and the benchmark's CPU-baseline leg
have an independent statement of what the reference computes.  Each function
restates, op for op, the ATen call sequence the reference issues on CPU tensors
(the reference itself falls back to CPU tensors when no accelerator is present,
``src/torch/TorchUtil.cpp:1467-1471``, ``src/comp/ParamStorage.cpp:62-66``) and
cites the lines it follows.  Where the arithmetic belongs to NVIDIA Apex
(commit f3a960f80244cf9e80558ab30f7f7e8cbf03c0a0, pinned by
``docker/ubuntu/runtime/Dockerfile:13`` and absent from the reference tree) the
published algorithm of ``amp_C.multi_tensor_scale`` is restated instead.

Pinning status (what independent evidence fixes each function; the checks live
in ``tests/test_oracle_pins.py``):

* ``calc_aligned_num_elems`` / ``segment_layout`` / ``bucket_layout``: integer
  closed forms + brute-force invariants + the worked examples fixed by the
  formula (fp16, 1000 elements over 8 ranks, ...).
* ``consolidate`` / ``zero_staging_pack`` / ``dist_param_*``: bit-exact against
  plain concatenation / slicing and the reference test's own invariant
  ``segment == full.flatten()[range]`` (``test/common.py:57-63``).
* ``unscale_and_check``: IEEE closed form (power-of-two scales are exact),
  numpy integer-bit widening, and torch's own
  ``_amp_foreach_non_finite_check_and_unscale_``.
* ``cast``: numpy ``astype(float16)`` (IEEE RNE) and an integer-arithmetic RNE
  bf16 rounding.
* ``grad_global_l2_norm`` / ``clip_grad_norm``: float64 numpy brute force and
  closed forms for constant tensors, threshold behaviour by special cases.  The
  per-tensor sums are accumulated in float64 and rounded to fp32 once; ATen's CPU
  fp32 accumulation (``per_tensor_norms_aten``) drifts by up to 1e-2 relative at
  these sizes and is only the timed baseline.
* ``LossScalerState.update_scale``: Apex's published ``LossScaler.update_scale``
  (``apex/amp/scaler.py`` at the pinned commit: halve on overflow, floor at
  ``min_loss_scale``, zero the clean-step counter; otherwise count the step;
  double, capped at ``max_loss_scale``, when the counter reaches ``scale_window``;
  a static scale never skips) restated, and pinned by hand-written sequences of
  (scale, counter, skip) literals.  The rank-sharing wrapper
  ``patched_update_scale`` follows ``pyrannc/amp/__init__.py:44-65`` and is pinned
  by case analysis.
* ``reference_step_cpu`` (the timed CPU baseline): flag exact, norm to 1e-4 (it
  sums in ATen's fp32) and bucket bit-exact given its own coefficient against
  ``fused_step`` on a mixed list, an overflow case and a no-clip case.
* Parity unpinned: only ``unscale_accumulate`` versus Apex's
  ``multi_tensor_axpby`` (whether that kernel contracts multiply and add into one
  fma is not visible from the reference tree); it is pinned against numpy's two
  roundings instead.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

DTYPES: Dict[str, torch.dtype] = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
ELEM_SIZE: Dict[str, int] = {"f32": 4, "f16": 2, "bf16": 2}


# --------------------------------------------------------------------------- layout

def calc_aligned_num_elems(numel: int, elem_size: int, split_num: int) -> int:
    """``calcAlignedNumElems`` (``src/torch/TorchUtil.cpp:1579-1591``): round ``numel`` up
    to a multiple of ``16 / elem_size * split_num`` elements."""
    alignment_base = 16
    assert alignment_base % elem_size == 0
    unit = alignment_base // elem_size * split_num
    n_blocks = numel // unit if numel % unit == 0 else numel // unit + 1
    return n_blocks * unit


@dataclass(frozen=True)
class SegmentLayout:
    aligned_size: int
    segment_size: int
    offsets: Tuple[int, ...]
    src_sizes: Tuple[int, ...]

    def range(self, index: int) -> Tuple[int, int]:
        """``getSegmentRange`` (``src/comp/DistributedParamLocatorBase.cpp:64-74``)."""
        return self.offsets[index], self.offsets[index] + self.src_sizes[index]


def segment_layout(numel: int, elem_size: int, nranks: int) -> SegmentLayout:
    """``DistributedParamLocatorBase::doRegister``
    (``src/comp/DistributedParamLocatorBase.cpp:18-27``)."""
    aligned = calc_aligned_num_elems(numel, elem_size, nranks)
    seg = aligned // nranks
    offsets: List[int] = []
    src_sizes: List[int] = []
    offset = 0
    for _ in range(nranks):
        offsets.append(offset)
        src = min(numel - offset, seg)
        src_sizes.append(src)
        offset += src
    return SegmentLayout(aligned, seg, tuple(offsets), tuple(src_sizes))


def bucket_layout(numels: Sequence[int], dtypes: Sequence[str]) -> Tuple[List[int], Dict[str, int]]:
    """``GradConsolidation`` constructor (``src/comp/ParamStorage.cpp:48-57``): per dtype, the
    element offset of parameter i is the running sum of the numels of earlier parameters of
    the same dtype, in the given order, with no padding.  Returns (offset per param,
    bucket length per dtype)."""
    running: Dict[str, int] = {}
    offsets: List[int] = []
    for n, dt in zip(numels, dtypes):
        assert dt in DTYPES  # ParamStorage.cpp:51-53
        offsets.append(running.get(dt, 0))
        running[dt] = running.get(dt, 0) + int(n)
    return offsets, running


# --------------------------------------------------------------------------- pack

def consolidate(grads: Sequence[Optional[torch.Tensor]], numels: Sequence[int],
                dtypes: Sequence[str]) -> Dict[str, torch.Tensor]:
    """``GradConsolidation::consolidate`` (``src/comp/ParamStorage.cpp:135-178``) from a cold
    start: buckets are ``torch::zeros`` (``:59-75``); a defined grad is ``copy_``-ed into its
    view (``:165``); an undefined one leaves its view zero (``:169-175``)."""
    offsets, lengths = bucket_layout(numels, dtypes)
    buckets = {dt: torch.zeros(n, dtype=DTYPES[dt]) for dt, n in lengths.items()}
    for g, n, dt, off in zip(grads, numels, dtypes, offsets):
        if g is None:
            continue
        assert g.numel() == n
        buckets[dt].narrow(0, off, n).view(g.shape).copy_(g)
    return buckets


def zero_staging_pack(grad: torch.Tensor, nranks: int, to_fp32: bool) -> torch.Tensor:
    """ZeRO reduce-scatter staging (``src/comp/ParamStorage.cpp:479-493``): a zero-filled
    buffer of ``calcAlignedNumElems`` elements, fp32 when masters are all-reduced and the
    param is half, whose first ``numel`` elements are ``copy_``-ed (cast) from the grad."""
    aligned = calc_aligned_num_elems(grad.numel(), grad.element_size(), nranks)
    dt = torch.float32 if (to_fp32 and grad.dtype == torch.float16) else grad.dtype
    buf = torch.zeros(aligned, dtype=dt)
    buf.narrow(0, 0, grad.numel()).copy_(grad.flatten())
    return buf


def zero_copy_back(grad: torch.Tensor, out_buf: torch.Tensor, offset: int) -> None:
    """After the reduce-scatter (``src/comp/ParamStorage.cpp:419-427``): copy
    ``min(out_buf.numel, grad.numel - offset)`` elements back into ``grad.flatten()[offset:]``."""
    length = min(out_buf.numel(), grad.numel() - offset)
    if length > 0:
        grad.view(-1).narrow(0, offset, length).copy_(out_buf.narrow(0, 0, length))


# --------------------------------------------------------------------------- unscale + flag

def unscale_and_check(model_grads: Sequence[torch.Tensor], inv_scale: float,
                      out_dtype: torch.dtype = torch.float32) -> Tuple[List[torch.Tensor], int]:
    """Apex ``multi_tensor_scale`` as called by ``LossScaler.unscale`` (external; caller in the
    reference: ``test/common.py:98-101``): ``out[i] = float(in[i]) * scale`` as one fp32
    multiply, stored in ``out_dtype``; the int flag becomes 1 iff any *input* element is
    +-inf or NaN."""
    scale = torch.tensor(inv_scale, dtype=torch.float32)
    outs: List[torch.Tensor] = []
    overflow = 0
    for g in model_grads:
        gf = g.to(torch.float32)
        if g.numel() and not bool(torch.isfinite(gf).all()):
            overflow = 1
        outs.append((gf * scale).to(out_dtype))
    return outs, overflow


# --------------------------------------------------------------------------- norm + clip

def per_tensor_norms_aten(grads: Sequence[Optional[torch.Tensor]]) -> List[Optional[float]]:
    """The literal reference op, ``grad.norm(2, ScalarType::Float).item<float>()``
    (``src/comp/ParamStorage.cpp:767-770``), as ATen's CPU kernel evaluates it.  Its fp32
    accumulation is close to sequential and drifts by ~1e-5 relative at 1e6 elements and
    ~2e-3 at 3e7 (measured), so it cannot arbitrate a 1e-6 bar; it is kept for the timed
    CPU baseline and as a loose cross-check."""
    out: List[Optional[float]] = []
    for g in grads:
        out.append(None if g is None else float(g.norm(2, dtype=torch.float32).item()))
    return out


def per_tensor_norms(grads: Sequence[Optional[torch.Tensor]]) -> List[Optional[float]]:
    """Per-tensor L2 norm as ``norm(2, ScalarType::Float).item<float>()`` defines it
    (``src/comp/ParamStorage.cpp:767-770``): sqrt of the sum of squares of the fp32 values,
    delivered as an fp32 number.  The sum is taken in float64 here so that the only rounding
    left is the final one to fp32 - the value every fp32 accumulation order approximates."""
    out: List[Optional[float]] = []
    for g in grads:
        if g is None:
            out.append(None)
            continue
        sq = float(g.detach().to(torch.float32).double().square().sum().item())
        out.append(float(torch.tensor(math.sqrt(sq), dtype=torch.float64).to(torch.float32).item()))
    return out


def grad_global_l2_norm(grads: Sequence[Optional[torch.Tensor]]) -> float:
    """``ParamStorage::calcGradGlobalL2Norm`` (``src/comp/ParamStorage.cpp:747-819``) at world
    size 1: per-tensor fp32 norms, then ``sqrt(sum double(n)^2)`` in the given (name-sorted)
    order."""
    norm_sq_sum = 0.0
    for n in per_tensor_norms(grads):
        if n is not None:
            norm_sq_sum += n * n          # ParamStorage.cpp:813-814, double arithmetic
    return math.sqrt(norm_sq_sum)


def clip_coefficient(global_norm: float, max_grad_norm: float) -> Optional[float]:
    """``ParamStorage::clipGradNorm`` (``src/comp/ParamStorage.cpp:723-725, 740``).
    ``max_grad_norm`` crosses the binding as a C ``float`` (``src/main.cpp:339-342``).
    Returns the double coefficient, or None when no clipping happens."""
    max_f = float(torch.tensor(max_grad_norm, dtype=torch.float32).item())
    g = global_norm + 1e-6
    if g > max_f:
        return max_f / g
    return None


def clip_grad_norm(grads: Sequence[Optional[torch.Tensor]], max_grad_norm: float) -> Tuple[float, Optional[float]]:
    """Norm + in-place clip.  ``grad.mul_(double)`` on an fp32 tensor multiplies by the scalar
    narrowed to fp32; on fp16/bf16 it computes in fp32 and rounds to the tensor dtype
    (``src/comp/ParamStorage.cpp:741``).  Returns (global norm, coefficient or None)."""
    norm = grad_global_l2_norm(grads)
    coef = clip_coefficient(norm, max_grad_norm)
    if coef is not None:
        for g in grads:
            if g is not None:
                g.mul_(coef)
    return norm, coef


# --------------------------------------------------------------------------- fused step

@dataclass
class FusedStepResult:
    buckets: Dict[str, torch.Tensor]   # packed destination, per bucket dtype
    overflow: int
    norm: float                        # double, as calc_grad_norm returns it
    coef: Optional[float]              # None when not clipped (or skipped on overflow)
    tensor_norms: List[float]


def fused_step(grads: Sequence[torch.Tensor], bucket_dtypes: Sequence[str], inv_scale: float,
               max_grad_norm: float) -> FusedStepResult:
    """The reference's per-step sequence on one rank, start to end:

    1. Apex unscale of the model grads into the master grads, which alias views of the
       consolidated bucket (``src/comp/ParamStorage.cpp:139-151`` points the master ``.grad``
       at its bucket view; the unscale kernel then writes there) -> ``unscale_and_check``
       + ``consolidate``;
    2. if the flag is set the step is skipped (no clip);
    3. otherwise ``clip_grad_norm`` on the bucket views.
    """
    numels = [g.numel() for g in grads]
    offsets, _ = bucket_layout(numels, bucket_dtypes)
    outs: List[torch.Tensor] = []
    overflow = 0
    for g, bdt in zip(grads, bucket_dtypes):
        o, f = unscale_and_check([g], inv_scale, DTYPES[bdt])
        outs.append(o[0])
        overflow |= f
    buckets = consolidate(outs, numels, bucket_dtypes)
    views = [buckets[bdt].narrow(0, off, n) for bdt, off, n in zip(bucket_dtypes, offsets, numels)]
    tnorms = [n if n is not None else 0.0 for n in per_tensor_norms(views)]
    norm = math.sqrt(sum(n * n for n in tnorms))
    coef = None
    if not overflow:
        coef = clip_coefficient(norm, max_grad_norm)
        if coef is not None:
            for v in views:
                v.mul_(coef)
    return FusedStepResult(buckets, overflow, norm, coef, tnorms)


# --------------------------------------------------------------------------- casts / masters

def cast(t: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """``Tensor.to(dtype)`` / ``copy_`` across dtypes (``DistributedParamLocator.cpp:76``,
    ``ParamStorage.cpp:493``, Apex master<->model copies): widening is exact, narrowing is
    IEEE round-to-nearest-even."""
    return t.to(dtype)


def master_from_model(model_params: Sequence[torch.Tensor]) -> List[torch.Tensor]:
    """Apex O2 master creation: ``param.detach().clone().float()``."""
    return [p.detach().clone().float() for p in model_params]


def master_copy_back(masters: Sequence[torch.Tensor], model_params: Sequence[torch.Tensor]) -> None:
    """Apex post-step master -> model copy (``multi_tensor_scale`` with scale 1.0)."""
    for m, p in zip(masters, model_params):
        p.copy_(m)


# --------------------------------------------------------------------------- dist params

class DistParamOracle:
    """``DistributedParamLocator`` (``src/comp/DistributedParamLocator.cpp:14-83``) and
    ``DistributedParamLocatorBase::gather`` (``DistributedParamLocatorBase.cpp:96-153``) for
    rank ``rank`` of ``nranks``; ``load`` takes every rank's oracle to play the all-gather."""

    def __init__(self, rank: int = 0, nranks: int = 1):
        self.rank, self.nranks = rank, nranks
        self.layouts: Dict[int, SegmentLayout] = {}
        self.parts: Dict[int, torch.Tensor] = {}
        self.shapes: Dict[int, Tuple[int, ...]] = {}

    def store(self, pid: int, param: torch.Tensor) -> torch.Tensor:
        lay = segment_layout(param.numel(), param.element_size(), self.nranks)
        self.layouts[pid] = lay
        self.shapes[pid] = tuple(param.shape)
        off, src = lay.offsets[self.rank], lay.src_sizes[self.rank]
        part = torch.zeros(src, dtype=param.dtype)
        if src > 0:
            part.copy_(torch.flatten(param).narrow(0, off, src))
        self.parts[pid] = part
        return part

    def set(self, pid: int, src_full: torch.Tensor) -> None:
        lay = self.layouts[pid]
        off, src = lay.offsets[self.rank], lay.src_sizes[self.rank]
        if src > 0:
            self.parts[pid].copy_(torch.flatten(src_full).narrow(0, off, src))

    def set_scalar_type(self, pid: int, dtype: torch.dtype) -> None:
        self.parts[pid] = self.parts[pid].to(dtype)

    def get_range(self, pid: int) -> Tuple[int, int]:
        return self.layouts[pid].range(self.rank)

    @staticmethod
    def load(pid: int, ranks: Sequence["DistParamOracle"]) -> torch.Tensor:
        lay = ranks[0].layouts[pid]
        seg, n = lay.segment_size, len(ranks)
        buf = torch.zeros(seg * n, dtype=ranks[0].parts[pid].dtype)
        for r, o in enumerate(ranks):
            send = torch.zeros(seg, dtype=buf.dtype)
            send.narrow(0, 0, o.parts[pid].numel()).copy_(o.parts[pid])
            buf.narrow(0, seg * r, seg).copy_(send)
        shape = ranks[0].shapes[pid]
        total = 1
        for s in shape:
            total *= s
        return buf.narrow(0, 0, total).view(shape)


def align_buffer(param: torch.Tensor, nranks: int) -> torch.Tensor:
    """``DistributedGradLocator::alignBuffer`` (``src/comp/DistributedGradLocator.cpp:50-63``):
    zero buffer of the aligned size holding the flattened param at its head."""
    aligned = calc_aligned_num_elems(param.numel(), param.element_size(), nranks)
    buf = torch.zeros(aligned, dtype=param.dtype)
    buf.narrow(0, 0, param.numel()).copy_(param.flatten())
    return buf


# --------------------------------------------------------------------------- loss scaler

@dataclass
class LossScalerState:
    """Apex ``LossScaler`` state and ``update_scale`` (external: ``apex/amp/scaler.py`` at the
    commit pinned by ``docker/ubuntu/runtime/Dockerfile:13``; the reference reads and writes
    ``_loss_scale`` / ``_unskipped`` and wraps ``update_scale``, ``pyrannc/amp/__init__.py:45-65``).
    Published algorithm: on overflow with a dynamic scale the scale is halved (not below
    ``min_loss_scale`` when one is given), the clean-step counter is zeroed and the step is
    skipped; otherwise the counter is incremented; when the counter reaches ``scale_window``
    the scale is doubled (not above ``max_loss_scale``) and the counter zeroed.  A static scale
    never changes and never skips."""
    loss_scale: float = 2.0 ** 16
    unskipped: int = 0
    scale_window: int = 2000
    min_loss_scale: Optional[float] = None
    max_loss_scale: float = 2.0 ** 24
    dynamic: bool = True

    def update_scale(self, had_overflow: bool) -> bool:
        if had_overflow and self.dynamic:
            should_skip = True
            if self.min_loss_scale:
                self.loss_scale = max(self.min_loss_scale, self.loss_scale / 2.0)
            else:
                self.loss_scale = self.loss_scale / 2.0
            self.unskipped = 0
        else:
            should_skip = False
            self.unskipped += 1
        if self.unskipped == self.scale_window and self.dynamic:
            self.loss_scale = min(self.max_loss_scale, self.loss_scale * 2.0)
            self.unskipped = 0
        return should_skip


def patched_update_scale(state: LossScalerState, had_overflow_local: bool,
                         other_flags: Sequence[int] = (), other_scales: Sequence[int] = ()) -> bool:
    """``patch_amp_scaler`` wrapper (``pyrannc/amp/__init__.py:44-65``): run the scaler's own
    update, all-reduce-SUM the int flag, and when any rank overflowed all-reduce-MIN
    ``int(loss_scale)``, store it, zero ``_unskipped`` and report a skip."""
    had = state.update_scale(had_overflow_local)
    flag = (1 if had else 0) + sum(int(f) for f in other_flags)
    if flag > 0:
        scale = min([int(state.loss_scale)] + [int(s) for s in other_scales])
        state.loss_scale = scale
        state.unskipped = 0
        return True
    return False


# --------------------------------------------------------------------------- timed CPU baseline

def reference_step_cpu(model_grads: Sequence[torch.Tensor], master_grad_views: Sequence[torch.Tensor],
                       inv_scale: float, max_grad_norm: float) -> Tuple[int, float, Optional[float]]:
    """The reference's per-step work exactly as it issues it on CPU tensors, one ATen op per
    tensor, writing into preallocated bucket views (used as the timed CPU baseline):

    * unscale + flag per tensor (Apex ``multi_tensor_scale`` semantics; the reference's host
      loop shape is that of ``src/comp/ParamStorage.cpp:135-178``): ``view.copy_(g)`` casts
      into the fp32 master-grad view, ``mul_(inv_scale)``, ``isfinite().all()``;
    * ``norm(2, Float).item()`` per tensor, double sum (``:767-770, 809-818``);
    * ``mul_(max / (norm + 1e-6))`` per tensor when it exceeds the bound (``:721-745``).
    Returns (overflow, norm, coef)."""
    overflow = 0
    for g, v in zip(model_grads, master_grad_views):
        v.copy_(g)
        if inv_scale != 1.0:
            v.mul_(inv_scale)
        if g.numel() and not bool(torch.isfinite(v).all()):
            overflow = 1
    if overflow:
        return 1, float("nan"), None
    norm_sq = 0.0
    for v in master_grad_views:
        n = float(v.norm(2, dtype=torch.float32).item())
        norm_sq += n * n
    norm = math.sqrt(norm_sq)
    coef = clip_coefficient(norm, max_grad_norm)
    if coef is not None:
        for v in master_grad_views:
            v.mul_(coef)
    return 0, norm, coef


# --------------------------------------------------------------------------- accumulation

def unscale_accumulate(master_grads: Sequence[torch.Tensor], model_grads: Sequence[Optional[torch.Tensor]],
                       inv_scale: float) -> int:
    """Gradient accumulation under amp (Apex ``unscale_with_stashed``, external):
    ``master_grad += float(model_grad) * inv_scale`` in place, the product rounded to fp32 before
    the sum, the sum rounded to the master's dtype; returns the inf/NaN flag of the model grads.
    Whether Apex's kernel fuses the two operations is not visible from the reference tree:
    parity unpinned against Apex; pinned here against float64 arithmetic (the two roundings are
    reproduced by numpy in the test)."""
    scale = torch.tensor(inv_scale, dtype=torch.float32)
    overflow = 0
    for m, g in zip(master_grads, model_grads):
        if g is None:
            continue
        gf = g.to(torch.float32)
        if g.numel() and not bool(torch.isfinite(gf).all()):
            overflow = 1
        m.copy_((m.to(torch.float32) + gf * scale).to(m.dtype))
    return overflow


# --------------------------------------------------------------------------- shared parameters

def sum_clone_grads(param_grads: List[Optional[torch.Tensor]],
                    clone_grads: Sequence[Sequence[Optional[torch.Tensor]]]) -> None:
    """``TorchDriver::backward``, "backward_sum_paramgrad" (``src/torch/TorchDriver.cpp:781-822``):
    per shared parameter ``grad_sum = zeros; for each clone with a gradient: grad_sum.add_(g);
    g.zero_()`` in clone order, then ``grad.add_(grad_sum)`` or, when the parameter has no
    gradient yet, ``grad = copy of grad_sum``.  In place on the lists given.  Additions happen
    in the tensors' own dtype (ATen computes a 16-bit ``add_`` in fp32 and rounds once)."""
    for i, clones in enumerate(clone_grads):
        if not clones:
            continue
        ref = next((g for g in clones if g is not None), param_grads[i])
        if ref is None:
            continue
        grad_sum = torch.zeros_like(ref)
        for g in clones:
            if g is not None:
                grad_sum.add_(g)
                g.zero_()
        if param_grads[i] is not None:
            param_grads[i].add_(grad_sum)
        else:
            param_grads[i] = grad_sum.clone()
