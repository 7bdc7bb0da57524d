"""Mixed-precision support of the per-step path.

Two layers live here:

* the functions of ``pyrannc/amp/__init__.py`` with their signatures and behaviour:
  ``register_amp_params`` (``:13-18``), ``named_master_params`` (``:21-41``),
  ``patch_amp_scaler`` (``:44-65``), ``unset_master_grads`` (``:68-70``);
* the part of NVIDIA Apex amp (O2) those functions lean on, which is not in the reference
  tree (``docker/ubuntu/runtime/Dockerfile:13`` pins an external commit): fp32 master
  parameters, ``scale_loss``, a ``LossScaler`` whose ``unscale`` is the fused HIP kernel
  (Apex's ``multi_tensor_scale``: ``master_grad = float(model_grad) * (1 / scale)`` plus an
  inf/NaN flag), the skip of ``optimizer.step`` after an overflow and the master -> model
  copy after a step.  Attribute names follow Apex (``_amp_state.loss_scalers``,
  ``optimizer._amp_stash.all_fp16_params`` ...) because the reference reads them.

The dynamic loss-scale schedule is Apex's published ``LossScaler.update_scale`` (halve on
overflow with an optional floor, zero the clean-step counter; otherwise count the step and
double, up to ``max_loss_scale``, every ``scale_window`` clean steps; a static scale never
skips), restated here because Apex itself is not in the reference tree.

Gradient accumulation follows PyTorch's convention: a master gradient that is still defined
when a ``scale_loss`` context exits (no ``zero_grad`` since the last one) is accumulated into
(``master_grad += float(model_grad) * inv_scale``, Apex's ``unscale_with_stashed``); one that
is ``None`` is overwritten.
"""
from __future__ import annotations

import contextlib
from typing import Iterator, List, Optional, Tuple

import torch

from .. import _lib, _pyrannc
from ..multi_tensor import TensorPlan
from ..tensor_coll import _allreduce_min, _allreduce_sum

try:        # the compiled module: the steady state of a training loop walks its parameter lists in C++
    from .. import _ranncgrad as _native
except ImportError:
    _native = None


class _StepResult:
    __slots__ = ("norm", "coef", "overflow", "clipped", "skipped")

    def __init__(self, d) -> None:
        self.norm, self.coef, self.overflow = d["norm"], d["coef"], d["overflow"]
        self.clipped, self.skipped = d["clipped"], d["skipped"]


class _CompiledStepPlan:
    """The operations of ``TensorPlan`` that this module uses, over a ``GradPlan`` of the compiled module: a
    device table that follows the gradients of a fixed list of parameters without a Python loop over them."""

    def __init__(self, grad_plan) -> None:
        self.gp = grad_plan
        self.plan = self                       # ``unscale_plan.plan.result_device_ptr()``

    def step_begin(self, inv_scale: float) -> None:
        self.gp.step_begin(inv_scale)

    def step_begin_scaled(self, inv_scale_ptr: int) -> None:
        self.gp.step_begin_scaled(inv_scale_ptr)

    def step_finish(self, max_norm: float, flags: int = 0) -> None:
        self.gp.step_finish(max_norm, flags)

    def step_decide(self, max_norm: float, flags: int = 0) -> None:
        self.gp.step_decide(max_norm, flags)

    def step_apply_clip(self, max_norm: float, flags: int = 0) -> None:
        self.gp.step_apply_clip(max_norm, flags)

    def unscale_pack(self, inv_scale: float) -> None:
        self.gp.unscale_pack(inv_scale)

    def result(self) -> _StepResult:
        return _StepResult(self.gp.result())

    def result_device_ptr(self) -> int:
        return self.gp.result_device_ptr()

    def drop_sources(self) -> None:
        self.gp.drop_sources()

    def is_open(self) -> bool:
        return self.gp.is_open()

    def close(self) -> None:
        self.gp.close()


class _CompiledLists:
    """The half parameters, their fp32 masters and the masters' gradient views as lists held by the compiled
    module, and the table from the half parameters' gradients to those views."""

    def __init__(self, stash: "_AmpStash") -> None:
        self.n = len(stash.all_fp16_params)
        self.dtype = stash.all_fp16_params[0].dtype
        self.half = _native.TensorList(stash.all_fp16_params)
        self.masters = _native.TensorList(stash.all_fp32_from_fp16_params)
        self.views = _native.TensorList(stash.master_grad_views)
        self.grad_plan = _native.GradPlan(self.half, self.views)
        self.plan = _CompiledStepPlan(self.grad_plan)


class _AmpState:
    def __init__(self) -> None:
        self.loss_scalers: List["LossScaler"] = []
        self.opt_level: Optional[str] = None


_amp_state = _AmpState()


class _AmpStash:
    """The lists Apex hangs on ``optimizer._amp_stash`` (read at ``pyrannc/amp/__init__.py:9-11``)."""

    def __init__(self) -> None:
        self.all_fp16_params: List[torch.Tensor] = []
        self.all_fp32_from_fp16_params: List[torch.Tensor] = []
        self.all_fp32_from_fp32_params: List[torch.Tensor] = []
        self.already_patched = False
        self.lazy_init_called = False
        self.unscale_plan: Optional[TensorPlan] = None
        self.unscale_cache = None          # param_storage._PlanCache holding unscale_plan
        self.optimizer_reads_model_grads = False    # a fused optimizer: its step kernel unscales and clips itself
        self.step_flags = _lib.RG_STEP_DEFAULT      # RG_STEP_IGNORE_OVERFLOW under a static loss scale
        self.copy_back_plan: Optional[TensorPlan] = None
        self.pending_finish = False        # fused mode: the write pass has not run yet
        self.pending_inv_scale = 1.0       #   ... the 1/loss_scale its read pass ran with
        self.pending_masters: List[torch.Tensor] = []      #   ... the masters and model gradients it covers
        self.pending_model_grads: List[torch.Tensor] = []
        self.decided_max_norm: Optional[float] = None      # clip_grad_norm asked for while the write is pending
        self.fused = False
        self._last_result = None           # rg_step_result of the last unscale, or the table to read it from
        self._last_result_plan = None
        # fused mode picks its strategy per step from what the last step did: when it clipped, read pass now and
        # one deferred write pass that applies the coefficient ((2s + d) bytes per element); when it did not, one
        # eager pass that writes while it sums ((s + d)), with an in-place multiply only if this step clips after all
        self.expect_clip = True
        self.clip_decided = False          # a clip decision was taken on the device since the last unscale
        self.sums_cover_all = False        # the eager pass's sums are the norm of every gradient clip_grad_norm covers
        # packed fp32 bucket the master gradients are views of (the reference's
        # consolidated_master_grads_, src/comp/ParamStorage.cpp:68-70, 92-97): stable
        # addresses, so the device table is built once
        self.master_grad_bucket: Optional[torch.Tensor] = None
        self.master_grad_views: List[torch.Tensor] = []
        # fp32 parameters (batch norm under O2): tables for the in-place unscale of fresh
        # gradients and for adding fresh gradients onto stashed ones (gradient accumulation)
        self.fp32_unscale_plans = None
        self.fp32_accumulate_plans = None
        self.device_scaler = None          # the LossScaler, when its schedule lives on the device
        self.compiled: Optional[_CompiledLists] = None     # made at the first steady-state exit of scale_loss
        self.feed = None                   # the GradPlan whose held gradients the pending write / step reads, if any


def _get_last_result(stash: _AmpStash):
    if stash._last_result is None and stash._last_result_plan is not None and stash._last_result_plan.is_open():
        stash._last_result = stash._last_result_plan.result()
    return stash._last_result


def _set_last_result(stash: _AmpStash, value) -> None:
    stash._last_result, stash._last_result_plan = value, None


#: ``rg_step_result`` of the last unscale.  Under a dynamic loss scale it is read at every ``scale_loss`` exit (the
#: schedule needs the flag); under a static one nothing on the host depends on it, so it is only fetched - from the
#: table's result block as the device holds it then - when somebody looks.
_AmpStash.last_result = property(_get_last_result, _set_last_result)


class LossScaler:
    """Loss scale with the fused unscale + overflow check."""

    def __init__(self, loss_scale="dynamic", init_scale: float = 2.0 ** 16, scale_factor: float = 2.0,
                 scale_window: int = 2000, min_loss_scale: Optional[float] = None,
                 max_loss_scale: float = 2.0 ** 24) -> None:
        self.dynamic = loss_scale == "dynamic"
        self._loss_scale = min(max_loss_scale, init_scale) if self.dynamic else float(loss_scale)
        self._scale_seq_len = scale_window
        self._scale_factor = scale_factor
        self._min_loss_scale = min_loss_scale
        self._max_loss_scale = max_loss_scale
        self._unskipped = 0
        self._has_overflow = False
        # the schedule on the device (``amp.initialize(..., device_loss_scale=True)``): 32 bytes of state that the
        # unscale, the optimizer step and a one-thread update kernel read and write; the host only looks on request
        self.state: Optional[torch.Tensor] = None
        self.update_flags = _lib.RG_SCALER_DYNAMIC

    @property
    def on_device(self) -> bool:
        return self.state is not None

    def to_device(self, device: torch.device) -> None:
        """Write the schedule, as the attributes of this object describe it, into device memory (at set-up, and again
        when those attributes were changed by hand)."""
        if not self.dynamic:
            raise ValueError("a static loss scale has no schedule to keep on the device")
        from ..multi_tensor import stream_handle
        if self.state is None:
            self.state = torch.zeros(_lib.SCALER_STATE_BYTES // 4, dtype=torch.float32, device=device)
        _lib.scaler_init(self.state.data_ptr(), float(self._loss_scale), float(self._min_loss_scale or 0.0),
                         float(self._max_loss_scale), int(self._scale_seq_len), float(self._scale_factor),
                         device.index or 0, stream_handle(device))
        self.scale_on_device = self.state[0]            # 0-dim view: ``loss * scale`` without a host read

    @property
    def inv_scale_ptr(self) -> int:
        return self.state.data_ptr() + _lib.SCALER_INV_SCALE_OFFSET

    def device_state(self) -> "_lib.ScalerState":
        """The schedule's state as the device holds it now (a host read: waits for the stream)."""
        return _lib.ScalerState.from_buffer_copy(self.state.cpu().numpy().tobytes())

    def update_on_device(self, result_ptr: int) -> None:
        """Queue the schedule's update for the step whose flag is in the result block at ``result_ptr``."""
        from ..multi_tensor import stream_handle
        dev = self.state.device
        _lib.scaler_update(self.state.data_ptr(), result_ptr, self.update_flags, dev.index or 0, stream_handle(dev))

    def loss_scale(self) -> float:
        if self.state is not None:
            return float(self.device_state().loss_scale)
        return self._loss_scale

    def clear_overflow_state(self) -> None:
        self._has_overflow = False

    def unscale(self, stash: _AmpStash, model_grads: List[torch.Tensor], master_grads: List[torch.Tensor],
                accumulate: bool = False, all_params: bool = False, plan=None, covers_all: bool = False) -> None:
        """``master_grad = float(model_grad) * (1 / scale)`` for every pair in one launch, with the
        inf/NaN flag and - for free - the gradient norm.  In fused mode only the read pass runs
        here; the values are written by ``finish_unscale``.  ``accumulate`` adds to the master
        gradients instead of overwriting them (always eager).  ``all_params``: the lists are every half
        parameter's gradient and every master's bucket view, in stash order - the shape of the table is then known
        to be last time's and only the gradients' addresses are compared."""
        # One device table for the whole run: when backward hands back gradients at new addresses (same
        # sizes and dtypes) the table is re-pointed in place, stream ordered - nothing is freed or allocated.
        if stash.unscale_cache is None:
            from ..param_storage import _PlanCache
            stash.unscale_cache = _PlanCache()
        if stash.clip_decided:
            # what the last step decided picks this step's strategy; it is read from the table that took the
            # decision, before the cache may replace that table by a new one (not at all when the optimizer reads
            # the model gradients itself: then there is one strategy, and the host does not wait for the device)
            if (stash.unscale_plan is not None and stash.unscale_plan.is_open()
                    and not (stash.fused and stash.optimizer_reads_model_grads)):
                stash.expect_clip = bool(stash.unscale_plan.result().clipped)
            stash.clip_decided = False
        # a new table is tuned on the spot, unless the master gradients hold values that are about to be added to
        if plan is not None:
            stash.unscale_plan = plan          # a table of the compiled module, already bound to this step's gradients
        elif all_params:
            stash.unscale_plan = stash.unscale_cache.get_same_shapes("all", model_grads, master_grads, tune_new=not accumulate)
        else:
            stash.unscale_plan = stash.unscale_cache.get(model_grads, master_grads, tune_new=not accumulate)
        deferred = not accumulate and stash.fused and (stash.expect_clip or stash.optimizer_reads_model_grads)
        # with the schedule on the device the deferred route never needs the scale on the host; the others do
        inv = None if (self.on_device and deferred) else 1.0 / self.loss_scale()
        stash.sums_cover_all = False
        with torch.no_grad():
            if accumulate:
                # one pass: unscale, flag, add, and the sums of the *results* - when the pass covers every master
                # gradient, clip_grad_norm needs no pass of its own to know the norm (clip_from_unscale_sums)
                stash.unscale_plan.unscale_accumulate(inv)
                stash.sums_cover_all = stash.fused and covers_all
            elif deferred:
                if inv is None:
                    stash.unscale_plan.step_begin_scaled(self.inv_scale_ptr)
                else:
                    stash.unscale_plan.step_begin(inv)
                stash.pending_finish = True
                stash.pending_inv_scale = inv
                stash.decided_max_norm = None
            else:
                stash.unscale_plan.unscale_pack(inv)
                stash.sums_cover_all = stash.fused
        if self.on_device:
            stash._last_result, stash._last_result_plan = None, stash.unscale_plan     # the device decides; nobody waits
        elif self.dynamic:
            stash.last_result = stash.unscale_plan.result()      # one host read, like the reference's .item()
            if stash.last_result.overflow:
                self._has_overflow = True
        else:
            stash._last_result, stash._last_result_plan = None, stash.unscale_plan     # a static scale never skips
        if not stash.pending_finish:
            # every kernel that reads the model gradients is queued: let go of them, so that backward
            # finds their memory free again (and, in the steady state, at the same addresses)
            stash.unscale_plan.drop_sources()
            stash.pending_model_grads = []
            stash.feed = None

    def update_scale(self) -> bool:
        """Returns True when the step must be skipped.  Own schedule (see module docstring)."""
        if self._has_overflow and self.dynamic:
            should_skip = True
            self._loss_scale = self._loss_scale / 2.0
            if self._min_loss_scale:
                self._loss_scale = max(self._min_loss_scale, self._loss_scale)
            self._unskipped = 0
        else:
            should_skip = False
            self._unskipped += 1
        if self._unskipped == self._scale_seq_len and self.dynamic:
            self._loss_scale = min(self._max_loss_scale, self._loss_scale * self._scale_factor)
            self._unskipped = 0
        return should_skip


def initialize(model: torch.nn.Module, optimizer: torch.optim.Optimizer, opt_level: str = "O2",
               loss_scale="dynamic", max_loss_scale: float = 2.0 ** 24, min_loss_scale: Optional[float] = None,
               half_dtype: torch.dtype = torch.float16, fused: bool = True, device_loss_scale: bool = False
               ) -> Tuple[torch.nn.Module, torch.optim.Optimizer]:
    """O2-style set-up: the model's floating-point parameters (batch-norm layers excepted)
    become ``half_dtype``; the optimizer is re-pointed at fp32 masters created as
    ``param.detach().clone().float()``; ``optimizer.step`` is wrapped to skip once after an
    overflow and to copy masters back into the model afterwards.

    ``fused=True`` (the default) defers the write of the unscaled master gradients from the ``scale_loss``
    exit to the next ``clip_grad_norm`` / ``optimizer.step``, so that unscale, norm, clip and pack move
    ``(2s + d)`` bytes per element (``(s + d)`` when the previous step did not clip) instead of the
    ``(s + d) + 3d`` of an eager unscale followed by a clip of the fp32 gradients.  Everything that hands
    master gradients out - ``amp.master_params``, ``RaNNCModule.get_param_grad`` / ``_calc_grad_norm`` /
    ``clip_grad_norm``, ``optimizer.step`` - completes the write first; only code that reaches into
    ``optimizer._amp_stash`` directly sees stale values until then (call ``amp.finish_unscale(optimizer)``).
    ``fused=False`` writes them at the ``scale_loss`` exit, as Apex does.
    When the optimizer is one of ``rannc_amd.fused_optim`` (and every stepped parameter is half
    precision) the write never happens: ``clip_grad_norm`` only takes the clip decision on the
    device and ``optimizer.step`` reads the scaled model gradients, applies ``1/scale`` and the
    clip coefficient, updates the masters and writes the model copies in one kernel.  Anything
    that looks at master gradients first writes them, and the step then takes them from memory.

    ``device_loss_scale=True`` (dynamic scale, ``fused=True``, a ``FusedAdam`` / ``FusedAdamW`` - made ``capturable``
    here): the loss scale and its schedule live in 32 bytes of device memory.  ``scale_loss`` multiplies the loss by
    the scale where it is, the unscale and the optimizer step read ``1 / scale`` there, an overflow gates the step
    on the device, and one thread updates the schedule after ``optimizer.step`` (Apex updates it at the context
    exit; with one backward per step that is the same sequence).  Nothing in a training step then waits for the
    device; ``scaler.loss_scale()`` and ``stash.last_result`` read it back on request.  Every stepped parameter
    must be half precision (no fp32 batch-norm parameters)."""
    if opt_level != "O2":
        raise ValueError("only opt_level='O2' (fp32 masters for half parameters) is provided")
    bn = torch.nn.modules.batchnorm._BatchNorm
    for mod in model.modules():
        if isinstance(mod, bn):
            continue
        for p in mod.parameters(recurse=False):
            if p.dtype == torch.float32:
                p.data = p.data.to(half_dtype)
        for name, b in mod.named_buffers(recurse=False):
            if b.dtype == torch.float32:
                mod._buffers[name] = b.to(half_dtype)
    stash = _AmpStash()
    stash.fused = fused
    stash.optimizer_reads_model_grads = bool(getattr(optimizer, "reads_grad_sources", False))
    optimizer._amp_stash = stash
    scaler = LossScaler(loss_scale, min_loss_scale=min_loss_scale, max_loss_scale=max_loss_scale)
    # A static scale never skips a step (Apex): an overflow must then reach the master gradients and the
    # optimizer as the inf/NaN it is - in fused mode too - instead of leaving last step's values in place.
    # RG_STEP_IGNORE_OVERFLOW makes the deferred write / the clip decision behave exactly like
    # ParamStorage::clipGradNorm on gradients that contain them (src/comp/ParamStorage.cpp:723-742).
    stash.step_flags = _lib.RG_STEP_DEFAULT if scaler.dynamic else _lib.RG_STEP_IGNORE_OVERFLOW
    if device_loss_scale:
        if not (scaler.dynamic and fused and stash.optimizer_reads_model_grads and hasattr(optimizer, "capturable")):
            raise ValueError("device_loss_scale needs a dynamic loss scale, fused=True and a FusedAdam / FusedAdamW")
        if any(p.dtype == torch.float32 for g in optimizer.param_groups for p in g["params"]):
            raise ValueError("device_loss_scale: every parameter the optimizer steps on must be half precision")
        if len(optimizer.state) and not optimizer.capturable:
            raise ValueError("device_loss_scale: the optimizer already holds host-counted state; build it with capturable=True")
        optimizer.capturable = True              # step counts on the device: a gated (skipped) step does not count
        first = next(p for g in optimizer.param_groups for p in g["params"])
        scaler.to_device(first.device)
    stash.device_scaler = scaler if device_loss_scale else None
    _amp_state.loss_scalers = [scaler]
    _amp_state.opt_level = opt_level
    _patch_step(optimizer)
    return model, optimizer


def _lazy_init_maybe_master_weights(optimizer: torch.optim.Optimizer) -> None:
    """Create the fp32 masters and re-point the optimizer at them.  As in Apex this happens
    lazily, at the first ``scale_loss``: by then ``patch_optimizer`` has replaced the
    optimizer's parameters by the ones this process owns (ZeRO: their local segments)."""
    stash = optimizer._amp_stash
    if stash.lazy_init_called:
        return
    stash.lazy_init_called = True
    for group in optimizer.param_groups:
        new_params = []
        for p in group["params"]:
            if p.dtype in (torch.float16, torch.bfloat16):
                master = p.detach().clone().float()
                master.requires_grad_(p.requires_grad)
                stash.all_fp16_params.append(p)
                stash.all_fp32_from_fp16_params.append(master)
                if p in optimizer.state:
                    optimizer.state[master] = optimizer.state.pop(p)
                new_params.append(master)
            else:
                stash.all_fp32_from_fp32_params.append(p)
                new_params.append(p)
        group["params"] = new_params
    if getattr(optimizer, "writes_model_copies", False) and stash.all_fp16_params:
        # a fused optimizer writes model = half(master) from its step kernel
        optimizer.set_model_copies(stash.all_fp32_from_fp16_params, [p.detach() for p in stash.all_fp16_params])
        stash.optimizer_copies_back = True


def master_params(optimizer: torch.optim.Optimizer) -> Iterator[torch.Tensor]:
    """``apex.amp.master_params``: every parameter the optimizer steps on.  Callers use it to get at the
    master gradients (``clip_grad_norm_(amp.master_params(optimizer), ...)``), so a deferred write of
    those gradients is completed first."""
    stash = getattr(optimizer, "_amp_stash", None)
    if stash is not None and stash.pending_finish:
        finish_unscale(optimizer)
    for group in optimizer.param_groups:
        for p in group["params"]:
            yield p


def finish_unscale(optimizer: torch.optim.Optimizer, max_norm: Optional[float] = None) -> None:
    """Fused mode: run the deferred write pass (clip to ``max_norm`` when > 0; by default to the
    value an earlier ``decide_clip`` recorded, else no clipping)."""
    stash = optimizer._amp_stash
    if stash.pending_finish:
        if max_norm is None:
            max_norm = stash.decided_max_norm or 0.0
        with torch.no_grad():
            stash.unscale_plan.step_finish(float(max_norm), stash.step_flags)
        stash.clip_decided = True
        stash.pending_finish = False
        stash.decided_max_norm = None
        stash.unscale_plan.drop_sources()
        stash.pending_model_grads = []
        stash.feed = None


def can_step_from_model_grads(optimizer: torch.optim.Optimizer) -> bool:
    """True while the unscaled gradients need not be written at all: the write pass is still
    pending, the optimizer is one whose step kernel can read the model gradients and the clip
    decision itself, and every parameter it steps on has a half-precision model gradient (fp32
    parameters are unscaled in place and would be missing from the norm)."""
    stash = optimizer._amp_stash
    return bool(stash.pending_finish and getattr(optimizer, "reads_grad_sources", False)
                and not any(p.grad is not None for p in stash.all_fp32_from_fp32_params))


def decide_clip(optimizer: torch.optim.Optimizer, max_norm: float) -> None:
    """Fused mode with a fused optimizer: take the clip decision on the device (no pass over the
    gradients); the optimizer's step kernel applies it while reading the model gradients."""
    stash = optimizer._amp_stash
    with torch.no_grad():
        stash.unscale_plan.step_decide(float(max_norm), stash.step_flags)
    stash.clip_decided = True
    stash.decided_max_norm = float(max_norm)


def clip_from_unscale_sums(optimizer: torch.optim.Optimizer, max_norm: float) -> bool:
    """Fused mode after an eager unscale: the norm of the master gradients is already on the device, so clipping
    is the decision plus - only if it says "clip" - one in-place multiply.  Returns False when those sums do not
    cover every gradient ``clip_grad_norm`` is about (fp32 parameters with gradients, accumulation)."""
    stash = optimizer._amp_stash
    if not stash.sums_cover_all or any(p.grad is not None for p in stash.all_fp32_from_fp32_params):
        return False
    with torch.no_grad():
        stash.unscale_plan.step_apply_clip(float(max_norm), stash.step_flags)
    stash.sums_cover_all = False
    stash.clip_decided = True
    return True


def _master_to_model(optimizer: torch.optim.Optimizer) -> None:
    """Apex's post-step copy (``multi_tensor_scale`` with scale 1): ``model = half(master)``,
    round to nearest even, one launch for all pairs."""
    stash = optimizer._amp_stash
    if not stash.all_fp16_params:
        return
    if stash.copy_back_plan is None:
        stash.copy_back_plan = TensorPlan([m.detach() for m in stash.all_fp32_from_fp16_params],
                                          [p.detach() for p in stash.all_fp16_params])
    with torch.no_grad():
        stash.copy_back_plan.scale_cast(1.0)


def _device_scaled_step(optimizer, stash: _AmpStash, old_step, args, kwargs):
    """``optimizer.step`` with the loss-scale schedule on the device: the step kernel reads ``1 / scale`` and the clip
    decision where they are and does nothing after an overflow; then one thread updates the schedule."""
    scaler = stash.device_scaler
    if not stash.pending_finish and stash.unscale_plan is None:
        return old_step(*args, **kwargs)                 # no scale_loss has run: a plain step
    result_ptr = stash.unscale_plan.plan.result_device_ptr()
    if can_step_from_model_grads(optimizer) and not (args or kwargs) and stash.pending_inv_scale is None:
        if stash.decided_max_norm is None:
            decide_clip(optimizer, 0.0)
        if stash.feed is not None:
            optimizer.set_grad_feed(stash.feed, stash.pending_masters)
        else:
            optimizer.set_grad_sources(stash.pending_masters, stash.pending_model_grads)
        optimizer.grad_scale_ptr, optimizer.gate = scaler.inv_scale_ptr, result_ptr
        try:
            ret = old_step()
        finally:
            optimizer.set_grad_sources([], [])
            optimizer.grad_scale_ptr, optimizer.gate = 0, 0
    else:
        # the master gradients were looked at (or built up over several backward passes): they are in memory,
        # unscaled; whether the step runs is then read from the device, as the host-side schedule would
        finish_unscale(optimizer)
        skipped = bool(stash.unscale_plan.result().skipped) or bool(scaler._has_overflow)
        ret = None if skipped else old_step(*args, **kwargs)
        scaler._has_overflow = False
    scaler.update_on_device(result_ptr)
    stash.pending_finish = False
    stash.decided_max_norm = None
    stash.unscale_plan.drop_sources()
    stash.pending_model_grads = []
    stash.feed = None
    return ret


def _patch_step(optimizer: torch.optim.Optimizer) -> None:
    stash = optimizer._amp_stash
    if stash.already_patched:
        return
    old_step = optimizer.step

    def new_step(*args, **kwargs):
        if stash.device_scaler is not None:
            return _device_scaled_step(optimizer, stash, old_step, args, kwargs)
        if getattr(stash, "skip_next_step", False):
            stash.skip_next_step = False
            stash.pending_finish = False
            if stash.unscale_plan is not None:
                stash.unscale_plan.drop_sources()
            stash.pending_model_grads = []
            stash.feed = None
            return None
        if can_step_from_model_grads(optimizer) and not (args or kwargs):
            # unscale, clip, update and model copy in one kernel: the step reads the still-scaled
            # model gradients and the clip decision from the device
            if stash.decided_max_norm is None:
                decide_clip(optimizer, 0.0)
            if stash.feed is not None:
                optimizer.set_grad_feed(stash.feed, stash.pending_masters)      # read where the compiled table reads
            else:
                optimizer.set_grad_sources(stash.pending_masters, stash.pending_model_grads)
            optimizer.grad_scale = stash.pending_inv_scale
            optimizer.gate = stash.unscale_plan.plan.result_device_ptr()
            try:
                ret = old_step()
            finally:
                optimizer.set_grad_sources([], [])
                optimizer.grad_scale, optimizer.gate = 1.0, 0
            stash.pending_finish = False
            stash.decided_max_norm = None
            stash.unscale_plan.drop_sources()
            stash.pending_model_grads = []
            stash.feed = None
            return ret
        finish_unscale(optimizer)
        ret = old_step(*args, **kwargs)
        if not getattr(stash, "optimizer_copies_back", False):
            _master_to_model(optimizer)
        return ret

    optimizer.step = new_step
    stash.already_patched = True


@contextlib.contextmanager
def scale_loss(loss: torch.Tensor, optimizer: torch.optim.Optimizer):
    """``with amp.scale_loss(loss, optimizer) as scaled_loss: scaled_loss.backward()``.
    On exit: unscale the model gradients into the master gradients (fused kernel), update the
    loss scale, and arm a one-shot skip of ``optimizer.step`` after an overflow."""
    scaler = _amp_state.loss_scalers[0]
    stash = optimizer._amp_stash
    _lazy_init_maybe_master_weights(optimizer)
    # Gradients that fp32 parameters already hold are unscaled: set them aside so that the
    # backward pass does not add scaled values onto them (Apex stashes them the same way).
    stashed_fp32 = {}
    for p in stash.all_fp32_from_fp32_params:
        if p.grad is not None:
            stashed_fp32[id(p)] = p.grad
            p.grad = None
    try:
        yield loss.float() * (scaler.scale_on_device if scaler.on_device else scaler.loss_scale())
    except BaseException:
        # the body failed: put the stashed gradients back (dropping a half-made scaled one) and let the error through
        for p in stash.all_fp32_from_fp32_params:
            if id(p) in stashed_fp32:
                p.grad = stashed_fp32[id(p)]
        raise
    model_grads, master_grads = [], []
    if stash.master_grad_bucket is None and stash.all_fp32_from_fp16_params:
        masters = stash.all_fp32_from_fp16_params
        offs, lens = _lib.bucket_layout([m.numel() for m in masters], [_lib.RG_F32] * len(masters))
        stash.master_grad_bucket = torch.empty(lens[_lib.RG_F32], dtype=torch.float32, device=masters[0].device)
        stash.master_grad_views = [stash.master_grad_bucket.narrow(0, o, m.numel()).view(m.shape)
                                   for o, m in zip(offs, masters)]
    half_params, masters_all = stash.all_fp16_params, stash.all_fp32_from_fp16_params
    scaler.clear_overflow_state()
    dropped_half_grads = False
    if _native is not None and half_params and _compiled_steady_exit(stash, scaler):
        dropped_half_grads = True
        model_grads_all, n_with_grad, n_live = [], -1, 0
    else:
        model_grads_all = [p.grad for p in half_params]
        n_with_grad = sum(1 for g in model_grads_all if g is not None)
        n_live = sum(1 for m in masters_all if m.grad is not None)
    if dropped_half_grads:
        pass
    elif n_with_grad == len(half_params) and n_live == 0 and half_params:
        # The steady state of a training loop: every half parameter has a fresh gradient and no master gradient
        # is alive (zero_grad dropped them).  Nothing is classified or sorted; the table keeps its shape.
        views = stash.master_grad_views
        for m, v in zip(masters_all, views):
            m.grad = v
        stash.pending_masters, stash.pending_model_grads = masters_all, model_grads_all
        scaler.unscale(stash, model_grads_all, views, accumulate=False, all_params=True)
    else:
        fresh, live = [], []
        for i, (g, m) in enumerate(zip(model_grads_all, masters_all)):
            if g is None:
                continue
            (fresh if m.grad is None else live).append(i)
        accumulate = bool(live)
        if accumulate:
            finish_unscale(optimizer)                 # a deferred write must land before it is added to
            from ..multi_tensor import fill_zero_
            for i in fresh:                           # mixed case: start the missing ones from zero
                m = masters_all[i]
                m.grad = stash.master_grad_views[i]
                fill_zero_(m.grad.view(-1)) if m.grad.is_contiguous() else m.grad.zero_()
        masters = []
        for i in sorted(fresh + live):
            m = masters_all[i]
            if m.grad is None:
                m.grad = stash.master_grad_views[i]
            model_grads.append(model_grads_all[i])
            master_grads.append(m.grad)
            masters.append(m)
        stash.pending_masters, stash.pending_model_grads = masters, list(model_grads)
        if model_grads:
            scaler.unscale(stash, model_grads, master_grads, accumulate=accumulate,
                           covers_all=len(model_grads) == len(half_params))
    # fp32 parameters keep their own .grad; it carries the loss scale too
    from ..param_storage import _PlanCache
    if stash.fp32_unscale_plans is None:
        stash.fp32_unscale_plans, stash.fp32_accumulate_plans = _PlanCache(), _PlanCache()
    fresh32, new32, old32 = [], [], []
    for p in stash.all_fp32_from_fp32_params:
        kept = stashed_fp32.get(id(p))
        if p.grad is None:
            p.grad = kept                          # nothing new: the stashed gradient stays
        elif kept is None:
            fresh32.append(p.grad)
        else:
            new32.append(p.grad)
            old32.append(kept)
            p.grad = kept                          # kept += new * inv below
    with torch.no_grad():
        if fresh32 or new32:
            inv = 1.0 / scaler.loss_scale()
        if fresh32:
            plan = stash.fp32_unscale_plans.get(fresh32, fresh32)
            plan.unscale_pack(inv)
            if scaler.dynamic and plan.result().overflow:       # a static scale never skips: nothing waits for the flag
                scaler._has_overflow = True
        if new32:
            plan = stash.fp32_accumulate_plans.get(new32, old32)
            plan.unscale_accumulate(inv)
            if scaler.dynamic and plan.result().overflow:       # a static scale never skips: nothing waits for the flag
                scaler._has_overflow = True
    if not scaler.on_device:                # on the device the schedule is updated after optimizer.step
        should_skip = scaler.update_scale()
        if should_skip:
            stash.skip_next_step = True
    if not dropped_half_grads:
        for p in stash.all_fp16_params:       # Apex O2 drops the half grads once they are unscaled
            p.grad = None


def _compiled_steady_exit(stash: _AmpStash, scaler: LossScaler) -> bool:
    """The steady state of a training loop - every half parameter has a fresh, contiguous gradient of its own dtype
    and no master gradient is alive - handled without a Python loop over the parameters: the compiled module
    counts the gradients, hangs the bucket views on the masters, re-points its table at the new gradients,
    and drops the half gradients once the kernels that read them are queued.  Returns False, having changed
    nothing, when the step is not of that kind (the general path then runs)."""
    lists = stash.compiled
    if lists is None:
        if any(p.dtype != stash.all_fp16_params[0].dtype for p in stash.all_fp16_params):
            return False
        lists = stash.compiled = _CompiledLists(stash)
    if lists.grad_plan.bind_steady(lists.masters, lists.dtype) != lists.n:
        return False
    if lists.grad_plan.rebuilt():
        lists.grad_plan.tune()               # the views hold nothing yet: measure the write order on them
    stash.pending_masters, stash.pending_model_grads = stash.all_fp32_from_fp16_params, None
    stash.feed = lists.grad_plan
    scaler.unscale(stash, None, None, accumulate=False, plan=lists.plan)
    lists.half.clear_grads()                 # Apex O2 drops the half grads once they are unscaled
    return True


# --------------------------------------------------------------------------- reference API

def zip_params(optimizer):
    """(fp32 master, half model parameter) pairs in stash order (``pyrannc/amp/__init__.py:9-11``); creates the
    masters first if no ``scale_loss`` has run yet."""
    stash = optimizer._amp_stash
    pairs = _master_model_pairs(optimizer)
    if stash.pending_finish:
        finish_unscale(optimizer)         # callers read master.grad through these pairs
    return pairs


def _master_model_pairs(optimizer):
    """The pairs themselves, for code that only wants to know which master belongs to which parameter."""
    _lazy_init_maybe_master_weights(optimizer)
    stash = optimizer._amp_stash
    return zip(stash.all_fp32_from_fp16_params, stash.all_fp16_params)


def register_amp_params(optimizer):
    """Tell the registry which fp32 master belongs to which model parameter (``pyrannc/amp/__init__.py:13-18``).
    Under ZeRO the optimizer holds local segments; they are registered under the id of the parameter they are
    a segment of."""
    segment_owner = getattr(optimizer, "param_zero_segment_to_id", {})
    for master, model_param in _master_model_pairs(optimizer):
        owner = segment_owner[model_param] if model_param in segment_owner else id(model_param)
        _pyrannc.register_amp_master_param(owner, master)


def named_master_params(model, optimizer, zero=False):
    """``(name, tensor the optimizer steps on)`` for every parameter (``pyrannc/amp/__init__.py:21-41``): the
    fp32 master of a half parameter, the parameter itself when it already is fp32.  With ``zero`` the tensors
    are local segments and the names come from the module's ``name_to_pid``; otherwise the order is that of
    ``model.named_parameters()``.  The reference's tests read the unscaled gradients through it
    (``p.grad for n, p in named_master_params(...)``, ``test/common.py:86``), so a deferred write of the master
    gradients is completed first (inside ``zip_params``)."""
    if not hasattr(optimizer._amp_stash, "all_fp32_from_fp16_params"):
        return
    stepped_for = {model_param: master for master, model_param in zip_params(optimizer)}
    if zero:
        name_of = {pid: name for name, pid in model.name_to_pid.items()}
        for segment in optimizer.param_zero_segment_to_id:
            if segment.dtype == torch.float:
                stepped_for[segment] = segment
        for model_param, master in stepped_for.items():
            yield name_of[optimizer.param_zero_segment_to_id[model_param]], master
    else:
        for p in model.parameters():
            if p.dtype == torch.float:
                stepped_for[p] = p
        for name, p in model.named_parameters():
            yield name, stepped_for[p]


def patch_amp_scaler():
    """Make the loss scaler's ``update_scale`` a collective decision (``pyrannc/amp/__init__.py:44-65``): the
    scaler's own update runs first; the overflow flag is summed over all ranks as an int32 on the device; if
    any rank overflowed, every rank adopts the smallest ``int(loss_scale)``, restarts its count of clean steps
    and reports that the step must be skipped."""
    scaler = _amp_state.loss_scalers[0]
    if getattr(scaler, "_rannc_patched", False):
        return
    if scaler.on_device:
        # one rank: the sum of the flags is the flag and the minimum of int(loss_scale) is int(loss_scale) - the
        # update kernel truncates the halved scale itself and zeroes its count of clean steps
        scaler.update_flags |= _lib.RG_SCALER_TRUNCATE
        scaler._rannc_patched = True
        return
    own_update = scaler.update_scale

    def update_scale_on_all_ranks():
        overflowed_here = own_update()
        if _pyrannc.get_world_size() == 1:
            # one rank: the sum of the flags is the flag and the minimum of int(loss_scale) is int(loss_scale);
            # the reference's two device round trips per step (a .cuda() and an .item()) have nothing to exchange
            if overflowed_here:
                scaler._loss_scale = int(scaler._loss_scale)
                scaler._unskipped = 0
            return overflowed_here
        flag = torch.tensor([1 if overflowed_here else 0], dtype=torch.int32).cuda()
        _allreduce_sum(flag)
        if flag.item() == 0:
            return False
        smallest = torch.tensor([int(scaler._loss_scale)], dtype=torch.int32).cuda()
        _allreduce_min(smallest)
        scaler._loss_scale = smallest.item()
        scaler._unskipped = 0
        return True

    scaler.update_scale = update_scale_on_all_ranks
    scaler._rannc_patched = True


def unset_master_grads(optimizer):
    """``pyrannc/amp/__init__.py:68-70``: drop every master gradient (a write that was still deferred with them)."""
    stash = getattr(optimizer, "_amp_stash", None)
    if stash is not None and stash.pending_finish:
        stash.pending_finish = False
        stash.decided_max_norm = None
        stash.unscale_plan.drop_sources()
        stash.pending_model_grads = []
        stash.feed = None
    for group in optimizer.param_groups:
        for p in group["params"]:
            p.grad = None
