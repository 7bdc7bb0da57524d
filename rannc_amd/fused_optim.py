"""Optimizers whose step is one launch of the HIP library over all parameters, with the
fp32 master -> fp16/bf16 model copy folded in.

The reference leaves the step to ``torch.optim`` (``optim.Adam`` at ``test/common.py:142,165``,
``optim.SGD`` at ``examples/tutorial.py:28``), patched by ``pyrannc/opt.py:205-312``; under amp
Apex then copies every master into its model parameter.  ``FusedAdam`` / ``FusedAdamW`` /
``FusedSGD`` keep ``torch.optim.Adam`` / ``AdamW`` / ``SGD``'s constructor arguments, parameter
groups and state layout (``step``, ``exp_avg``, ``exp_avg_sq``; ``momentum_buffer``), so state
dicts, ``patch_optimizer`` and the checkpoint slicing of ``pyrannc/opt.py:186-202`` work on
them unchanged.  There is no CPU path: parameters must live on the GPU.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from . import _lib
from .multi_tensor import dtype_code, stream_handle

try:        # the compiled module: lists of parameters walked in C++
    from . import _ranncgrad as _native
except ImportError:
    _native = None


_data_ptr = torch.Tensor.data_ptr
_is_contiguous = torch.Tensor.is_contiguous


def _own_step(impl):
    """``step`` as ``torch.optim.Optimizer`` would wrap it, minus the cost: torch puts every optimizer's ``step``
    inside a profiler range and two hook loops (about 10 us per call - a quarter of a whole training step's host
    time on a small model).  Here the registered step hooks are called exactly as torch calls them, the range is
    opened only while a profiler is recording, and gradient mode is switched off without building a context
    object.  The ``hooked`` mark tells ``Optimizer.__init__`` not to wrap the function again."""
    from itertools import chain
    from torch.optim import optimizer as _topt

    def step(self, *args, **kwargs):
        full = (self,) + args
        if _topt._global_optimizer_pre_hooks or self._optimizer_step_pre_hooks:
            for hook in chain(_topt._global_optimizer_pre_hooks.values(), self._optimizer_step_pre_hooks.values()):
                result = hook(self, full, kwargs)
                if result is not None:
                    if isinstance(result, tuple) and len(result) == 2:
                        full, kwargs = result
                    else:
                        raise RuntimeError(f"{hook} must return None or a tuple of (new_args, new_kwargs), but got {result}.")
        grad_was_on = torch.is_grad_enabled()
        if grad_was_on:
            torch._C._set_grad_enabled(False)
        try:
            if torch.autograd._profiler_enabled():
                with torch.autograd.profiler.record_function(f"Optimizer.step#{self.__class__.__name__}.step"):
                    out = impl(*full, **kwargs)
            else:
                out = impl(*full, **kwargs)
        finally:
            if grad_was_on:
                torch._C._set_grad_enabled(True)
        if _topt._global_optimizer_post_hooks or self._optimizer_step_post_hooks:
            for hook in chain(self._optimizer_step_post_hooks.values(), _topt._global_optimizer_post_hooks.values()):
                hook(self, full, kwargs)
        return out

    step.hooked = True
    step.__doc__ = impl.__doc__
    step.__wrapped__ = impl
    return step


class _Steady:
    """What a group's last full step established, for the steps after it: as long as the same parameters all
    have contiguous gradients of the same dtype, a step is one pointer comparison per gradient and one launch."""
    __slots__ = ("params_obj", "n", "param_ids", "table", "key", "grad_ptrs", "grad_dtype", "steps_buf", "steps_np", "count", "device",
                 "param_ptr_ends", "fed_by")


class _FusedBase(torch.optim.Optimizer):
    def __init__(self, params, defaults):
        super().__init__(params, defaults)
        self._steady: Dict[int, _Steady] = {}
        self._tables: Dict[Tuple, Tuple[_lib.OptimTable, Tuple, List]] = {}
        self._model_copies: Dict[int, torch.Tensor] = {}
        self._steps: Dict[int, Tuple[torch.Tensor, int]] = {}     # id(param) -> (its step tensor, value)
        #: device pointer of an ``rg_step_result`` (``TensorPlan.plan.result_device_ptr()``): the step
        #: multiplies the gradients by its clip coefficient and does nothing when it says "skipped".
        #: The host-side bookkeeping (step counts, the first-step flag of momentum buffers) advances
        #: regardless, so a caller that sets ``gate`` must itself skip ``step()`` whenever the device
        #: would (``amp`` does: a dynamic scaler skips on the host, a static one never gates).
        self.gate: int = 0
        #: every gradient is multiplied by this first
        self.grad_scale: float = 1.0
        #: device address of a float to multiply by instead (a loss scaler's ``1 / scale`` kept on the device,
        #: ``rg_scaler_state.inv_scale``), so that a step recorded in a HIP graph follows the scale; 0: off
        self.grad_scale_ptr: int = 0
        self._grad_sources: Dict[int, torch.Tensor] = {}
        self._feed = None                          # see set_grad_feed
        self._feed_params: List[torch.Tensor] = []
        self._feed_offsets: Optional[Dict[int, int]] = None
        self._native_lists: Dict[int, Tuple] = {}  # group index -> (its params list, its length, compiled TensorList)

    #: the step can read gradients from tensors other than ``param.grad`` (see ``set_grad_sources``)
    reads_grad_sources = True

    def set_grad_sources(self, params, grads) -> None:
        """For the next steps ``grads[i]`` (any supported dtype, e.g. the still-scaled fp16 model
        gradient) is read as the gradient of ``params[i]`` instead of ``params[i].grad``; together
        with ``grad_scale`` and ``gate`` this folds unscale and clip into the step.  Empty lists
        switch it off."""
        self._grad_sources = {id(p): g for p, g in zip(params, grads) if g is not None}
        self._feed, self._feed_params, self._feed_offsets = None, [], None

    def set_grad_feed(self, feed, params) -> None:
        """``set_grad_sources`` for gradients that a table of the compiled module (a ``GradPlan``) holds:
        ``params[i]`` reads the plan's i-th gradient.  A group whose parameters are a run of ``params`` and whose
        last step left a steady-state record gets the new addresses pushed into its table by the compiled module -
        no Python loop over the parameters; anything else falls back to the tensors themselves."""
        self._grad_sources = {}
        self._feed, self._feed_params = feed, params
        offsets: Optional[Dict[int, int]] = {}
        off = 0
        for gi, group in enumerate(self.param_groups):
            ps = group["params"]
            n = len(ps)
            if n == 0:
                continue
            if off + n > len(params) or ps[0] is not params[off] or ps[-1] is not params[off + n - 1]:
                offsets = None
                break
            offsets[gi] = off
            off += n
        self._feed_offsets = offsets

    def _sources_from_feed(self) -> None:
        """The fed gradients as tensors, for the paths that look at every parameter."""
        if self._feed is not None and not self._grad_sources:
            self._grad_sources = {id(p): g for p, g in zip(self._feed_params, self._feed.sources()) if g is not None}

    def load_state_dict(self, state_dict) -> None:
        super().load_state_dict(state_dict)
        self._steady.clear()          # the state tensors are new objects: the next step rebuilds tables and counters
        self._tables.clear()
        self._steps.clear()

    def invalidate_tables(self) -> None:
        """Forget what earlier steps established about where parameters, gradients, state and model copies live.
        For code that re-homes a parameter's ``.data`` (or a model copy) between steps: the next step then looks at
        every tensor again and pushes all addresses to the device."""
        self._steady.clear()
        self._tables.clear()

    def _steady_grads(self, gi: int, group) -> Optional[Tuple["_Steady", List[torch.Tensor]]]:
        """The group's steady-state record and this step's gradients, or None when anything about the group
        differs from the step that made the record (then the full path runs and makes a new one)."""
        st = self._steady.get(gi)
        params = group["params"]
        if st is None or st.params_obj is not params or len(params) != st.n:
            return None
        if self._feed is not None and not self._grad_sources:
            off = self._feed_offsets.get(gi) if self._feed_offsets is not None else None
            if (off is not None and self._feed.held() >= off + st.n and dtype_code(st.grad_dtype) == self._feed.source_dtype()
                    and (params[0].data_ptr(), params[-1].data_ptr()) == st.param_ptr_ends):
                if st.fed_by is not self._feed:
                    self._feed.forget_optim(st.table.handle)      # whatever an earlier table at this address was told
                    st.fed_by = self._feed
                if self._feed.push_sources_to_optim(st.table.handle, off, st.n) or st.grad_ptrs is not None:
                    # the table was re-pointed behind the back of the records kept here: they no longer say where it
                    # points, so that a later step through the general path pushes every address again
                    st.grad_ptrs = None
                    hit = self._tables.get(st.key)
                    if hit is not None and hit[0] is st.table:
                        self._tables[st.key] = (hit[0], None, hit[2])
                return st, None
            self._sources_from_feed()
        if self._grad_sources:
            grads = list(map(self._grad_sources.get, st.param_ids))
        else:
            grads = [p.grad for p in params]
        for g in grads:
            if g is None:
                return None
        dt = st.grad_dtype
        for g in grads:
            if g.dtype != dt:
                return None
        if not all(map(_is_contiguous, grads)):
            return None
        # a parameter whose storage was replaced (``p.data = ...``) since the record was made: first and last are
        # looked at here, code that re-homes others calls ``invalidate_tables``
        if (params[0].data_ptr(), params[-1].data_ptr()) != st.param_ptr_ends:
            return None
        ptrs = list(map(_data_ptr, grads))
        if ptrs != st.grad_ptrs:
            st.table.update_pointers(grads=ptrs, stream=stream_handle(st.device))
            st.grad_ptrs = ptrs
            st.fed_by = None      # a feed's record of what it last pushed into this table is stale from here on
            # the full path's record of what the table points at must not outlive this re-pointing: a later
            # full step with the old addresses would otherwise find them "unchanged" and skip the update
            hit = self._tables.get(st.key)
            if hit is not None and hit[0] is st.table and hit[1] is not None:
                self._tables[st.key] = (hit[0], (hit[1][0], tuple(ptrs)) + tuple(hit[1][2:]), hit[2])
        return st, grads

    def _make_steady(self, gi: int, group, table, grads: List[torch.Tensor], count: Optional[int]) -> None:
        params = group["params"]
        st = _Steady()
        st.params_obj, st.n = params, len(params)
        st.param_ids = [id(p) for p in params]
        st.table = table
        st.key = table.cache_key
        st.param_ptr_ends = (params[0].data_ptr(), params[-1].data_ptr())
        st.grad_ptrs = [g.data_ptr() for g in grads]
        st.fed_by = None
        st.grad_dtype = grads[0].dtype
        st.device = params[0].device
        st.count = count
        st.steps_buf = st.steps_np = None
        if count is not None:
            # every parameter's ``step`` becomes a view of one host vector: a step is one add, not one per parameter
            st.steps_buf = torch.full((len(params),), float(count), dtype=torch.float32)
            st.steps_np = st.steps_buf.numpy()          # same memory; numpy adds to a short vector in a tenth of the time
            for i, p in enumerate(params):
                self.state[p]["step"] = st.steps_buf[i]
                self._steps.pop(id(p), None)      # from here on the tensor itself is the count
        self._steady[gi] = st

    def zero_grad(self, set_to_none: bool = True) -> None:
        """``torch.optim.Optimizer.zero_grad`` without its per-parameter bookkeeping."""
        if not set_to_none:
            return super().zero_grad(set_to_none=False)
        for gi, group in enumerate(self.param_groups):
            params = group["params"]
            if _native is None:
                for p in params:
                    p.grad = None
                continue
            known = self._native_lists.get(gi)
            if known is None or known[0] is not params or known[1] != len(params):
                known = self._native_lists[gi] = (params, len(params), _native.TensorList(params))
            known[2].clear_grads()

    def _scale_source(self, table: _lib.OptimTable) -> _lib.OptimTable:
        """Tell the table where the gradient scale lives, when that changed since its last launch."""
        if getattr(table, "scale_source", 0) != self.grad_scale_ptr:
            table.set_grad_scale_source(self.grad_scale_ptr)
            table.scale_source = self.grad_scale_ptr
        return table

    def _grad_of(self, p: torch.Tensor) -> Optional[torch.Tensor]:
        if self._feed is not None:
            self._sources_from_feed()
        return self._grad_sources.get(id(p), p.grad) if self._grad_sources else p.grad

    # -- model copies (amp): written by the step kernel instead of a separate copy pass
    writes_model_copies = True

    def set_model_copies(self, masters, models) -> None:
        """``models[i]`` (fp16/bf16/fp32, same size) receives ``round(masters[i])`` at every step."""
        for m, c in zip(masters, models):
            if c.numel() != m.numel() or not c.is_contiguous() or c.device != m.device:
                raise ValueError("model copy must be a contiguous tensor of the master's size and device")
            dtype_code(c.dtype)
            self._model_copies[id(m)] = c
        self._tables.clear()
        self._steady.clear()

    def _check_param(self, p: torch.Tensor, g: torch.Tensor) -> None:
        if p.dtype != torch.float32:
            raise ValueError(f"fused optimizers step fp32 parameters (masters), got {p.dtype}")
        if not p.is_cuda or not p.is_contiguous():
            raise ValueError("fused optimizers need contiguous GPU parameters")
        if g.is_sparse:
            raise ValueError("sparse gradients are not supported")
        if not g.is_contiguous() or g.device != p.device or g.numel() != p.numel():
            raise ValueError("gradient must be contiguous, on the parameter's device and of its size")

    def _table(self, key: Tuple, params: List[torch.Tensor], grads: List[torch.Tensor],
               state1: Optional[List[torch.Tensor]], state2: Optional[List[torch.Tensor]]) -> _lib.OptimTable:
        """Table for this exact list of parameters and gradient dtypes, re-pointed when any address moved."""
        copies = [self._model_copies.get(id(p)) for p in params]
        key = key + (tuple(g.dtype for g in grads),)
        ptrs = (tuple(p.data_ptr() for p in params), tuple(g.data_ptr() for g in grads),
                tuple(s.data_ptr() for s in state1) if state1 is not None else None,
                tuple(s.data_ptr() for s in state2) if state2 is not None else None,
                tuple(c.data_ptr() if c is not None else 0 for c in copies))
        hit = self._tables.get(key)
        dev = params[0].device
        if hit is None:
            table = _lib.OptimTable(dev.index, ptrs[0], ptrs[1], ptrs[2], ptrs[3],
                                    ptrs[4] if any(ptrs[4]) else None, [p.numel() for p in params],
                                    [dtype_code(g.dtype) for g in grads],
                                    [dtype_code(c.dtype) if c is not None else _lib.RG_F32 for c in copies])
        else:
            table, old, _ = hit
            if old != ptrs:
                table.update_pointers(ptrs[0], ptrs[1], ptrs[2], ptrs[3], ptrs[4] if any(ptrs[4]) else None,
                                      stream_handle(dev))
        # the table borrows raw pointers: keep what it points at alive - except the gradients, which only have to
        # live until the launch that reads them is queued (their memory is reused in stream order) and whose
        # release lets the next backward find the same addresses free
        self._tables[key] = (table, ptrs, [params, state1, state2, copies])
        table.cache_key = key
        return table


class FusedAdam(_FusedBase):
    """``torch.optim.Adam`` (amsgrad off) as one launch per parameter group."""

    _decoupled = False

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0, maximize=False,
                 capturable=False):
        """``capturable``: as in ``torch.optim.Adam`` - the step count lives on the device (``state["step"]`` is a
        0-dim float32 GPU tensor), nothing about a step is decided on the host, and ``step()`` may be recorded in
        a HIP graph and replayed.  Every parameter of a group must then have a gradient at every step, at the same
        address (graph capture needs that anyway), and the first ``step()`` - which allocates the state - has to
        run outside a capture.

        What a capture freezes: ``lr``, ``betas``, ``eps``, ``weight_decay`` and ``maximize`` of every group, and
        ``grad_scale`` when it is passed by value, are kernel arguments and so become part of the recorded graph -
        changing ``param_groups[i]["lr"]`` afterwards affects eager steps only, a replayed graph keeps the values
        of the capture (record a new graph after a learning-rate change).  What a replay does follow, because it
        is read from device memory: the step count and its bias corrections, the gate (clip coefficient, skip)
        and, with ``grad_scale_ptr``, 1 / loss scale."""
        if lr < 0 or eps < 0 or not 0 <= betas[0] < 1 or not 0 <= betas[1] < 1 or weight_decay < 0:
            raise ValueError("invalid Adam hyper-parameters")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, maximize=maximize))
        self.capturable = bool(capturable)
        self._clocks: Dict[int, torch.Tensor] = {}       # group index -> its rg_adam_clock (8 float32 words on the device)

    def load_state_dict(self, state_dict) -> None:
        super().load_state_dict(state_dict)
        self._clocks.clear()          # re-seeded from the loaded ``step`` values by the next step

    def _capturable_step(self, gi: int, group) -> None:
        """One group's step with its count on the device: advance the clock (one thread), then the update kernel."""
        params = group["params"]
        if not params:
            return
        clock = self._clocks.get(gi)
        steady = self._steady_grads(gi, group) if clock is not None else None
        if steady is not None:
            # same parameters, all with usable gradients, as at the step that made the record: the table is in place
            # (re-pointed at the gradients by _steady_grads), only the two launches remain
            st, _ = steady
            b1, b2 = group["betas"]
            stream = stream_handle(st.device)
            _lib.adam_clock_advance(clock.data_ptr(), group["lr"], b1, b2, self.gate, st.device.index, stream)
            self._scale_source(st.table).adam_step_clocked(clock.data_ptr(), group["lr"], b1, b2, group["eps"],
                                                           group["weight_decay"], decoupled=self._decoupled,
                                                           maximize=group["maximize"], grad_scale=self.grad_scale,
                                                           gate=self.gate, stream=stream)
            return
        self._steady.pop(gi, None)
        grads = [self._grad_of(p) for p in params]
        if any(g is None for g in grads):
            raise RuntimeError("a capturable optimizer needs a gradient for every parameter at every step")
        dev = params[0].device
        if clock is None:
            counts = set()
            for p, g in zip(params, grads):
                self._check_param(p, g)
                st = self.state[p]
                if len(st) == 0:
                    st["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    counts.add(0)
                else:
                    counts.add(int(st["step"]))
            if len(counts) != 1:
                raise RuntimeError("a capturable optimizer keeps one step count per group; the loaded counts differ")
            clock = torch.zeros(_lib.ADAM_CLOCK_BYTES // 4, dtype=torch.float32, device=dev)
            count = counts.pop()
            if count:
                clock.view(torch.int64)[0] = count
                clock[4] = float(count)
            for p in params:
                self.state[p]["step"] = clock[4]          # every parameter's count is the group's, on the device
            self._clocks[gi] = clock
        ms = [self.state[p]["exp_avg"] for p in params]
        vs = [self.state[p]["exp_avg_sq"] for p in params]
        table = self._table((gi, "capturable"), params, grads, ms, vs)
        b1, b2 = group["betas"]
        stream = stream_handle(dev)
        _lib.adam_clock_advance(clock.data_ptr(), group["lr"], b1, b2, self.gate, dev.index, stream)
        self._scale_source(table).adam_step_clocked(clock.data_ptr(), group["lr"], b1, b2, group["eps"], group["weight_decay"],
                                decoupled=self._decoupled, maximize=group["maximize"], grad_scale=self.grad_scale,
                                gate=self.gate, stream=stream)
        self._make_steady(gi, group, table, grads, None)

    @_own_step
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        if self.capturable:
            for gi, group in enumerate(self.param_groups):
                self._capturable_step(gi, group)
            return loss
        for gi, group in enumerate(self.param_groups):
            steady = self._steady_grads(gi, group)
            if steady is not None:
                st, _ = steady
                st.count += 1
                st.steps_np += 1.0
                b1, b2 = group["betas"]
                self._scale_source(st.table).adam_step(group["lr"], b1, b2, group["eps"], group["weight_decay"], st.count,
                                   decoupled=self._decoupled, maximize=group["maximize"], grad_scale=self.grad_scale,
                                   gate=self.gate, stream=stream_handle(st.device))
                continue
            self._steady.pop(gi, None)
            by_step: Dict[int, List[torch.Tensor]] = {}
            step_tensors = []
            grad_of: Dict[int, torch.Tensor] = {}
            for p in group["params"]:
                g = self._grad_of(p)
                if g is None:
                    continue
                self._check_param(p, g)
                grad_of[id(p)] = g
                st = self.state[p]
                if len(st) == 0:
                    st["step"] = torch.tensor(0.0, dtype=torch.float32)
                    st["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                # ``step`` stays a tensor (torch.optim's state layout); its integer value is mirrored
                # here so that a step costs one batched increment instead of one tensor op per parameter
                t = st["step"]
                seen = self._steps.get(id(p))
                count = (seen[1] if seen is not None and seen[0] is t else int(t)) + 1
                self._steps[id(p)] = (t, count)
                step_tensors.append(t)
                by_step.setdefault(count, []).append(p)
            if step_tensors:
                torch._foreach_add_(step_tensors, 1)
            for step, ps in by_step.items():
                ms = [self.state[p]["exp_avg"] for p in ps]
                vs = [self.state[p]["exp_avg_sq"] for p in ps]
                table = self._table((gi, tuple(id(p) for p in ps)), ps, [grad_of[id(p)] for p in ps], ms, vs)
                b1, b2 = group["betas"]
                self._scale_source(table).adam_step(group["lr"], b1, b2, group["eps"], group["weight_decay"], step,
                                decoupled=self._decoupled, maximize=group["maximize"], grad_scale=self.grad_scale,
                                gate=self.gate, stream=stream_handle(ps[0].device))
                if len(by_step) == 1 and len(ps) == len(group["params"]):
                    self._make_steady(gi, group, table, [grad_of[id(p)] for p in ps], step)
        return loss


class FusedAdamW(FusedAdam):
    """``torch.optim.AdamW``: weight decay applied to the parameter, not the gradient."""

    _decoupled = True

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2, maximize=False,
                 capturable=False):
        super().__init__(params, lr, betas, eps, weight_decay, maximize, capturable)


class FusedSGD(_FusedBase):
    """``torch.optim.SGD`` as one launch per parameter group (two on the step that creates
    momentum buffers for only some of the parameters)."""

    def __init__(self, params, lr=1e-3, momentum=0.0, dampening=0.0, weight_decay=0.0, nesterov=False, maximize=False):
        if lr < 0 or momentum < 0 or weight_decay < 0:
            raise ValueError("invalid SGD hyper-parameters")
        if nesterov and (momentum <= 0 or dampening != 0):
            raise ValueError("Nesterov momentum requires a momentum and zero dampening")
        super().__init__(params, dict(lr=lr, momentum=momentum, dampening=dampening, weight_decay=weight_decay,
                                      nesterov=nesterov, maximize=maximize))

    @_own_step
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for gi, group in enumerate(self.param_groups):
            steady = self._steady_grads(gi, group)
            if steady is not None:
                st, _ = steady
                self._scale_source(st.table).sgd_step(group["lr"], group["momentum"], group["dampening"], group["weight_decay"],
                                  group["nesterov"], group["maximize"], first_step=False, grad_scale=self.grad_scale,
                                  gate=self.gate, stream=stream_handle(st.device))
                continue
            self._steady.pop(gi, None)
            fresh, seasoned = [], []
            grad_of: Dict[int, torch.Tensor] = {}
            for p in group["params"]:
                g = self._grad_of(p)
                if g is None:
                    continue
                self._check_param(p, g)
                grad_of[id(p)] = g
                st = self.state[p]
                if group["momentum"] != 0 and st.get("momentum_buffer") is None:
                    # zeros, not empty: if the first launch is gated off on the device the buffer must
                    # not reach the next step with whatever the memory held
                    st["momentum_buffer"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    fresh.append(p)
                else:
                    seasoned.append(p)
            for first, ps in ((True, fresh), (False, seasoned)):
                if not ps:
                    continue
                bufs = [self.state[p]["momentum_buffer"] for p in ps] if group["momentum"] != 0 else None
                table = self._table((gi, first, tuple(id(p) for p in ps)), ps, [grad_of[id(p)] for p in ps], bufs, None)
                self._scale_source(table).sgd_step(group["lr"], group["momentum"], group["dampening"], group["weight_decay"],
                               group["nesterov"], group["maximize"], first_step=first, grad_scale=self.grad_scale,
                               gate=self.gate, stream=stream_handle(ps[0].device))
                if not first and not fresh and len(ps) == len(group["params"]):
                    self._make_steady(gi, group, table, [grad_of[id(p)] for p in ps], None)
        return loss
