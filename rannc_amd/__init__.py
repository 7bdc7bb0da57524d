"""rannc_amd: the per-step parameter/gradient path of RaNNC on one MI355X.

``RaNNCModule`` keeps the constructor arguments and the hot-path methods of
``pyrannc.RaNNCModule`` (``pyrannc/__init__.py:206-593``): ``clip_grad_norm``,
``_calc_grad_norm``, ``zero_grad``, ``get_param``, the ZeRO segment accessors and the
optimizer patching.  The wrapped model runs as it is, on one GPU: tracing, profiling,
partitioning and pipelining are not part of this package.  All arithmetic on parameters and
gradients goes through ``libranncgrad`` (hand-written HIP for gfx950); there is no CPU or
PyTorch fallback for it.
"""
from __future__ import annotations

import ctypes
import logging

import torch

from . import _pyrannc
from .dist_param import (DistributeModelParams, get_dist_param_range, get_dist_param_segment,  # noqa: F401
                         load_dist_param, remove_dist_param, set_dist_param, set_dist_param_dtype,
                         store_dist_param)
from .opt import patch_optimizer

logger = logging.getLogger("rannc")


def get_rank() -> int:
    return _pyrannc.get_rank()


def get_world_size() -> int:
    return _pyrannc.get_world_size()


def barrier() -> None:
    _pyrannc.barrier()


def clear() -> None:
    _pyrannc.clear()


class RaNNCModule(_pyrannc.RaNNCModule):
    r"""
    Wraps a ``torch.nn.Module`` (``pyrannc/__init__.py:206-252``).

    :param model: Model to wrap.
    :param optimizer: Optimizer; it is patched so that it steps on the parameters this
        process owns (``patch_optimizer``).
    :param enable_apex_amp: Master parameters and gradients are fp32 (amp O2).
    :param allreduce_amp_master_params: Gradients are reduced in fp32.
    :param enable_zero: ZeRO-style sharding of master parameters / optimizer state
        (requires ``enable_apex_amp``).
    :param consolidate_grads: keep gradients in per-dtype flat buckets (the reference's
        ``consolidate_grads`` configuration item, ``src/Config.cpp:32,146``).
    """

    def __init__(self, model, optimizer=None, gather_inputs=True, enable_apex_amp=False,
                 allreduce_amp_master_params=False, enable_zero=False, check_unused_values=True,
                 offload_params=False, consolidate_grads=False):
        if enable_zero and not enable_apex_amp:                      # pyrannc/__init__.py:224-225
            raise ValueError("enable_zero requires enable_apex_amp")
        super().__init__(enable_apex_amp, allreduce_amp_master_params, enable_zero, check_unused_values,
                         offload_params)
        self.model = model
        self.optimizer = optimizer
        self.gather_inputs = gather_inputs
        self.enable_apex_amp = enable_apex_amp
        self.allreduce_amp_master_params = allreduce_amp_master_params
        self.enable_zero = enable_zero
        self.offload_params = offload_params
        self.consolidate_grads = consolidate_grads
        self.amp_master_param_registered = False
        self.ready = False
        self.used_param_ids = set()
        self.name_to_param = {}
        self.name_to_pid = {}
        self.device = torch.device("cuda", torch.cuda.current_device()) if torch.cuda.is_available() \
            else torch.device("cpu")

    # ------------------------------------------------------------------ deployment
    def _deploy(self) -> None:
        if self.device.type != "cuda":
            raise RuntimeError("rannc_amd needs a GPU: parameters and gradients are processed by HIP kernels only")
        named = dict(self.model.named_parameters())
        for n, p in named.items():
            if not p.is_cuda:
                raise ValueError(f"parameter {n} is on {p.device}; move the model to the GPU first")
        self.name_to_param = named
        ids = self.init(named, consolidate_grads=self.consolidate_grads)
        self.name_to_pid = ids
        self.used_param_ids = set(ids.values())
        if self.enable_zero:                                          # pyrannc/__init__.py:289-290
            self.align_params()
        if self.optimizer is not None:
            patch_optimizer(self, self.optimizer)
        self.ready = True

    def __call__(self, *args, **kwargs):
        if not self.ready:
            self._deploy()
        if self.enable_zero:
            self.sync_param_zero(False)                               # GraphLauncher.cpp:366-368
        self.prepare_backward()                                       # GraphLauncher.cpp:468
        out = self.model(*args, **kwargs)
        if torch.is_grad_enabled():
            self._hook_end_of_backward(out)
        return out

    def _hook_end_of_backward(self, out) -> None:
        """What the reference does when a backward pass through the module ends
        (``GraphLauncher::backward``, ``src/comp/GraphLauncher.cpp:484-486``, then
        ``RaNNCTensorBackward::apply``, ``src/comp/Backward.cpp:101-108``): point the gradients of
        the ZeRO segments at their slice of the parameters' gradients and run the gradient
        exchange (for one process: the staging pack and copy-back).  Hooked on the outputs and
        run once, after autograd has produced every gradient of the pass."""
        tensors = [t for t in (out if isinstance(out, (tuple, list)) else [out])
                   if isinstance(t, torch.Tensor) and t.requires_grad]
        if not tensors:
            return
        state = {"queued": False}

        def at_end():
            state["queued"] = False
            with torch.no_grad():
                if self.enable_zero:
                    self.set_grad_to_local_param_segment()
                    self.allreduce_grads_zero()
                else:
                    self.allreduce_grads()

        def on_grad(grad):
            if not state["queued"]:
                state["queued"] = True
                torch.autograd.Variable._execution_engine.queue_callback(at_end)
            return grad

        for t in tensors:
            t.register_hook(on_grad)

    # ------------------------------------------------------------------ the wrapped module's own interface
    def _only_used(self, items, from_global: bool, named: bool):
        """Entries of the wrapped module's parameter / buffer iterators that this process works on
        (``_param_gen`` / ``_named_param_gen``, ``pyrannc/__init__.py:575-583``); all of them with one rank."""
        for item in items:
            tensor = item[1] if named else item
            if from_global or id(tensor) in self.used_param_ids:
                yield item

    def parameters(self, *args, from_global=False, **kwargs):
        """Parameters this process holds once deployed (``pyrannc/__init__.py:343-349``)."""
        if not self.ready:
            return self.model.parameters(*args, **kwargs)
        return self._only_used(self.model.parameters(*args, **kwargs), from_global, named=False)

    def named_parameters(self, *args, from_global=False, **kwargs):
        if not self.ready:
            return self.model.named_parameters(*args, **kwargs)
        return self._only_used(self.model.named_parameters(*args, **kwargs), from_global, named=True)

    def buffers(self, *args, **kwargs):
        """Buffers of the wrapped module (``pyrannc/__init__.py:359-372``).  The reference filters them through the ids
        of the parameters in use, which no buffer carries, so a deployed module yields none; with one rank the module
        runs as it is and its buffers are simply its own."""
        return self.model.buffers(*args, **kwargs)

    def named_buffers(self, *args, **kwargs):
        return self.model.named_buffers(*args, **kwargs)

    def train(self, mode=True):
        """A deployed reference module cannot change mode (``pyrannc/__init__.py:323-335``: it only warns); here the
        wrapped module runs eagerly, so the mode is simply passed on.  Returns ``self`` like ``nn.Module.train``."""
        self.model.train(mode)
        return self

    def eval(self):
        return self.train(False)

    def enable_dropout(self, enable):
        """Switch dropout layers on or off without touching the rest of the module's mode
        (``pyrannc/__init__.py:510-521``; the reference flips the flag inside its traced graph)."""
        for m in self.model.modules():
            if isinstance(m, torch.nn.modules.dropout._DropoutNd):
                m.train(bool(enable))

    def to(self, *args, **kwargs):
        """Ignored with a warning, as in the reference (``pyrannc/__init__.py:312-317``): where the parameters live
        is the runtime's business.  Move the model before wrapping it."""
        logger.warning("to() was ignored. A RaNNC model cannot be moved across devices.")
        return self

    def cuda(self, *args, **kwargs):
        """Ignored with a warning (``pyrannc/__init__.py:319-324``)."""
        logger.warning("cuda() was ignored. A RaNNC model cannot be moved across devices.")
        return self

    def __getattr__(self, attr):
        """Anything this wrapper does not define is looked up on the wrapped module (``pyrannc/__init__.py:526-537``)."""
        model = self.__dict__.get("model")
        if model is None or not hasattr(model, attr):
            raise AttributeError(f"This model has no attribute '{attr}'")
        return getattr(model, attr)

    # ------------------------------------------------------------------ per-step API
    def _setup_amp_params(self):
        if not self.amp_master_param_registered:                      # pyrannc/__init__.py:374-379
            from .amp import patch_amp_scaler, register_amp_params
            register_amp_params(self.optimizer)
            patch_amp_scaler()
            self.amp_master_param_registered = True

    def clip_grad_norm(self, max_grad_norm):
        r"""
        Clips gradients by their global L2 norm (``pyrannc/__init__.py:381-394``): iff
        ``norm + 1e-6 > max_grad_norm`` every gradient is multiplied by
        ``max_grad_norm / (norm + 1e-6)``.  With amp in fused mode the pending unscale is
        completed and clipped in the same pass over the gradients; with a fused optimizer on
        top only the decision is taken here and the optimizer's step kernel applies it.
        """
        if not self.ready:
            self._deploy()
        if self.enable_apex_amp:
            self._setup_amp_params()
            stash = getattr(self.optimizer, "_amp_stash", None)
            max_f = ctypes.c_float(float(max_grad_norm)).value      # crosses the binding as a C float
            if stash is not None and stash.pending_finish:
                from .amp import can_step_from_model_grads, decide_clip, finish_unscale
                if can_step_from_model_grads(self.optimizer):
                    decide_clip(self.optimizer, max_f)      # the optimizer's step kernel applies it
                    return
                if not any(p.grad is not None for p in stash.all_fp32_from_fp32_params):
                    finish_unscale(self.optimizer, max_f)
                    return
                finish_unscale(self.optimizer)
            elif stash is not None:
                from .amp import clip_from_unscale_sums
                if clip_from_unscale_sums(self.optimizer, max_f):
                    return
        super().clip_grad_norm(max_grad_norm)

    def _calc_grad_norm(self):
        if not self.ready:
            self._deploy()
        if self.enable_apex_amp:
            self._setup_amp_params()
            stash = getattr(self.optimizer, "_amp_stash", None)
            if stash is not None and stash.pending_finish:
                from .amp import finish_unscale
                finish_unscale(self.optimizer)
        return super().calc_grad_norm()

    def zero_grad(self):
        r"""Sets zeros to gradients of model parameters (``pyrannc/__init__.py:453-457``)."""
        if not self.ready:
            self._deploy()
        super().zero_grad()

    def get_param(self, name, amp_master_param=False):
        if name not in self.name_to_pid:
            raise RuntimeError(f"Parameter not found: {name}")       # pyrannc/__init__.py:466-467
        return super().get_param(self.name_to_pid[name], amp_master_param)

    def get_param_grad(self, name, amp_master_param=False):
        stash = getattr(self.optimizer, "_amp_stash", None)
        if amp_master_param and stash is not None and stash.pending_finish:
            from .amp import finish_unscale
            finish_unscale(self.optimizer)        # the master gradients are about to be looked at: write them
        if name not in self.name_to_pid:
            raise RuntimeError(f"Parameter not found: {name}")       # pyrannc/__init__.py:480-481
        return super().get_param_grad(self.name_to_pid[name], amp_master_param)

    def _sync_orig_params(self, sync_all_ranks=False, sync_grad=False, name_pattern=None):
        """Write the values the runtime holds back into the user's module (``pyrannc/__init__.py:539-573``): under
        ZeRO the segments are gathered first; then every named parameter (those whose name contains
        ``name_pattern``, if given) is overwritten with the root rank's copy, and its gradient too on request."""
        if not self.ready:
            return
        if self.enable_zero:
            self.sync_param_zero(sync_grad)
        for name in sorted(self.name_to_param):
            if name_pattern is not None and name_pattern not in name:
                continue
            pid, param = self.name_to_pid[name], self.name_to_param[name]
            synced = self.sync_param(pid)
            if synced is not None:
                with torch.no_grad():
                    if getattr(param, "distributed", False) and param.size() != synced.size():
                        param.data = synced          # a placeholder left behind by the sharding: take the full tensor
                        if hasattr(self.optimizer, "invalidate_tables"):
                            self.optimizer.invalidate_tables()
                    else:
                        param.copy_(synced.view(param.size()))
            if sync_grad:
                synced_grad = self.sync_param_grad(pid)
                if synced_grad is not None:
                    with torch.no_grad():
                        if param.grad is None:
                            param.grad = torch.zeros_like(param)
                        param.grad.copy_(synced_grad.view(param.size()))
        _pyrannc.barrier()

    # ------------------------------------------------------------------ checkpoints
    def state_dict(self, *args, no_hook=False, amp_master_params=True, rank0_only=True, **kwargs):
        r"""
        ``state_dict`` of the wrapped model (``pyrannc/__init__.py:401-436``): once deployed, one
        entry per parameter name - parameters that share data appear under every one of their
        names - holding the fp32 amp master when ``amp_master_params`` and amp are on.  Like the
        reference it lists parameters only.  ``no_hook`` leaves out the model's state-dict hooks.
        """
        if not self.ready:
            return self.model.state_dict(*args, **kwargs)
        stashed = None
        if no_hook:
            stashed = {m: m._state_dict_hooks for m in self.model.modules()}
            for m in stashed:
                m._state_dict_hooks = type(m._state_dict_hooks)()
        shared = {}
        for n, p in self.model.named_parameters(remove_duplicate=False):
            shared.setdefault(id(p), []).append(n)
        new_state_dict = {}
        try:
            for n in self.model.state_dict(*args, **kwargs):
                if n in self.name_to_param:
                    param = self.get_param(n, amp_master_params and self.enable_apex_amp)
                    for alias in shared.get(id(self.name_to_param[n]), [n]):
                        new_state_dict[alias] = param
        finally:
            if stashed is not None:
                for m, hooks in stashed.items():
                    m._state_dict_hooks = hooks
        return new_state_dict

    def load_state_dict(self, *args, **kwargs):
        r"""
        Loads a ``state_dict`` into the wrapped model (``pyrannc/__init__.py:438-451``).  A deployed
        module is undeployed first, so the next forward pass registers the new values.
        """
        if self.ready:
            self.undeploy()
            self.ready = False
            self.amp_master_param_registered = False
        return self.model.load_state_dict(*args, **kwargs)

    @property
    def use_amp_master_params_flag(self):
        return self.use_amp_master_params()

    def __del__(self):
        try:
            self.undeploy()
        except Exception:
            pass
