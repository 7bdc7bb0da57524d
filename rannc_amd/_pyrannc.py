"""The entry points of the reference's extension module ``pyrannc._pyrannc``
(``src/main.cpp:30-522``) that the per-step parameter/gradient path uses, with the same
names, argument meaning and error behaviour, for one process on one GPU.

Everything that only exists to trace, partition or pipeline a model is absent.
Unknown ids raise ``ValueError`` (the reference's ``std::invalid_argument``); library
failures raise ``RuntimeError``.
"""
from __future__ import annotations

from typing import Optional, Dict, Tuple

import ctypes
import torch

from .dist_param_locator import DistributedParamLocator
from .param_storage import ParamStorage

try:        # the compiled module: the registry and the per-step loops over parameters in C++
    from . import _ranncgrad as _native
except ImportError:      # not built: the same operations driven from Python over the ctypes binding
    _native = None

_param_storage = ParamStorage()
_dist_param_locator = DistributedParamLocator()
_tracing_state = True


def get_param_storage() -> ParamStorage:
    return _param_storage


def get_dist_param_locator() -> DistributedParamLocator:
    return _dist_param_locator


# -- process state (src/main.cpp:55-59); one process, one GPU
def get_rank() -> int:
    return 0


def get_world_size() -> int:
    return 1


def barrier() -> None:
    return None


def clear() -> None:
    global _param_storage
    for gid in list(_param_storage.graph_params):
        _param_storage.undeploy(gid)
    _param_storage = ParamStorage()
    _dist_param_locator.clear()
    if _native is not None:
        _native.reset_param_storage()


def set_tracing_state(enable: bool) -> None:
    global _tracing_state
    _tracing_state = bool(enable)


# -- tensor collectives (src/main.cpp:78-136).  With one rank a sum or a min over ranks,
# -- a broadcast and an all-gather return their input.
def allreduce_tensor(tensor: torch.Tensor, sum: bool) -> None:   # noqa: A002 - the reference's name
    if not isinstance(tensor, torch.Tensor):
        raise ValueError("allreduce_tensor expects a tensor")


def bcast_tensor(tensor: torch.Tensor, root: int) -> torch.Tensor:
    if root != 0:
        raise ValueError(f"root {root} is not a rank of this world (size 1)")
    return tensor.cuda()


def all_gather(ten: torch.Tensor, buf: torch.Tensor) -> None:
    if buf.numel() != ten.numel():
        raise ValueError("all_gather: receive buffer must hold world_size * numel elements")
    from .multi_tensor import copy_cast_
    with torch.no_grad():
        copy_cast_(buf.view(-1), ten.contiguous().view(-1))


# -- amp masters (src/main.cpp:191-200)
def register_amp_master_param(model_param_id: int, param: torch.Tensor) -> None:
    _param_storage.register_amp_master_param(model_param_id, id(param), param)
    if _native is not None:
        _native.register_amp_master_param(model_param_id, param)


# -- distributed parameters (src/main.cpp:202-245)
def store_dist_param(param: torch.Tensor) -> torch.Tensor:
    return _dist_param_locator.store(id(param), param)


def load_dist_param(pid: int) -> torch.Tensor:
    return _dist_param_locator.load(pid)


def set_dist_param(pid: int, param: torch.Tensor) -> None:
    _dist_param_locator.set(pid, param)


def get_dist_param_segment(pid: int) -> torch.Tensor:
    return _dist_param_locator.get_segment(pid)


def set_dist_param_dtype(pid: int, dtype: torch.dtype) -> None:
    _dist_param_locator.set_scalar_type(pid, dtype)


def get_dist_param_range(pid: int) -> Tuple[int, int]:
    return _dist_param_locator.get_segment_range(pid)


def remove_dist_param(pid: int) -> None:
    _dist_param_locator.remove(pid)


def dist_param_registered(pid: int) -> bool:
    return _dist_param_locator.registered(pid)


def gather_tensor_zero(ten: torch.Tensor, pid: int) -> torch.Tensor:
    """``src/main.cpp`` ``gather_tensor_zero`` -> ``ParamStorage::gatherTensorZero``
    (``src/comp/ParamStorage.cpp:670-685``): the per-rank pieces of a tensor laid out like the ZeRO
    segments of parameter ``pid``, gathered and viewed in the parameter's shape."""
    if _native is not None:
        try:
            return _native.get_param_storage().gather_tensor_zero(ten, pid)
        except ValueError:
            pass                   # deployed through the Python registry (gradient buckets)
    return _param_storage.gather_tensor_zero(ten, pid)


def get_param_ranks(pid: int):
    if _native is None or not _native.get_param_storage().has_param(pid):
        _param_storage.get_param_tensor(pid)
    return {0}


class RaNNCModule:
    """The methods of the bound C++ ``RaNNCModule`` (``src/main.cpp:257-450``) that sit on the
    per-step path.  ``init`` only registers the parameters of the (whole, unpartitioned)
    model under one graph id; there is no tracing, profiling or partitioning.

    The work is done by the class of the same name in the compiled module (``rannc_amd._ranncgrad``: registry and
    loops over parameters in C++, as in the reference).  Two cases are driven from Python over the ctypes binding
    instead: ``consolidate_grads`` (the gradient buckets live in ``param_storage.GradConsolidation``) and a
    package whose compiled module has not been built."""

    _next_id = 0

    def __init__(self, use_amp_master_params: bool = False, allreduce_amp_master_params: bool = False,
                 enable_zero: bool = False, check_unused_values: bool = True, offload_params: bool = False):
        self._use_amp_master_params = bool(use_amp_master_params)
        self._allreduce_amp_master_params = bool(allreduce_amp_master_params)
        self._enable_zero = bool(enable_zero)
        self._ctor_args = (self._use_amp_master_params, self._allreduce_amp_master_params, self._enable_zero,
                           bool(check_unused_values), bool(offload_params))
        self.graph_id = f"graph_{RaNNCModule._next_id}"
        RaNNCModule._next_id += 1
        self._deployed = False
        self._n = None            # the compiled class, once ``init`` has chosen it

    def init(self, named_params: Dict[str, torch.Tensor], consolidate_grads: bool = False) -> Dict[str, int]:
        """Register ``name -> parameter`` and deploy them; returns ``name -> id``
        (``RaNNCModule::init`` returns the used-parameter ids, ``src/comp/RaNNCModule.cpp:160-501``)."""
        if _native is not None and not consolidate_grads:
            self._n = _native.RaNNCModule(*self._ctor_args)
            ids = self._n.init(dict(named_params), False)
            self._deployed = True
            return ids
        ids = {}
        for name, p in named_params.items():
            _param_storage.register_param(id(p), p)
            ids[name] = id(p)
        _param_storage.deploy(self.graph_id, ids, enable_zero=self._enable_zero, consolidate=consolidate_grads,
                              use_amp_master_params=self._use_amp_master_params,
                              allreduce_amp_master_params=self._allreduce_amp_master_params)
        self._deployed = True
        return ids

    def _check(self) -> None:
        if not self._deployed:
            raise RuntimeError("RaNNCModule is not initialised")

    def prepare_backward(self) -> None:
        self._check()
        if self._n is None:
            _param_storage.prepare_backward(self.graph_id)

    def allreduce_grads(self) -> None:
        self._check()
        if self._n is not None:
            return self._n.allreduce_grads()
        _param_storage.allreduce_param_grads(self.graph_id)

    def allreduce_grads_zero(self) -> None:
        self._check()
        if self._n is not None:
            return self._n.allreduce_grads_zero()
        self._staging = _param_storage.allreduce_param_grads_zero(self.graph_id)

    def clip_grad_norm(self, max_grad_norm: float) -> None:
        self._check()
        if self._n is not None:
            return self._n.clip_grad_norm(max_grad_norm)          # narrowed to a C float at the binding
        _param_storage.clip_grad_norm(self.graph_id, ctypes.c_float(float(max_grad_norm)).value,
                                      self._use_amp_master_params)

    def calc_grad_norm(self) -> float:
        self._check()
        if self._n is not None:
            return self._n.calc_grad_norm()
        return _param_storage.calc_grad_global_l2_norm(self.graph_id, self._use_amp_master_params)

    def zero_grad(self) -> None:
        self._check()
        if self._n is not None:
            return self._n.zero_grad()
        _param_storage.clear_param_grads(self.graph_id)

    def use_amp_master_params(self) -> bool:
        return self._use_amp_master_params

    def align_params(self) -> None:
        self._check()
        if self._n is not None:
            return self._n.align_params()
        _param_storage.align_buffer_zero(self.graph_id)

    def sync_param_zero(self, grad: bool) -> None:
        self._check()
        if self._n is not None:
            return self._n.sync_param_zero(grad)
        _param_storage.bcast_params_zero(self.graph_id, grad)

    def set_grad_to_local_param_segment(self) -> None:
        self._check()
        if self._n is not None:
            return self._n.set_grad_to_local_param_segment()
        _param_storage.set_grad_to_local_param_segment(self.graph_id)

    def get_local_param_range(self, param_id: int) -> Tuple[int, int]:
        self._check()
        if self._n is not None:
            return self._n.get_local_param_range(param_id)
        return _param_storage.get_local_param_range(self.graph_id, param_id)

    def get_local_param_segment(self, param_id: int) -> torch.Tensor:
        self._check()
        if self._n is not None:
            return self._n.get_local_param_segment(param_id)
        return _param_storage.get_local_param_segment(self.graph_id, param_id)

    def _owned_tensor(self, param_id: int, amp_master_param: bool) -> torch.Tensor:
        if amp_master_param and _param_storage.has_amp_master_param(param_id):
            return _param_storage.get_amp_master_param_tensor(param_id)
        return _param_storage.get_param_tensor(param_id)

    def _in_param_shape(self, ten: torch.Tensor, param_id: int) -> torch.Tensor:
        """Under ZeRO the tensor this process steps on is a flat local segment; the reference hands callers
        the gathered tensor in the parameter's shape (``ParamStorage::doGatherParam`` ->
        ``gatherTensorZero``, ``src/comp/ParamStorage.cpp:1201-1232, 670-685``)."""
        shape = _param_storage.get_param_tensor(param_id).shape
        if ten.shape != shape and ten.numel() == shape.numel():
            return ten.detach().view(shape)
        return ten

    def get_param(self, param_id: int, amp_master_param: bool) -> torch.Tensor:
        self._check()
        if self._n is not None:
            return self._n.get_param(param_id, amp_master_param)
        return self._in_param_shape(self._owned_tensor(param_id, amp_master_param), param_id)

    def get_param_grad(self, param_id: int, amp_master_param: bool) -> torch.Tensor:
        """``gatherParamGrad`` (``src/comp/ParamStorage.cpp:1197-1213``): the gradient of the tensor this
        process steps on, zeros when it has none, in the parameter's shape."""
        self._check()
        if self._n is not None:
            return self._n.get_param_grad(param_id, amp_master_param)
        owner = self._owned_tensor(param_id, amp_master_param)
        grad = owner.grad if owner.grad is not None else torch.zeros_like(owner)
        return self._in_param_shape(grad, param_id)

    def _sync(self, param_id: int, grad: bool) -> Optional[torch.Tensor]:
        """``ParamStorage::doSyncParam`` + ``bcastParam`` (``src/comp/ParamStorage.cpp:1079-1133``) at one rank: the
        root's copy of the parameter (or of its gradient, zeros when it has none) as a fresh tensor on the host;
        ``None`` for a parameter no rank holds (the reference returns an undefined tensor)."""
        self._check()
        if self._n is not None:
            return self._n.sync_param_grad(param_id) if grad else self._n.sync_param(param_id)
        if param_id not in _param_storage.params:
            return None
        param = _param_storage.get_param_tensor(param_id)
        if grad:
            src = param.grad if param.grad is not None else torch.zeros_like(param)
        else:
            src = param
        return src.detach().clone().cpu()

    def sync_param(self, param_id: int) -> Optional[torch.Tensor]:
        return self._sync(param_id, False)

    def sync_param_grad(self, param_id: int) -> Optional[torch.Tensor]:
        return self._sync(param_id, True)

    def undeploy(self) -> None:
        if self._deployed:
            if self._n is not None:
                self._n.undeploy()
                self._n = None
            else:
                _param_storage.undeploy(self.graph_id)
            self._deployed = False
