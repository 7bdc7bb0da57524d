"""Parameter / gradient registry of one process: the host-side logic of the reference's
``ParamStorage``, ``GradConsolidation`` and ``DistributedGradLocator``
(``src/comp/ParamStorage.cpp``, ``src/comp/DistributedGradLocator.cpp``).

The reference issues one ATen op per tensor from C++ loops; here every loop over parameters
is one launch of the HIP library over a device-side table (``multi_tensor.TensorPlan``).
PyTorch supplies the memory; buckets and aligned buffers are torch tensors owned by this
registry, and parameters' ``.grad`` / ``.data`` are re-pointed at views of them exactly as
the reference does.

World size is 1 in this build: the collectives the reference interleaves with this work
(all-reduce of buckets, reduce-scatter, all-gather) are identities, and the rank-set / tag
bookkeeping that only exists to drive them is not reproduced.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import _lib
from .multi_tensor import TensorPlan, dtype_code, fill_zero_

try:        # the compiled module: per-step loops over parameters in C++
    from . import _ranncgrad as _native
except ImportError:
    _native = None

_DTYPE_ORDER = (torch.float32, torch.float16, torch.bfloat16)


def _zeros(n: int, dtype: torch.dtype, device: torch.device) -> torch.Tensor:
    """``torch::zeros`` of the reference (``src/comp/ParamStorage.cpp:59-75``,
    ``src/torch/TorchUtil.cpp:1463-1477``): memory from PyTorch, cleared by the fill kernel."""
    return fill_zero_(torch.empty(n, dtype=dtype, device=device))


class BufferTensorCache:
    """Buffers that live across steps, keyed by a caller-chosen name and re-made only when the requested type
    changes (``BufferTensorCache``, ``src/torch/TorchUtil.cpp:1434-1461``).  Besides saving the allocations it
    keeps the buffers' addresses fixed, so the device tables that point at them are built once."""

    def __init__(self) -> None:
        self._bufs: Dict[str, torch.Tensor] = {}

    def get(self, key: str, numel: int, dtype: torch.dtype, device: torch.device) -> torch.Tensor:
        buf = self._bufs.get(key)
        if buf is None or buf.numel() != numel or buf.dtype != dtype or buf.device != device:
            buf = self._bufs[key] = torch.empty(numel, dtype=dtype, device=device)
        return buf

    def clear(self, prefix: str = "") -> None:
        for key in [k for k in self._bufs if k.startswith(prefix)]:
            del self._bufs[key]


class _PlanCache:
    """Reuses a device table while the tensors it describes stay where they are."""

    def __init__(self) -> None:
        self._key: Optional[tuple] = None
        self._plan: Optional[TensorPlan] = None
        self._token = None
        self._src_ptrs: Optional[List[int]] = None
        self._orders: Dict[tuple, int] = {}       # layout (sizes and dtypes) -> write order measured for it

    def get_same_shapes(self, token, srcs: Sequence[torch.Tensor], dsts: Sequence[torch.Tensor],
                        tune_new: bool = False) -> TensorPlan:
        """``get`` for a caller that vouches, by passing the same ``token`` as last time, that the list has the
        sizes, dtypes and destinations it had then (the same parameters, all with gradients): only the source
        addresses are looked at - one ``data_ptr`` per tensor instead of a signature per pair."""
        if self._plan is None or token is None or token != self._token or not all(map(torch.Tensor.is_contiguous, srcs)):
            plan = self.get(srcs, dsts, tune_new)
            self._token = token
            self._src_ptrs = list(map(torch.Tensor.data_ptr, srcs))
            return plan
        ptrs = list(map(torch.Tensor.data_ptr, srcs))
        if ptrs != self._src_ptrs:
            self._plan.repoint_sources(ptrs)
            self._src_ptrs = ptrs
            self._key = None                  # the general signature no longer describes the table
        self._plan._srcs = list(srcs)
        return self._plan

    def get(self, srcs: Sequence[Optional[torch.Tensor]], dsts: Optional[Sequence[Optional[torch.Tensor]]],
            tune_new: bool = False) -> TensorPlan:
        """``tune_new``: a table that has to be built is also tuned (``TensorPlan.tune``: the destinations are
        overwritten, so only for callers whose destinations hold nothing they still need)."""
        def sig(ts):
            if ts is None:
                return None
            return tuple((0 if t is None else t.data_ptr(), 0 if t is None else t.numel(),
                          None if t is None else t.dtype) for t in ts)
        key = (sig(srcs), sig(dsts))
        self._token = None
        if self._plan is not None and key == self._key:
            return self._plan
        if self._plan is not None:
            # same shapes and dtypes, new addresses: refresh the table in place
            same_shape = self._key is not None and len(self._key[0]) == len(key[0]) and all(
                a[1:] == b[1:] and (a[0] == 0) == (b[0] == 0) for a, b in zip(self._key[0], key[0])) and (
                (self._key[1] is None) == (key[1] is None)) and (key[1] is None or all(
                    a[1:] == b[1:] and (a[0] == 0) == (b[0] == 0) for a, b in zip(self._key[1], key[1])))
            if same_shape:
                self._plan.update(srcs, dsts)
                self._key = key
                return self._plan
            self._plan.close()
        self._plan = TensorPlan(srcs, dsts)
        if tune_new and dsts is not None:
            # measured once per layout: a table rebuilt for the same sizes and dtypes takes the order found then,
            # so that its destinations are not overwritten by another measurement
            layout = (tuple(k[1:] for k in key[0]), tuple(k[1:] for k in key[1]))
            if layout in self._orders:
                self._plan.set_write_order(self._orders[layout])
            else:
                self._orders[layout] = self._plan.tune()
        self._key = key
        return self._plan

    def clear(self) -> None:
        if self._plan is not None:
            self._plan.close()
        self._plan, self._key, self._token, self._src_ptrs = None, None, None, None


class GradConsolidation:
    """Per-dtype flat gradient buckets with every parameter's ``.grad`` a view into them
    (``GradConsolidation``, ``src/comp/ParamStorage.cpp:33-191``)."""

    def __init__(self, storage: "ParamStorage", param_ids: Sequence[int], use_amp_master_params: bool,
                 consolidate_master_params: bool):
        assert len(param_ids) > 0                                          # ParamStorage.cpp:86
        self.storage = storage
        self.param_ids = list(param_ids)          # not sorted: they are local (ParamStorage.cpp:47)
        self.use_amp_master_params = use_amp_master_params
        self.consolidate_master_params = consolidate_master_params
        params = [storage.get_param_tensor(pid) for pid in self.param_ids]
        device = params[0].device
        codes = [dtype_code(p.dtype) for p in params]                      # ValueError on other dtypes (:51-53)
        offsets, lengths = _lib.bucket_layout([p.numel() for p in params], codes)   # :48-57
        self.offsets = dict(zip(self.param_ids, offsets))
        self.consolidated_grads: Dict[torch.dtype, torch.Tensor] = {}
        self.consolidated_master_grads: Dict[torch.dtype, torch.Tensor] = {}
        present = {p.dtype for p in params}
        for dt in _DTYPE_ORDER:
            if dt not in present:
                continue
            n = lengths[dtype_code(dt)]
            if consolidate_master_params and dt == torch.float16:         # :68-70
                self.consolidated_master_grads[dt] = _zeros(n, torch.float32, device)
            else:
                self.consolidated_grads[dt] = _zeros(n, dt, device)
        self.consolidated_amp_fp32_next: Optional[torch.Tensor] = None
        self._double_fp32 = use_amp_master_params and torch.float32 in self.consolidated_grads   # :77-84
        if self._double_fp32:
            self.consolidated_amp_fp32_next = _zeros(self.consolidated_grads[torch.float32].numel(), torch.float32, device)
        self.grad_tensors: Dict[int, torch.Tensor] = {}
        self.amp_grad_tensors_next: Dict[int, torch.Tensor] = {}
        self.amp_master_grad_tensors: Dict[int, torch.Tensor] = {}
        for pid, p in zip(self.param_ids, params):
            off = self.offsets[pid]
            if consolidate_master_params and p.dtype == torch.float16:    # :92-98
                self.amp_master_grad_tensors[pid] = self.consolidated_master_grads[p.dtype].narrow(0, off, p.numel()).view(p.shape)
                continue
            self.grad_tensors[pid] = self.consolidated_grads[p.dtype].narrow(0, off, p.numel()).view(p.shape)
            if p.dtype == torch.float32 and self._double_fp32:            # :104-111
                self.amp_grad_tensors_next[pid] = self.consolidated_amp_fp32_next.narrow(0, off, p.numel()).view(p.shape)
            else:
                self.amp_grad_tensors_next[pid] = self.grad_tensors[pid]
        self._copy_plan = _PlanCache()
        self._zero_plan = _PlanCache()
        self._compiled: Dict[int, object] = {}     # id of a view map -> the compiled module's GradBuckets over it

    def consolidate(self) -> None:
        """``GradConsolidation::consolidate`` (``src/comp/ParamStorage.cpp:118-179``): swap the
        two fp32 buckets under amp, then make every ``.grad`` the bucket view - copying a grad
        that lives elsewhere, zeroing the view of a grad that does not exist.  The copies and
        the zero fills of all parameters are two launches."""
        if self._double_fp32:                                             # :119-133
            self.amp_grad_tensors_next, self.grad_tensors = self.grad_tensors, self.amp_grad_tensors_next
            cur = self.consolidated_grads[torch.float32]
            self.consolidated_grads[torch.float32] = self.consolidated_amp_fp32_next
            self.consolidated_amp_fp32_next = cur
        if _native is not None and not self.consolidate_master_params:
            # the walk over the parameters in C++ (two launches at most); one object per view map, since the two
            # fp32 buckets of an amp run swap places at every call
            buckets = self._compiled.get(id(self.grad_tensors))
            if buckets is None:
                params = [self.storage.get_param_tensor(pid) for pid in self.param_ids]
                views = [self.grad_tensors[pid] for pid in self.param_ids]
                buckets = self._compiled[id(self.grad_tensors)] = _native.GradBuckets(_native.TensorList(params),
                                                                                      _native.TensorList(views))
            with torch.no_grad():
                buckets.consolidate()
            return
        copy_src: List[torch.Tensor] = []
        copy_dst: List[torch.Tensor] = []
        zero_dst: List[torch.Tensor] = []
        for pid in self.param_ids:
            p = self.storage.get_param_tensor(pid)
            if self.consolidate_master_params and p.dtype == torch.float16:
                master = self.storage.get_amp_master_param_tensor(pid)    # :139-151
                if master.grad is None:
                    master.grad = self.amp_master_grad_tensors[pid]
                    zero_dst.append(master.grad)
                continue
            con = self.grad_tensors[pid]
            if p.grad is not None:
                if p.grad.data_ptr() == con.data_ptr():                   # :158-160
                    continue
                copy_src.append(p.grad.contiguous())
                copy_dst.append(con)
                p.grad = con                                              # :163-166
            else:
                p.grad = con                                              # :169-175
                zero_dst.append(con)
        with torch.no_grad():
            if copy_src:
                self._copy_plan.get(copy_src, copy_dst).scale_cast(1.0)
            if zero_dst:
                self._zero_plan.get([None] * len(zero_dst), zero_dst).zero()

    def get_consolidated_grads(self) -> List[torch.Tensor]:
        """``getConsolidatedGrads`` (``src/comp/ParamStorage.cpp:181-191``)."""
        return list(self.consolidated_grads.values()) + list(self.consolidated_master_grads.values())


class DistributedGradLocator:
    """ZeRO-style views of a parameter and its gradient for a group of ``nranks`` processes
    (``src/comp/DistributedGradLocator.cpp:10-101``,
    ``src/comp/DistributedParamLocatorBase.cpp:14-80``)."""

    def __init__(self) -> None:
        self.params: Dict[int, torch.Tensor] = {}
        self.layouts: Dict[int, Tuple[int, int, List[int], List[int]]] = {}
        self.nranks: Dict[int, int] = {}
        self.my_indices: Dict[int, int] = {}
        self.buf_tensors: Dict[int, torch.Tensor] = {}
        self.local_param_segments: Dict[int, torch.Tensor] = {}

    def register_grad(self, pid: int, param: torch.Tensor, nranks: int = 1, my_index: int = 0) -> None:
        self.layouts[pid] = _lib.segment_layout(param.numel(), param.element_size(), nranks)   # doRegister
        self.params[pid] = param
        self.nranks[pid] = nranks
        self.my_indices[pid] = my_index

    def registered(self, pid: int) -> bool:
        return pid in self.layouts

    def get_segment_range(self, pid: int, index: Optional[int] = None) -> Tuple[int, int]:
        _, _, offs, srcs = self._layout(pid)
        i = self.my_indices[pid] if index is None else index
        return offs[i], offs[i] + srcs[i]

    def _layout(self, pid: int):
        if pid not in self.layouts:
            raise ValueError(f"Parameter is not registered: {pid}")
        return self.layouts[pid]

    def get_segment(self, pid: int, index: int, grad: bool) -> torch.Tensor:
        lo, hi = self.get_segment_range(pid, index)                        # :36-48
        param = self.params[pid]
        ten = param.grad if grad else param
        if ten is None:
            raise RuntimeError(f"Parameter {pid} has no gradient")
        assert param.numel() >= hi                                         # checkIndices
        return ten.view(-1).narrow(0, lo, hi - lo)

    def get_local_param_segment(self, pid: int) -> torch.Tensor:
        if pid not in self.local_param_segments:                           # :17-26
            param = self.params[pid]
            seg = self.get_segment(pid, self.my_indices[pid], False).detach()
            seg.requires_grad_(param.requires_grad)
            self.local_param_segments[pid] = seg
        return self.local_param_segments[pid]

    def set_grad_to_local_param_segment(self, pid: int) -> None:
        seg = self.get_local_param_segment(pid)                            # :28-34
        if seg.requires_grad:
            seg.grad = self.get_segment(pid, self.my_indices[pid], True)

    def align_buffer(self, pid: int, plans: Optional[Tuple[List, List]] = None) -> torch.Tensor:
        """Re-home the parameter into a zero-padded buffer of the aligned size (:50-63).
        With ``plans`` the copy is only queued, so a caller can batch all parameters."""
        param = self.params[pid]
        aligned = self._layout(pid)[0]
        buf = torch.empty(aligned, dtype=param.dtype, device=param.device)
        pad = buf.narrow(0, param.numel(), aligned - param.numel())
        head = buf.narrow(0, 0, param.numel())
        src = param.detach().contiguous().view(-1)
        if plans is None:
            with torch.no_grad():
                TensorPlan([src, None], [head, pad]).scale_cast(1.0)
                torch.cuda.current_stream(param.device).synchronize()
        else:
            plans[0].extend([src, None])
            plans[1].extend([head, pad])
        self.buf_tensors[pid] = buf
        param.data = head.view(param.shape)
        self.local_param_segments.pop(pid, None)
        return buf

    def get_buffer(self, pid: int, grad: bool = False) -> torch.Tensor:
        buf = self.buf_tensors[pid]                                        # :65-71
        return buf.grad if grad else buf

    def get_buffer_segment(self, pid: int, index: int, grad: bool = False) -> torch.Tensor:
        seg = self._layout(pid)[1]                                         # :73-86
        buf = self.get_buffer(pid, grad)
        return buf.view(-1).narrow(0, seg * index, seg)

    def remove(self, pid: int) -> None:
        for d in (self.params, self.layouts, self.nranks, self.my_indices, self.buf_tensors, self.local_param_segments):
            d.pop(pid, None)

    def clear(self) -> None:
        for d in (self.params, self.layouts, self.nranks, self.my_indices, self.buf_tensors, self.local_param_segments):
            d.clear()


class ParamStorage:
    """Registry keyed by Python ``id()`` of the parameter (``src/bind/PybindUtil.cpp:8-12``),
    with the per-step operations of ``src/comp/ParamStorage.cpp``."""

    def __init__(self) -> None:
        self.params: Dict[int, torch.Tensor] = {}
        self.amp_master_params: Dict[int, torch.Tensor] = {}
        self.amp_param_id_map: Dict[int, int] = {}
        self.graph_params: Dict[str, Dict[str, int]] = {}
        self.grad_cons: Dict[str, GradConsolidation] = {}
        self.zero_grad_locators: Dict[str, DistributedGradLocator] = {}
        self.consolidate = False
        self.use_amp_master_params: Dict[str, bool] = {}
        self.allreduce_amp_master_params = False
        self._sorted_ids: Dict[str, List[int]] = {}
        self._staging = BufferTensorCache()
        self._clip_plans: Dict[Tuple[str, bool], _PlanCache] = {}
        self._zero_plans: Dict[str, _PlanCache] = {}
        self._scale_plans: Dict[Tuple[str, bool], _PlanCache] = {}
        self._stage_plans: Dict[str, _PlanCache] = {}

    # ------------------------------------------------------------------ registry
    def register_param(self, pid: int, tensor: torch.Tensor) -> None:
        self.params[pid] = tensor                                          # registerParam :195-205

    def get_param_tensor(self, pid: int) -> torch.Tensor:
        if pid not in self.params:                                         # :269-273
            raise ValueError(f"Parameter not found: {pid}")
        return self.params[pid]

    def register_amp_master_param(self, model_pid: int, master_pid: int, tensor: torch.Tensor) -> None:
        self.amp_master_params[model_pid] = tensor                         # :715-719
        self.amp_param_id_map[master_pid] = model_pid

    def has_amp_master_param(self, pid: int) -> bool:
        return pid in self.amp_master_params

    def get_amp_master_param_tensor(self, pid: int) -> torch.Tensor:
        if pid not in self.amp_master_params:                              # :648-650
            raise ValueError(f"Amp master parameter not found: {pid}")
        return self.amp_master_params[pid]

    def get_param_ids(self, graph_id: str) -> Dict[str, int]:
        return self.graph_params[graph_id]

    def sorted_param_ids(self, graph_id: str) -> List[int]:
        """``getSortedParamIDs`` (``src/comp/ParamStorage.cpp:23-31``): ids in name order (sorted once per
        deployment: the per-step operations all walk this list)."""
        cached = self._sorted_ids.get(graph_id)
        if cached is None:
            m = self.graph_params[graph_id]
            cached = self._sorted_ids[graph_id] = [m[name] for name in sorted(m)]
        return cached

    def zero_enabled(self, graph_id: str) -> bool:
        return graph_id in self.zero_grad_locators

    # ------------------------------------------------------------------ deployment
    def deploy(self, graph_id: str, graph_params: Dict[str, int], enable_zero: bool = False,
               consolidate: bool = False, use_amp_master_params: bool = False,
               allreduce_amp_master_params: bool = False) -> None:
        """The slice of ``ParamStorage::deploy`` (``src/comp/ParamStorage.cpp:827-1022``) that
        prepares the per-step path: name-sorted id list, ZeRO locator, gradient buckets."""
        self.graph_params[graph_id] = dict(graph_params)
        self._sorted_ids.pop(graph_id, None)
        self.consolidate = consolidate
        self.use_amp_master_params[graph_id] = use_amp_master_params
        self.allreduce_amp_master_params = allreduce_amp_master_params
        ids = self.sorted_param_ids(graph_id)
        if enable_zero:
            loc = DistributedGradLocator()
            for pid in ids:
                loc.register_grad(pid, self.get_param_tensor(pid), 1, 0)
            self.zero_grad_locators[graph_id] = loc
        grad_ids = [pid for pid in ids if self.get_param_tensor(pid).requires_grad]
        if consolidate and grad_ids:
            consolidate_master = use_amp_master_params and allreduce_amp_master_params
            self.grad_cons[graph_id] = GradConsolidation(self, grad_ids, use_amp_master_params, consolidate_master)

    def undeploy(self, graph_id: str) -> None:
        self.graph_params.pop(graph_id, None)
        self._sorted_ids.pop(graph_id, None)
        self.grad_cons.pop(graph_id, None)
        self.zero_grad_locators.pop(graph_id, None)
        for d in (self._clip_plans, self._scale_plans):
            for k in [k for k in d if k[0] == graph_id]:
                d.pop(k).clear()
        if graph_id in self._zero_plans:
            self._zero_plans.pop(graph_id).clear()
        for k in [k for k in self._stage_plans if k.split("/")[0] == graph_id]:
            self._stage_plans.pop(k).clear()
        self._staging.clear(graph_id + "/")

    # ------------------------------------------------------------------ per-step operations
    def prepare_backward(self, graph_id: str) -> None:
        if self.consolidate:                                               # :627-631
            self.consolidate_grads(graph_id)

    def consolidate_grads(self, graph_id: str) -> None:
        if graph_id in self.grad_cons:                                     # :705-713
            self.grad_cons[graph_id].consolidate()

    def _selected(self, graph_id: str, use_amp_master: bool) -> List[torch.Tensor]:
        """The tensor whose gradient counts for a parameter: its amp master, its local ZeRO
        segment, or the parameter itself (``src/comp/ParamStorage.cpp:726-738, 755-766``)."""
        out: List[torch.Tensor] = []
        for pid in self.sorted_param_ids(graph_id):
            if use_amp_master and pid in self.amp_master_params:
                out.append(self.amp_master_params[pid])
            elif self.zero_enabled(graph_id):
                out.append(self.zero_grad_locators[graph_id].get_local_param_segment(pid))
            else:
                out.append(self.get_param_tensor(pid))
        return out

    def _defined_grads(self, graph_id: str, use_amp_master: bool) -> List[torch.Tensor]:
        grads = []
        for t in self._selected(graph_id, use_amp_master):
            if t.grad is not None:
                g = t.grad
                if not g.is_contiguous():
                    raise ValueError("gradients must be contiguous")
                grads.append(g)
        return grads

    def calc_grad_global_l2_norm(self, graph_id: str, use_amp_master: bool) -> float:
        """``calcGradGlobalL2Norm`` (``src/comp/ParamStorage.cpp:747-819``): one read-only
        launch over all gradients in name order, one read-back instead of one ``.item()``
        per parameter."""
        grads = self._defined_grads(graph_id, use_amp_master)
        if not grads:
            return 0.0
        plan = self._clip_plans.setdefault((graph_id, use_amp_master), _PlanCache()).get(grads, grads)
        plan.grad_norm()
        return float(plan.result().norm)

    def clip_grad_norm(self, graph_id: str, max_grad_norm: float, use_amp_master: bool) -> None:
        """``clipGradNorm`` (``src/comp/ParamStorage.cpp:721-745``): norm, then every gradient
        multiplied in place by ``max / (norm + 1e-6)`` iff that sum exceeds ``max``; decided
        and applied on the device without a host round trip."""
        grads = self._defined_grads(graph_id, use_amp_master)
        if not grads:
            return
        plan = self._clip_plans.setdefault((graph_id, use_amp_master), _PlanCache()).get(grads, grads)
        with torch.no_grad():
            plan.fused_step(1.0, float(max_grad_norm), _lib.RG_STEP_IGNORE_OVERFLOW)

    def do_scale_grads(self, graph_id: str, unscale: bool, amp_master_grads: bool, world_size: int = 1) -> None:
        """``doScaleGrads`` (``src/comp/ParamStorage.cpp:598-615``): ``grad *= 1/world`` or
        ``grad *= world``."""
        ratio = 1.0 / float(world_size)
        grads = []
        for pid in self.sorted_param_ids(graph_id):
            p = self.amp_master_params[pid] if (amp_master_grads and pid in self.amp_master_params) else self.get_param_tensor(pid)
            if p.grad is not None:
                grads.append(p.grad)
        if not grads:
            return
        plan = self._scale_plans.setdefault((graph_id, amp_master_grads), _PlanCache()).get(grads, grads)
        with torch.no_grad():
            plan.scale_cast(1.0 / ratio if unscale else ratio)

    def scale_grads(self, graph_id: str, amp_master_grads: bool, world_size: int = 1) -> None:
        self.do_scale_grads(graph_id, False, amp_master_grads, world_size)

    def unscale_grads(self, graph_id: str, amp_master_grads: bool, world_size: int = 1) -> None:
        self.do_scale_grads(graph_id, True, amp_master_grads, world_size)

    def clear_param_grads(self, graph_id: str) -> None:
        """``clearParamGrads`` (``src/comp/ParamStorage.cpp:540-557``)."""
        with torch.no_grad():
            if self.consolidate and graph_id in self.grad_cons:
                for g in self.grad_cons[graph_id].get_consolidated_grads():
                    fill_zero_(g)
                return
            grads = [self.get_param_tensor(pid).grad for pid in self.sorted_param_ids(graph_id)]
            grads = [g for g in grads if g is not None]
            if grads:
                self._zero_plans.setdefault(graph_id, _PlanCache()).get([None] * len(grads), grads).zero()

    # ------------------------------------------------------------------ world-size-1 collectives
    def allreduce_param_grads(self, graph_id: str) -> None:
        """``allReduceParamGrads`` (``src/comp/ParamStorage.cpp:347-394``): a sum over one
        process, pre-multiplied by 1/1 - nothing to do."""

    def allreduce_param_grads_zero(self, graph_id: str) -> List[torch.Tensor]:
        """``allReduceParamGradsZero`` (``src/comp/ParamStorage.cpp:440-520``) for a group of
        one: every defined gradient is packed (cast to fp32 for half parameters when masters
        are all-reduced) into a zero-padded staging buffer of the aligned size, the
        reduce-scatter over one rank returns the buffer itself, and the first ``numel``
        elements are copied back over the gradient (``:419-427``).  All parameters share two
        launches.  Returns the staging buffers (kept alive by the caller, as ``:433`` does)."""
        srcs: List[Optional[torch.Tensor]] = []
        dsts: List[torch.Tensor] = []
        back_src: List[torch.Tensor] = []
        back_dst: List[torch.Tensor] = []
        bufs: List[torch.Tensor] = []
        for pid in self.sorted_param_ids(graph_id):
            param = self.get_param_tensor(pid)
            if not param.requires_grad or param.grad is None:              # :471-478
                continue
            grad = param.grad
            aligned = _lib.aligned_numel(grad.numel(), grad.element_size(), 1)
            bdt = torch.float32 if (self.allreduce_amp_master_params and param.dtype == torch.float16) else param.dtype
            buf = self._staging.get(f"{graph_id}/{pid}", aligned, bdt, grad.device)
            srcs += [grad.view(-1), None]
            dsts += [buf.narrow(0, 0, grad.numel()), buf.narrow(0, grad.numel(), aligned - grad.numel())]
            back_src.append(buf.narrow(0, 0, grad.numel()))
            back_dst.append(grad.view(-1))
            bufs.append(buf)
        if srcs:
            # the staging buffers persist (BufferTensorCache), so the tables are built once
            with torch.no_grad():
                self._stage_plans.setdefault(graph_id + "/pack", _PlanCache()).get(srcs, dsts).scale_cast(1.0)
                self._stage_plans.setdefault(graph_id + "/back", _PlanCache()).get(back_src, back_dst).scale_cast(1.0)
        return bufs

    def bcast_params_zero(self, graph_id: str, grad: bool = False) -> None:
        """``bcastParamsZero`` (``src/comp/ParamStorage.cpp:559-596``): the all-gather of one
        segment into its own buffer - nothing to do."""

    def set_grad_to_local_param_segment(self, graph_id: str) -> None:
        if self.zero_enabled(graph_id):                                    # :522-529
            loc = self.zero_grad_locators[graph_id]
            for pid in self.sorted_param_ids(graph_id):
                if self.get_param_tensor(pid).grad is not None:
                    loc.set_grad_to_local_param_segment(pid)

    def align_buffer_zero(self, graph_id: str) -> None:
        if self.zero_enabled(graph_id):                                    # :531-538
            loc = self.zero_grad_locators[graph_id]
            srcs: List = []
            dsts: List = []
            for pid in self.sorted_param_ids(graph_id):
                loc.align_buffer(pid, (srcs, dsts))
            if srcs:
                with torch.no_grad():
                    TensorPlan(srcs, dsts).scale_cast(1.0)

    def gather_tensor_zero(self, ten: torch.Tensor, pid: int) -> torch.Tensor:
        """``gatherTensorZero`` (``src/comp/ParamStorage.cpp:670-685``) with one rank: the only piece is the
        whole flattened tensor; it comes back in the parameter's shape
        (``DistributedParamLocatorBase::gather``, ``src/comp/DistributedParamLocatorBase.cpp:149-152``)."""
        for graph_id, loc in self.zero_grad_locators.items():
            if loc.registered(pid) and pid in self.graph_params.get(graph_id, {}).values():
                param = loc.params[pid]
                if ten.numel() != param.numel():
                    raise ValueError(f"tensor has {ten.numel()} elements, parameter {pid} has {param.numel()}")
                return ten.detach().reshape(param.shape)
        raise ValueError(f"Param is not registered for zero: {pid}")

    def get_local_param_range(self, graph_id: str, pid: int) -> Tuple[int, int]:
        return self.zero_grad_locators[graph_id].get_segment_range(pid)

    def get_local_param_segment(self, graph_id: str, pid: int) -> torch.Tensor:
        return self.zero_grad_locators[graph_id].get_local_param_segment(pid)
