"""Multi-tensor operations on PyTorch-ROCm tensors, backed by libranncgrad.

``TensorPlan`` ties a list of (source, destination) tensor pairs to one device-side
descriptor table.  PyTorch supplies device memory and the current stream; all arithmetic
runs in the HIP library.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from . import _lib

_CODES = {torch.float32: _lib.RG_F32, torch.float16: _lib.RG_F16, torch.bfloat16: _lib.RG_BF16}


def dtype_code(dtype: torch.dtype) -> int:
    """The reference admits float, half and bfloat16 only (assert at
    ``src/comp/ParamStorage.cpp:51-53``); anything else is a ``ValueError`` here."""
    try:
        return _CODES[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype}: expected float32, float16 or bfloat16") from None


try:        # the compiled module asks PyTorch's stream registry directly (a fifth of the Python route's cost)
    from ._ranncgrad import current_stream as _native_current_stream
except ImportError:
    _native_current_stream = None


def stream_handle(device: torch.device) -> int:
    """The ``hipStream_t`` PyTorch currently launches on for ``device``, as an integer."""
    if _native_current_stream is not None:
        index = device.index
        return _native_current_stream(torch.cuda.current_device() if index is None else index)
    return int(torch.cuda.current_stream(device).cuda_stream)


def _check_tensor(t: torch.Tensor, device: torch.device, what: str, i: int) -> None:
    if not t.is_cuda:
        raise ValueError(f"{what}[{i}] is not on a GPU (device {t.device})")
    if t.device != device:
        raise ValueError(f"{what}[{i}] is on {t.device}, expected {device}")
    if not t.is_contiguous():
        raise ValueError(f"{what}[{i}] is not contiguous")


class TensorPlan:
    """Descriptor table over tensor pairs.  ``srcs[i] is None`` = no gradient (reads as
    zeros); ``dsts`` may be None for a norm-only plan; ``dsts[i] is srcs[i]`` = in place."""

    def __init__(self, srcs: Sequence[Optional[torch.Tensor]], dsts: Optional[Sequence[Optional[torch.Tensor]]] = None,
                 chunk_elems: int = 0, device: Optional[torch.device] = None):
        n = len(srcs)
        if dsts is None:
            dsts = [None] * n
        if len(dsts) != n:
            raise ValueError("srcs and dsts differ in length")
        if device is None:
            for t in list(srcs) + list(dsts):
                if t is not None:
                    device = t.device
                    break
        if device is None:
            device = torch.device("cuda", torch.cuda.current_device())
        device = torch.device(device)
        if device.type != "cuda":
            raise ValueError(f"TensorPlan needs GPU tensors, got {device}")
        if device.index is None:
            device = torch.device("cuda", torch.cuda.current_device())
        self.device = device
        sp: List[Optional[int]] = []
        dp: List[Optional[int]] = []
        numels: List[int] = []
        sd: List[int] = []
        dd: List[int] = []
        for i, (s, d) in enumerate(zip(srcs, dsts)):
            if s is None and d is None:
                raise ValueError(f"pair {i} has neither source nor destination")
            if s is not None:
                _check_tensor(s, device, "src", i)
            if d is not None:
                _check_tensor(d, device, "dst", i)
            if s is not None and d is not None and s.numel() != d.numel():
                raise ValueError(f"pair {i}: source has {s.numel()} elements, destination {d.numel()}")
            ref = s if s is not None else d
            numels.append(int(ref.numel()))
            sd.append(dtype_code((s if s is not None else d).dtype))
            dd.append(dtype_code((d if d is not None else s).dtype))
            sp.append(int(s.data_ptr()) if s is not None and s.numel() else None)
            dp.append(int(d.data_ptr()) if d is not None and d.numel() else None)
        # keep the memory alive for as long as the table points at it
        self._srcs, self._dsts = list(srcs), list(dsts)
        self._numels, self._sd, self._dd = numels, sd, dd
        self.plan = _lib.Plan(device.index, sp, dp, numels, sd, dd, chunk_elems)

    @property
    def n(self) -> int:
        return self.plan.n

    def _stream(self) -> int:
        return stream_handle(self.device)

    def update(self, srcs: Optional[Sequence[Optional[torch.Tensor]]] = None,
               dsts: Optional[Sequence[Optional[torch.Tensor]]] = None) -> None:
        """Point the table at new tensors of the same sizes and dtypes."""
        def ptrs(ts, old, codes, what):
            if ts is None:
                return None
            if len(ts) != self.n:
                raise ValueError(f"{what}: expected {self.n} tensors")
            out = []
            for i, t in enumerate(ts):
                if t is None:
                    out.append(None)
                    continue
                _check_tensor(t, self.device, what, i)
                if t.numel() != self._numels[i] or dtype_code(t.dtype) != codes[i]:
                    raise ValueError(f"{what}[{i}] changed size or dtype")
                out.append(int(t.data_ptr()) if t.numel() else None)
            return out
        sp = ptrs(srcs, self._srcs, self._sd, "src")
        dp = ptrs(dsts, self._dsts, self._dd, "dst")
        self.plan.update_pointers(sp, dp, self._stream())
        if srcs is not None:
            self._srcs = list(srcs)
        if dsts is not None:
            self._dsts = list(dsts)

    def tune(self) -> int:
        """Let the library measure, on these very tensors, which hand-out order of tiles to the XCDs is fastest
        for the plan's writing passes, and keep it.  Overwrites the destinations with ``cast(src)`` and waits for
        the stream: call it once, right after building a plan whose destinations hold nothing yet."""
        return self.plan.tune(self._stream())

    def write_order(self) -> int:
        return self.plan.write_order

    def set_write_order(self, order: int) -> None:
        """Use an order measured earlier (on a table of the same layout) instead of measuring again."""
        self.plan.set_write_order(order)

    def repoint_sources(self, src_ptrs: Sequence[int]) -> None:
        """New source addresses (one per tensor, same sizes and dtypes, contiguous) without any per-tensor check:
        for callers that have established those facts themselves."""
        if len(src_ptrs) != self.n:
            raise ValueError(f"expected {self.n} source addresses")
        self.plan.update_pointers(src_ptrs, None, self._stream())

    def drop_sources(self) -> None:
        """Stop keeping the source tensors alive (the table still points at their memory).  For callers
        that have queued every kernel reading them and will ``update`` the table before its next use;
        memory PyTorch then reuses on the same stream is ordered behind those kernels."""
        self._srcs = [None] * len(self._srcs)

    def fused_step(self, inv_scale: float, max_norm: float, flags: int = _lib.RG_STEP_DEFAULT) -> None:
        self.plan.fused_step(inv_scale, max_norm, flags, self._stream())

    def step_begin(self, inv_scale: float) -> None:
        self.plan.step_begin(inv_scale, self._stream())

    def step_begin_scaled(self, inv_scale_ptr: int) -> None:
        """``step_begin`` whose kernels read ``inv_scale`` from device memory (the loss scaler's state)."""
        self.plan.step_begin_scaled(inv_scale_ptr, self._stream())

    def step_finish(self, max_norm: float, flags: int = _lib.RG_STEP_DEFAULT) -> None:
        self.plan.step_finish(max_norm, flags, self._stream())

    def step_decide(self, max_norm: float, flags: int = _lib.RG_STEP_DEFAULT) -> None:
        self.plan.step_decide(max_norm, flags, self._stream())

    def unscale_pack(self, inv_scale: float) -> None:
        self.plan.unscale_pack(inv_scale, self._stream())

    def step_apply_clip(self, max_norm: float, flags: int = _lib.RG_STEP_DEFAULT) -> None:
        self.plan.step_apply_clip(max_norm, flags, self._stream())

    def accumulate(self, scale: float = 1.0) -> None:
        self.plan.accumulate(scale, self._stream())

    def unscale_accumulate(self, inv_scale: float) -> None:
        self.plan.unscale_accumulate(inv_scale, self._stream())

    def grad_norm(self) -> None:
        self.plan.grad_norm(self._stream())

    def scale_cast(self, scale: float = 1.0) -> None:
        self.plan.scale_cast(scale, self._stream())

    def zero(self) -> None:
        self.plan.zero(self._stream())

    def result(self) -> _lib.StepResult:
        return self.plan.read_result(self._stream())

    def tensor_norms(self) -> List[float]:
        return self.plan.read_tensor_norms(self._stream())

    def close(self) -> None:
        self.plan.close()

    def is_open(self) -> bool:
        return self.plan.is_open()


def fill_zero_(t: torch.Tensor) -> torch.Tensor:
    """``t.zero_()`` through the library's fill kernel."""
    if not t.is_cuda or not t.is_contiguous():
        raise ValueError("fill_zero_ needs a contiguous GPU tensor")
    if t.numel():
        _lib.fill_zero(int(t.data_ptr()), t.numel() * t.element_size(), t.device.index, stream_handle(t.device))
    return t


def copy_cast_(dst: torch.Tensor, src: Optional[torch.Tensor], scale: float = 1.0) -> torch.Tensor:
    """``dst.copy_(src)`` (with dtype conversion, optionally scaled) for one pair of contiguous
    GPU tensors, without building a table; ``src is None`` stores zeros."""
    if not dst.is_cuda or not dst.is_contiguous():
        raise ValueError("copy_cast_ needs a contiguous GPU destination")
    if src is not None:
        if src.device != dst.device or not src.is_contiguous():
            raise ValueError("copy_cast_ needs a contiguous source on the destination's device")
        if src.numel() != dst.numel():
            raise ValueError(f"copy_cast_: source has {src.numel()} elements, destination {dst.numel()}")
    if dst.numel():
        sdt = dtype_code(src.dtype if src is not None else dst.dtype)
        _lib.scale_cast_single(int(src.data_ptr()) if src is not None else None, int(dst.data_ptr()), dst.numel(),
                               sdt, dtype_code(dst.dtype), scale, dst.device.index, stream_handle(dst.device))
    return dst
