"""Construction-time parameter sharding: ``DistributedParamLocator``
(``src/comp/DistributedParamLocator.cpp:14-83``) with ``gather``
(``src/comp/DistributedParamLocatorBase.cpp:96-153``) for a world of one process.

Copies and casts run in the HIP library; the layout arithmetic is the library's
``rg_segment_layout``.  With one rank the all-gather is the identity, so ``load`` is
"pad the segment to the segment size, narrow to numel, view, move to the host".
"""
from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from . import _lib
from .multi_tensor import copy_cast_, dtype_code


class DistributedParamLocator:
    def __init__(self, rank: int = 0, world_size: int = 1) -> None:
        self.rank, self.world_size = rank, world_size
        self.layouts: Dict[int, Tuple[int, int, List[int], List[int]]] = {}
        self.shapes: Dict[int, torch.Size] = {}
        self.requires_grad: Dict[int, bool] = {}
        self.param_parts: Dict[int, torch.Tensor] = {}

    def _layout(self, pid: int):
        if pid not in self.layouts:
            raise ValueError(f"Parameter is not registered: {pid}")
        return self.layouts[pid]

    def store(self, pid: int, param: torch.Tensor) -> torch.Tensor:
        """Register the layout and return this rank's segment, a fresh tensor holding
        ``flatten(param)[offset : offset + src_size]`` (``:14-38``)."""
        dtype_code(param.dtype)
        lay = _lib.segment_layout(param.numel(), param.element_size(), self.world_size)
        self.layouts[pid] = lay
        self.shapes[pid] = param.shape
        self.requires_grad[pid] = bool(param.requires_grad)
        off, src = lay[2][self.rank], lay[3][self.rank]
        flat = param.detach().contiguous().view(-1).narrow(0, off, src)
        if param.is_cuda:
            part = torch.empty(src, dtype=param.dtype, device=param.device)
            if src > 0:
                with torch.no_grad():
                    copy_cast_(part, flat)
        else:
            # A parameter still on the host (modules are built there): its slice is uploaded,
            # which is a transfer and not arithmetic, and the segment lives on the GPU.
            if not torch.cuda.is_available():
                raise RuntimeError("store_dist_param needs a GPU: segments are kept in device memory")
            part = flat.to(torch.device("cuda", torch.cuda.current_device()))
        part.requires_grad_(param.requires_grad)
        self.param_parts[pid] = part
        return part

    def get_segment(self, pid: int) -> torch.Tensor:
        self._layout(pid)
        return self.param_parts[pid]

    def set(self, pid: int, src: torch.Tensor) -> None:
        """Copy this rank's slice of a full tensor into the segment (``:51-67``)."""
        lay = self._layout(pid)
        off, n = lay[2][self.rank], lay[3][self.rank]
        if n > 0:
            part = self.param_parts[pid]
            with torch.no_grad():
                copy_cast_(part.detach(), src.detach().to(part.device).contiguous().view(-1).narrow(0, off, n))

    def set_scalar_type(self, pid: int, dtype: torch.dtype) -> None:
        """``param_part.to(stype)`` with requires_grad preserved (``:69-83``)."""
        self._layout(pid)
        dtype_code(dtype)
        part = self.param_parts[pid]
        if part.dtype == dtype:
            return
        new = torch.empty(part.numel(), dtype=dtype, device=part.device)
        with torch.no_grad():
            copy_cast_(new, part.detach())
        new.requires_grad_(self.requires_grad[pid])
        self.param_parts[pid] = new

    def get_segment_range(self, pid: int) -> Tuple[int, int]:
        lay = self._layout(pid)
        return lay[2][self.rank], lay[2][self.rank] + lay[3][self.rank]

    def load(self, pid: int) -> torch.Tensor:
        """``gather`` with one rank (``DistributedParamLocatorBase.cpp:96-153``): the segment,
        zero-padded to the segment size, narrowed to numel, viewed in the original shape,
        on the host, detached, requires_grad restored."""
        lay = self._layout(pid)
        part = self.param_parts[pid]
        seg = lay[1]
        buf = torch.empty(seg * self.world_size, dtype=part.dtype, device=part.device)
        with torch.no_grad():
            copy_cast_(buf.narrow(0, 0, part.numel()), part.detach())
            if seg > part.numel():
                copy_cast_(buf.narrow(0, part.numel(), seg - part.numel()), None)
        numel = 1
        for s in self.shapes[pid]:
            numel *= int(s)
        out = buf.narrow(0, 0, numel).view(self.shapes[pid]).cpu().detach()
        out.requires_grad_(self.requires_grad[pid])
        return out

    def registered(self, pid: int) -> bool:
        return pid in self.layouts

    def remove(self, pid: int) -> None:
        for d in (self.layouts, self.shapes, self.requires_grad, self.param_parts):
            d.pop(pid, None)

    def clear(self) -> None:
        for d in (self.layouts, self.shapes, self.requires_grad, self.param_parts):
            d.clear()
