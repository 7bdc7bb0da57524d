"""Gradient summation over the clones of shared parameters.

When a parameter is used at several places of a sub-graph the reference gives every use
its own clone and, at the end of each backward, folds the clones' gradients into the
parameter's (``TorchDriver::backward``, block "backward_sum_paramgrad",
``src/torch/TorchDriver.cpp:781-822``): ``grad_sum = 0; for clone: grad_sum += clone.grad;
clone.grad = 0``, then ``param.grad += grad_sum`` (or ``param.grad = copy of grad_sum`` when
the parameter had none) - one ``add_`` / ``zero_`` / ``copy_`` launch per tensor.  Here each
of those loops is one launch over all shared parameters (``rg_accumulate``, ``rg_zero``,
``rg_scale_cast``); the order of the additions, and so every bit, is the reference's.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from .multi_tensor import fill_zero_
from .param_storage import _PlanCache


class CloneGradSummer:
    """``params[i]`` is a shared parameter, ``clones[i]`` its clones in the reference's order."""

    def __init__(self, params: Sequence[torch.Tensor], clones: Sequence[Sequence[torch.Tensor]]):
        if len(params) != len(clones):
            raise ValueError("one list of clones per parameter")
        for p, cl in zip(params, clones):
            for c in cl:
                if c.numel() != p.numel() or c.dtype != p.dtype or c.device != p.device:
                    raise ValueError("a clone must have its parameter's size, dtype and device")
        self.params = list(params)
        self.clones = [list(cl) for cl in clones]
        # the [GRAD_SUM] buffers of the reference's buffer cache: one flat allocation per dtype
        self._sums: List[Optional[torch.Tensor]] = [None] * len(self.params)
        by_dtype = {}
        for i, p in enumerate(self.params):
            if self.clones[i]:
                by_dtype.setdefault((p.dtype, p.device), []).append(i)
        self._flat = []
        for (dt, dev), idx in by_dtype.items():
            flat = torch.empty(sum(self.params[i].numel() for i in idx), dtype=dt, device=dev)
            off = 0
            for i in idx:
                n = self.params[i].numel()
                self._sums[i] = flat.narrow(0, off, n).view(self.params[i].shape)
                off += n
            self._flat.append(flat)
        self._plans = {}

    def _plan(self, tag, srcs, dsts):
        cache = self._plans.setdefault(tag, _PlanCache())
        return cache.get(srcs, dsts)

    @torch.no_grad()
    def sum_into_params(self) -> None:
        for flat in self._flat:
            fill_zero_(flat)                                              # grad_sum.zero_()
        depth = max((len(cl) for cl in self.clones), default=0)
        for k in range(depth):                                            # grad_sum.add_(clone.grad); clone.grad.zero_()
            srcs, dsts = [], []
            for i, cl in enumerate(self.clones):
                if k < len(cl) and cl[k].grad is not None:
                    if not cl[k].grad.is_contiguous():
                        raise ValueError("clone gradients must be contiguous")
                    srcs.append(cl[k].grad)
                    dsts.append(self._sums[i])
            if srcs:
                self._plan(("add", k, len(srcs)), srcs, dsts).accumulate(1.0)
                self._plan(("zero", k, len(srcs)), [None] * len(srcs), srcs).zero()
        add_src, add_dst, new_src, new_dst = [], [], [], []
        for i, p in enumerate(self.params):
            if not self.clones[i]:
                continue
            if p.grad is not None:                                        # grad.add_(grad_sum)
                if not p.grad.is_contiguous():
                    raise ValueError("parameter gradients must be contiguous")
                add_src.append(self._sums[i])
                add_dst.append(p.grad)
            else:                                                         # grad = buffer; grad.copy_(grad_sum)
                p.grad = torch.empty_like(self._sums[i])
                new_src.append(self._sums[i])
                new_dst.append(p.grad)
        if add_src:
            self._plan(("padd", len(add_src)), add_src, add_dst).accumulate(1.0)
        if new_src:
            self._plan(("pnew", len(new_src)), new_src, new_dst).scale_cast(1.0)
