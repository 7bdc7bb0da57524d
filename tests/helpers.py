"""Shared test utilities: bit-level comparison and misaligned device arenas."""
from __future__ import annotations

from typing import List, Sequence

import torch

INT_VIEW = {torch.float32: torch.int32, torch.float16: torch.int16, torch.bfloat16: torch.int16}
TORCH_DTYPE = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def assert_bits_equal(got: torch.Tensor, want: torch.Tensor, what: str = "") -> None:
    """Bit-for-bit equality; two NaNs match whatever their payloads (NaN payload bits are
    not specified by the path: library and hardware conversions quiet them differently)."""
    assert got.dtype == want.dtype and got.shape == want.shape, (what, got.dtype, want.dtype, got.shape, want.shape)
    g = got.detach().cpu().contiguous()
    w = want.detach().cpu().contiguous()
    same = g.view(INT_VIEW[g.dtype]) == w.view(INT_VIEW[w.dtype])
    both_nan = torch.isnan(g) & torch.isnan(w)
    ok = same | both_nan
    if not bool(ok.all()):
        bad = (~ok).flatten().nonzero().flatten()
        i = int(bad[0])
        raise AssertionError(
            f"{what}: {bad.numel()} of {g.numel()} elements differ; first at {i}: "
            f"got {g.flatten()[i].item()!r} want {w.flatten()[i].item()!r}")


def place_in_arena(tensors: Sequence[torch.Tensor], device, lead_elems: int = 1, gap_elems: int = 1,
                   fill: float = 0.0) -> List[torch.Tensor]:
    """Copy CPU tensors (one dtype) into a single device allocation, `lead_elems` elements in
    and `gap_elems` apart, so that most views start off any 16-byte boundary.  Returns the
    device views (each contiguous, flat shape preserved)."""
    assert len({t.dtype for t in tensors}) <= 1
    if not tensors:
        return []
    dt = tensors[0].dtype
    total = lead_elems + sum(t.numel() + gap_elems for t in tensors)
    arena = torch.full((total,), fill, dtype=dt, device=device)
    views = []
    off = lead_elems
    for t in tensors:
        v = arena.narrow(0, off, t.numel()).view(t.shape)
        v.copy_(t)
        views.append(v)
        off += t.numel() + gap_elems
    return views
