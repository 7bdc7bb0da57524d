"""Helper of the optimizer wrapper (``pyrannc/utils.py:4-7``)."""
import torch


def _to_in_place(tensors, device):
    """Re-home the storage of every tensor on ``device``.  The tensor objects stay the same, so the module,
    the optimizer and the registry keep pointing at them."""
    with torch.no_grad():
        for t in tensors:
            t.data = t.data.to(device=device, dtype=t.dtype)
