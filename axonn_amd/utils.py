"""Flat-buffer helper, same contract as axonn/utils.py:11-30."""

from typing import List

import torch


def _coalesce_and_reassign(tensors: List[torch.Tensor]) -> torch.Tensor:
    """Packs `tensors` back to back (no padding) into one flat 1-D buffer and
    re-points every tensor's `.data` at its slice of that buffer."""
    if len(tensors) == 0:
        return torch.empty(0)
    first = tensors[0]
    total = sum(t.numel() for t in tensors)
    flat = torch.empty(total, dtype=first.dtype, device=first.device)
    offset = 0
    for t in tensors:
        n = t.numel()
        view = flat[offset:offset + n].view(t.shape)
        view.copy_(t.data)
        t.data = view
        offset += n
    return flat
