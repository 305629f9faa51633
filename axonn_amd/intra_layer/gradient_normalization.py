"""Gradient clipping by a global p-norm, same signature and return value as
axonn/intra_layer/gradient_normalization.py:37-95.

The reference takes one `torch.norm(g, p)` per gradient, all-reduces the p-th power
of every tensor-parallel group's norm and multiplies every gradient by the clamped
coefficient.  With one rank per group the total is the p-norm over all gradients
(for p = 0, torch.norm's count: the number of gradients with a non-zero element);
here one multi-tensor kernel reads the gradients once (sum of |g|^p in fp32 per
workgroup, fp64 across workgroups), leaves norm and coefficient on the device, and
a second multi-tensor kernel scales the gradients in place - no host
synchronisation.  `get_total_norm` takes any order, +inf and -inf included (the largest
and the smallest |g|), as the reference's passes any order on to torch.norm (:18-34);
`clip_grad_norm_` raises for p = inf as the reference does (:38-39), and for p = -inf,
where the reference's `norm ** norm_type` (:74-85) has no meaning.
"""

from collections import defaultdict

import torch
from torch import inf

from .. import ops


def get_total_norm(tensors, norm_type=2.0, error_if_nonfinite=False):
    """p-norm over a list of tensors (gradient_normalization.py:18-34)."""
    if len(tensors) == 0:
        return torch.tensor(0.0)
    result = _scan(tensors, 0.0, norm_type)
    total = result.total_norm.clone()
    if error_if_nonfinite and not bool(torch.isfinite(total)):
        raise RuntimeError(
            f"The total norm of order {norm_type} for gradients from "
            "`parameters` is non-finite, so it cannot be clipped. To disable "
            "this error and scale the gradients by the non-finite norm anyway, "
            "set `error_if_nonfinite=False`"
        )
    return total


def _scan(grads, max_norm, norm_type=2.0):
    by_dtype = defaultdict(list)
    for g in grads:
        by_dtype[g.dtype].append(g.detach())
    result = None
    for group in by_dtype.values():
        result = ops.mt_scan(group, 1.0, max_norm, result=result, accumulate=result is not None,
                             norm_type=norm_type)
    return result


def clip_grad_norm_(parameters, max_norm, norm_type=2.0, error_if_nonfinite=False):
    if norm_type == inf or norm_type == -inf:
        raise NotImplementedError
    if isinstance(parameters, torch.Tensor):
        parameters = [parameters]
    grads = []
    for p in parameters:
        if hasattr(p, "is_tensor_parallel") and p.is_tensor_parallel:
            assert hasattr(
                p, "process_group_for_norm_reduction"
            ), "each tensor parallel tensor should have a process group for all-reducing norms"
        if p.grad is not None:
            grads.append(p.grad)
    max_norm = float(max_norm)
    norm_type = float(norm_type)
    if len(grads) == 0:
        return torch.tensor(0.0)
    result = _scan(grads, max_norm, norm_type)
    total_norm = result.total_norm.clone()
    if error_if_nonfinite and not bool(torch.isfinite(total_norm)):
        raise RuntimeError(
            f"The total norm of order {norm_type} for gradients from "
            "`parameters` is non-finite, so it cannot be clipped. To disable "
            "this error and scale the gradients by the non-finite norm anyway, "
            "set `error_if_nonfinite=False`"
        )
    by_dtype = defaultdict(list)
    for g in grads:
        by_dtype[g.dtype].append(g.detach())
    for group in by_dtype.values():
        ops.mt_scale(group, 1.0, scan=result, use_clip=True)
    return total_norm
