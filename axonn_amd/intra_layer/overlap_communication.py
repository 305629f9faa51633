"""Deferred weight-gradient accumulation and the `optimize_communication`
context, same surface as axonn/intra_layer/overlap_communication.py.

On one GPU there is no communication to overlap.  What remains of the
reference's behaviour is (a) the module flags the Linear backward reads
(:11-13) and (b) the way weight gradients reach `param.grad` when
`overlap_reduce_scatter` is on: the backward returns no weight gradient and the
gradient is added to `param.grad` by this module (:33-47).  Here the wgrad
kernel performs that addition itself (dW += dY^T X, accumulate in place), so
`accumulate()` only has work left for gradients that could not be fused.
"""

from contextlib import contextmanager

import torch

OVERLAP_REDUCE_SCATTER = False
OVERLAP_ALL_REDUCE = False
ALL_GATHER_ITERATOR = None

handles = []
pending_grad_accumulations = []
weights_cache = {}


def register_handle(handle):
    handles.append(handle)


def clear_handles():
    global handles
    handles = []


def accumulate_later(param, grad):
    pending_grad_accumulations.append([param, grad])


@torch.no_grad()
def accumulate():
    global pending_grad_accumulations
    for param, grad in pending_grad_accumulations:
        if param.grad is None:
            param.grad = grad.to(param.dtype)
        else:
            param.grad.add_(grad.to(param.dtype))
    pending_grad_accumulations = []


def clear_weights_cache():
    global weights_cache
    weights_cache = {}


@contextmanager
def overlap_all_gathers_for_checkpointed_forward(model_object_for_overlapping_allgathers):
    yield None


@contextmanager
def optimize_communication(
    overlap_all_reduce=True,
    overlap_reduce_scatter=False,
    overlap_all_gather=False,
    model_object_for_overlapping_allgathers=None,
    *args,
    **kwargs,
):
    """Same arguments as the reference (:124-159).  `overlap_reduce_scatter`
    switches the Linear backward to in-place accumulation of dW into
    `weight.grad`; the other flags have nothing to act on with one rank."""
    global OVERLAP_ALL_REDUCE, OVERLAP_REDUCE_SCATTER
    if overlap_all_gather and model_object_for_overlapping_allgathers is None:
        raise ValueError(
            "You need to pass your model as an argument - "
            "optimize_communication(...,model_object_"
            "for_overlapping_allgathers=model, ...)"
            "if overlap_all_gather is True"
        )
    OVERLAP_ALL_REDUCE = overlap_all_reduce
    OVERLAP_REDUCE_SCATTER = overlap_reduce_scatter
    try:
        yield None
    finally:
        clear_handles()
        accumulate()
        clear_weights_cache()
        OVERLAP_ALL_REDUCE = False
        OVERLAP_REDUCE_SCATTER = False
