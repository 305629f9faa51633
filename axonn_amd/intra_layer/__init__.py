"""Intra-layer (tensor-parallel) layers and helpers on a one-GPU grid; the
names axonn/intra_layer/__init__.py exports for the hot path."""

from contextlib import contextmanager

import torch

from .fully_connected import Linear, AsyncLinear, FusedLinear  # noqa: F401
from .embedding import Embedding  # noqa: F401
from .communication import Drop, Gather  # noqa: F401
from .gradient_normalization import clip_grad_norm_  # noqa: F401
from .overlap_communication import optimize_communication  # noqa: F401
from .automatic_parallelism import auto_parallelize  # noqa: F401
from .overlap_communication import (  # noqa: F401
    overlap_all_gathers_for_checkpointed_forward,
)

NO_GRADIENT_SYNC = False


@contextmanager
def no_grad_sync():
    """axonn/intra_layer/__init__.py:27-35."""
    global NO_GRADIENT_SYNC
    old_val = NO_GRADIENT_SYNC
    try:
        NO_GRADIENT_SYNC = True
        yield None
    finally:
        NO_GRADIENT_SYNC = old_val


@torch.no_grad()
def sync_gradients(model, gradient_attr_name="grad", mean=False, vectorize=False,
                   expert_mode=False):
    """Gradient all-reduce over the data- and depth-parallel groups
    (axonn/intra_layer/__init__.py:114-173).  Every group has one rank here, so
    the sums are the gradients themselves and the mean divides by one."""
    return None
