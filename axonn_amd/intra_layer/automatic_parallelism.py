"""`auto_parallelize`: models declared inside the context get the tensor-parallel
Linear wherever they ask for `torch.nn.Linear`
(axonn/intra_layer/automatic_parallelism.py:14-97; the Embedding half of the
reference is commented out there, :89-97, and is not mirrored)."""

from contextlib import contextmanager

import torch.nn as nn

from axonn_amd import axonn as ax

_TorchLinear = nn.Linear


def is_parallelizable_linear(in_features, out_features):
    """The layer can be sharded over the current grid: rows over G_intra_r, columns
    over G_intra_c, the shard's elements over G_intra_d (:14-21).  Always true on
    the 1 x 1 x 1 grid this build runs."""
    rows, cols, depth = ax.config.G_intra_r, ax.config.G_intra_c, ax.config.G_intra_d
    if out_features % rows or in_features % cols:
        return False
    return (out_features * in_features // (rows * cols)) % depth == 0


class _LinearFactory:
    """Stands in for `nn.Linear` inside the context: calling it builds the parallel
    layer when the shape allows, else the original class (:33-62)."""

    def __new__(cls, in_features, out_features, *args, bias=True, device=None, dtype=None, **kwargs):
        from .fully_connected import Linear

        make = Linear if is_parallelizable_linear(in_features, out_features) else _TorchLinear
        layer = make(in_features, out_features, *args, bias=bias, **kwargs)
        if device is not None:
            layer = layer.to(device)
        if dtype is not None:
            layer = layer.to(dtype)
        return layer


@contextmanager
def auto_parallelize():
    nn.Linear = _LinearFactory
    try:
        yield None
    finally:
        nn.Linear = _TorchLinear
