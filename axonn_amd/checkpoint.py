"""Per-shard checkpoint files, with the reference's interface (axonn/checkpoint.py).

Every tensor-parallel rank of the first data-parallel group writes its own shard of the
state under a folder named after its (row, column, depth) coordinates (:11-15, :18-27).
`Linear` and `Embedding` accept such sharded 1-D weights as well as full 2-D ones when a
state dict is loaded.

The reference's `load` looks for `<folder>/<prefix>_<name>.pt` (:34-36), a path its
`save` never writes (`<folder>/<prefix>/<name>.pt`), and returns its argument unchanged
(:37-38).  Here `load` reads the file `save` wrote and returns what it held.
"""

import os

import torch

from . import config


def get_prefix_for_checkpoint():
    return "tp_row_%d_col_%d_depth_%d" % (
        config.intra_layer_row_parallel_rank,
        config.intra_layer_column_parallel_rank,
        config.intra_layer_depth_parallel_rank,
    )


def _checkpoint_file(checkpoint_folder, checkpoint_name):
    return os.path.join(checkpoint_folder, get_prefix_for_checkpoint(), "%s.pt" % checkpoint_name)


def save(state, checkpoint_folder, checkpoint_name, overwrite=True):
    if config.data_parallel_rank != 0:
        return
    checkpoint_file = _checkpoint_file(checkpoint_folder, checkpoint_name)
    os.makedirs(os.path.dirname(checkpoint_file), exist_ok=True)
    if os.path.exists(checkpoint_file) and not overwrite:
        raise ValueError(f"Checkpoint {checkpoint_file} already exists")
    torch.save(state, checkpoint_file)


def load(state, checkpoint_folder, checkpoint_name, map_location=None):
    """Returns the state `save` wrote for this rank.  `state` is accepted for the
    reference's call shape; a dict passed in is updated in place and returned."""
    assert os.path.isdir(checkpoint_folder), f"folder {checkpoint_folder} does not exist"
    loaded = torch.load(_checkpoint_file(checkpoint_folder, checkpoint_name),
                        map_location=map_location, weights_only=True)
    if isinstance(state, dict) and isinstance(loaded, dict):
        state.update(loaded)
        return state
    return loaded
