"""Runtime bootstrap for the one-GPU grid (axonn/axonn.py:21-67,
axonn/communication.py:21-236).

The reference builds NCCL sub-groups for data / row / column / depth parallelism.
This build covers the per-GPU hot path only, so `init` accepts the reference's
arguments, requires every degree to be 1 and hands the layers process-group
stand-ins of size one, on which every collective of the reference is the identity
(axonn/intra_layer/communication.py:24-25, :37-38, :71-72).
"""

from typing import Optional

from . import config

is_initialized = False
comm_handle = None
enable_timers = False
timers = None


class SingleRankGroup:
    """Stand-in for a torch.distributed process group with one member."""

    def __init__(self, name):
        self.name = name

    def size(self):
        return 1

    def rank(self):
        return 0

    def __repr__(self):
        return "SingleRankGroup(%s)" % self.name


def get_world_size(group=None):
    """torch.distributed.get_world_size for the stand-in groups."""
    if group is None or isinstance(group, SingleRankGroup):
        return 1
    raise NotImplementedError("axonn_amd runs on one GPU; got process group %r" % (group,))


def get_rank(group=None):
    if group is None or isinstance(group, SingleRankGroup):
        return 0
    raise NotImplementedError("axonn_amd runs on one GPU; got process group %r" % (group,))


class communication_handle:
    """The attributes of axonn/communication.py:21-236 that the hot path reads,
    for a 1 x 1 x 1 x 1 grid."""

    def __init__(self, G_inter=1, G_data=1, G_intra_r=1, G_intra_c=1, G_intra_d=1,
                 gpus_per_node=None):
        degrees = dict(G_inter=G_inter, G_data=G_data, G_intra_r=G_intra_r,
                       G_intra_c=G_intra_c, G_intra_d=G_intra_d)
        for name, value in degrees.items():
            if value != 1:
                raise NotImplementedError(
                    "axonn_amd covers the per-GPU hot path on one MI355X: %s must be 1 "
                    "(got %r)" % (name, value)
                )
        self.world_rank = 0
        self.world_size = 1
        self.G_inter, self.G_data = 1, 1
        self.G_intra_r, self.G_intra_c, self.G_intra_d = 1, 1, 1
        self.G_intra = 1
        self.gpus_per_node = 1 if gpus_per_node is None else gpus_per_node
        self.local_rank = 0
        self.inter_layer_parallel_rank = 0
        self.data_parallel_rank = 0
        self.intra_layer_parallel_rank = 0
        self.intra_layer_column_parallel_rank = 0
        self.intra_layer_row_parallel_rank = 0
        self.intra_layer_depth_parallel_rank = 0
        self.coll_nccl_comm = SingleRankGroup("data")
        self.depth_intra_layer_parallel_group = SingleRankGroup("depth")
        self.intra_layer_group = SingleRankGroup("intra")
        self.inner_intra_layer_parallel_group = SingleRankGroup("inner")
        self.outer_intra_layer_parallel_group = SingleRankGroup("outer")

    def get_intra_layer_groups(self, tensor_parallel_dims=None):
        """(inner, outer, depth) groups, axonn/communication.py:166-236."""
        if tensor_parallel_dims is not None and tuple(tensor_parallel_dims) != (1, 1, 1):
            raise NotImplementedError(
                "tensor_parallel_dims must be (1, 1, 1) on one GPU, got %r"
                % (tuple(tensor_parallel_dims),)
            )
        return (
            self.inner_intra_layer_parallel_group,
            self.outer_intra_layer_parallel_group,
            self.depth_intra_layer_parallel_group,
        )


def init(
    G_inter: int = 1,
    G_data: int = 1,
    G_intra_r: int = 1,
    G_intra_c: int = 1,
    G_intra_d: int = 1,
    gpus_per_node: Optional[int] = None,
    enable_internal_timers: bool = False,
) -> None:
    """Same signature as the reference's `init` (axonn/axonn.py:21-29)."""
    global comm_handle, is_initialized, enable_timers
    comm_handle = communication_handle(
        G_inter, G_data, G_intra_r, G_intra_c, G_intra_d, gpus_per_node=gpus_per_node
    )
    config.G_inter = G_inter
    config.G_data = G_data
    config.G_intra = G_intra_r * G_intra_c * G_intra_d
    config.G_intra_r = G_intra_r
    config.G_intra_c = G_intra_c
    config.G_intra_d = G_intra_d
    is_initialized = True
    enable_timers = enable_internal_timers


def _handle():
    """The communication handle, creating the one-GPU grid on first use."""
    if comm_handle is None:
        init()
    return comm_handle
