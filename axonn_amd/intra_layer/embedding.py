"""Tensor-parallel Embedding on a one-GPU grid, with the reference's interface
(axonn/intra_layer/embedding.py) and its arithmetic in gfx950 kernels.

What is kept from the reference: the constructor signature with torch.nn.Embedding's
arguments first (:57-74), the checks on padding_idx (:78-88), the flat 1-D `weight`
parameter holding the [num_embeddings, embedding_dim / G] shard row-major (:24-32,
:139), normal(0, 1) default init (:52-54), the zeroed padding row (:136-137), the
parameter tags read by gradient sync and clipping (:141-148), the state-dict loader
that accepts a full 2-D or a sharded 1-D weight (:191-222), and the data flow of
`forward` (:155-177): depth all-gather of the weight, lookup, gather of the output
columns unless in expert mode.

What differs: the lookup `F.embedding` (:164-172) and its autograd run as HIP
kernels (a row gather; a sorted, atomics-free dense weight gradient that adds in
token order; the max_norm renormalisation); `sparse=True` is refused, since the
optimizer path here takes dense gradients only.
"""

import torch

from .. import axonn as ax
from .. import ops
from ..axonn import get_world_size
from .communication import Drop, ForwardGather_BackwardReduceScatter, Gather


def _flat_shard(table, column_group, row_group, depth_group):
    """This rank's part of a full [num_embeddings, embedding_dim] table as the flat vector
    the parameter holds: the columns of `column_group`'s slice, every row (`row_group`
    has one member), row-major, and of that vector the slice of `depth_group`
    (axonn/intra_layer/embedding.py:23-32 fixes this order; it is the checkpoint
    format).  On one GPU: the table, flattened."""
    with torch.no_grad():
        part = Drop.apply(table, column_group)
        part = Drop.apply(part.t().contiguous(), row_group).t().contiguous()
        return Drop.apply(part.reshape(-1), depth_group)


def default_init_method(weight, padding_idx=None):
    """normal(0, 1), torch.nn.Embedding's own default (:52-54)."""
    with torch.no_grad():
        return torch.nn.init.normal_(weight)


def _resolve_padding_idx(padding_idx, num_embeddings):
    """torch.nn.Embedding's rule (:78-88): in range, negative values count from the end."""
    if padding_idx is None:
        return None
    assert -num_embeddings <= padding_idx < num_embeddings, "Padding_idx must be within num_embeddings"
    return padding_idx + num_embeddings if padding_idx < 0 else padding_idx


class _Lookup(torch.autograd.Function):
    """weight[ids] and its dense weight gradient on the HIP kernels."""

    @staticmethod
    def forward(ctx, ids, weight, padding_idx, scale_grad_by_freq):
        ctx.save_for_backward(ids)
        ctx.num_embeddings = weight.shape[0]
        ctx.padding_idx = padding_idx
        ctx.scale_grad_by_freq = scale_grad_by_freq
        ctx.weight_dtype = weight.dtype
        return ops.embedding_fwd(ids, weight)

    @staticmethod
    def backward(ctx, grad_output):
        (ids,) = ctx.saved_tensors
        grad_weight = None
        if ctx.needs_input_grad[1]:
            if grad_output.dtype not in (torch.bfloat16, torch.float32):
                grad_output = grad_output.float()
            grad_weight = ops.embedding_bwd(
                ids, grad_output, ctx.num_embeddings, padding_idx=ctx.padding_idx,
                scale_grad_by_freq=ctx.scale_grad_by_freq,
                out_dtype=ctx.weight_dtype if ctx.weight_dtype in (torch.bfloat16, torch.float32)
                else torch.float32,
            )
            if grad_weight.dtype != ctx.weight_dtype:
                grad_weight = grad_weight.to(ctx.weight_dtype)
        return None, grad_weight, None, None


def embedding(ids, weight, padding_idx=None, max_norm=None, norm_type=2.0,
              scale_grad_by_freq=False, sparse=False):
    """F.embedding with the same arguments, on the HIP kernels."""
    if sparse:
        raise NotImplementedError("sparse gradients are not supported: the table's gradient "
                                  "is dense")
    if max_norm is not None:
        ops.embedding_renorm_(weight.detach(), ids, max_norm, norm_type)
    return _Lookup.apply(ids, weight, padding_idx, scale_grad_by_freq)


class Embedding(torch.nn.Module):
    """`torch.nn.Embedding`'s arguments, then the reference's (:57-74).  `weight` is the
    flat shard; `forward` returns [..., embedding_dim] (in expert mode: this rank's
    columns)."""

    def __init__(
        self,
        num_embeddings,
        embedding_dim,
        padding_idx=None,
        max_norm=None,
        norm_type=2.0,
        scale_grad_by_freq=False,
        sparse=False,
        _weight=None,
        _freeze=False,
        *args,
        transpose=False,
        init_method=None,
        expert_mode=False,
        **kwargs,
    ):
        assert _weight is None, "_weight argument is not supported."
        super().__init__()
        handle = ax._handle()
        self.inner_group = handle.inner_intra_layer_parallel_group
        self.outer_group = handle.outer_intra_layer_parallel_group
        self.depth_group = handle.depth_intra_layer_parallel_group
        self.inner_group_size, self.outer_group_size, self.depth_group_size = (
            get_world_size(g) for g in (self.inner_group, self.outer_group, self.depth_group))
        # The embedding width is split over one of the two tensor-parallel groups (the
        # outer one unless `transpose`), the other must be trivial: the vocabulary is
        # never split (:107-134).
        self._column_group, self._row_group = (
            (self.inner_group, self.outer_group) if transpose else (self.outer_group, self.inner_group))
        assert get_world_size(self._row_group) == 1
        columns = get_world_size(self._column_group)
        assert embedding_dim % columns == 0

        self.num_embeddings = self.in_features = self.local_in_features = num_embeddings
        self.embedding_dim = self.out_features = embedding_dim
        self.local_out_features = embedding_dim // columns
        self.padding_idx = _resolve_padding_idx(padding_idx, num_embeddings)
        self.max_norm, self.norm_type = max_norm, norm_type
        self.scale_grad_by_freq, self.sparse = scale_grad_by_freq, sparse
        self.expert_mode, self.transpose = expert_mode, transpose

        # Drawn as the full table on the device (as the reference does, :34-49), then cut.
        device = "cuda" if torch.cuda.is_available() else "cpu"
        table = torch.empty((num_embeddings, embedding_dim), device=device)
        (init_method or default_init_method)(table)
        shard = _flat_shard(table, self._column_group, self._row_group, self.depth_group).cpu()
        if self.padding_idx is not None:
            # The shard is row-major, so a row of the table is a run of the flat vector;
            # this rank zeroes the part of it that falls into its depth slice.  (The
            # reference indexes the 1-D parameter with the row number, :136-137, which
            # zeroes a single element; the whole row is what torch.nn.Embedding gives.)
            first = (self.padding_idx * self.local_out_features
                     - handle.intra_layer_depth_parallel_rank * shard.numel())
            last = first + self.local_out_features
            shard[max(first, 0):max(min(last, shard.numel()), 0)] = 0

        self.weight = torch.nn.Parameter(shard, requires_grad=not _freeze)
        # read by gradient sync and clipping (:141-148)
        self.weight.is_tensor_parallel = True
        self.weight.needs_depth_parallel_gradient_sync = False
        self.weight.process_group_for_norm_reduction = handle.intra_layer_group
        # a full 2-D table in a checkpoint is cut to this rank's shard on the way in (:191-222)
        self._register_load_state_dict_pre_hook(self._shard_incoming_weight)

    def get_output_feature_size(self):
        return self.local_out_features

    def forward(self, x):
        table = ForwardGather_BackwardReduceScatter.apply(self.weight, self.depth_group)
        rows = embedding(x, table.view(self.local_in_features, self.local_out_features), self.padding_idx,
                         self.max_norm, self.norm_type, self.scale_grad_by_freq, self.sparse)
        return rows if self.expert_mode else Gather.apply(rows, self._column_group)

    def _shard_incoming_weight(self, state_dict, prefix, *unused):
        key = prefix + "weight"
        incoming = state_dict.get(key)
        if incoming is None:
            return
        shard_len = self.local_in_features * self.local_out_features // self.depth_group_size
        if incoming.dim() == 2 and tuple(incoming.shape) == (self.in_features, self.out_features):
            state_dict[key] = _flat_shard(incoming, self._column_group, self._row_group, self.depth_group)
        else:
            assert incoming.dim() == 1 and incoming.numel() == shard_len, \
                "This is neither a full checkpoint nor a sharded checkpoint"
