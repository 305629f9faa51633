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


def divide(a, b):
    assert a % b == 0
    return a // b


@torch.no_grad()
def extract_local_params_from_full_params(params, out_features_group, in_features_group,
                                          depth_group):
    """[num_embeddings, embedding_dim] -> this rank's flat shard (columns first)."""
    params = Drop.apply(params, out_features_group)
    params = Drop.apply(torch.t(params).contiguous(), in_features_group)
    params = torch.t(params).contiguous()
    return Drop.apply(params.reshape(-1), depth_group)


@torch.no_grad()
def initialize_params(out_features, in_features, out_features_group, in_features_group,
                      depth_group, init_method, init_device=None):
    if init_device is None:
        init_device = "cuda" if torch.cuda.is_available() else "cpu"
    params = torch.empty((in_features, out_features), device=init_device)
    init_method(params)
    return extract_local_params_from_full_params(
        params, out_features_group, in_features_group, depth_group
    ).cpu()


@torch.no_grad()
def default_init_method(weight, padding_idx=None):
    return torch.nn.init.normal_(weight)


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
        super(Embedding, self).__init__()
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        if padding_idx is not None:
            if padding_idx > 0:
                assert padding_idx < num_embeddings, "Padding_idx must be within num_embeddings"
            elif padding_idx < 0:
                assert padding_idx >= -num_embeddings, "Padding_idx must be within num_embeddings"
                padding_idx = num_embeddings + padding_idx
        self.padding_idx = padding_idx
        self.max_norm = max_norm
        self.norm_type = norm_type
        self.scale_grad_by_freq = scale_grad_by_freq
        self.sparse = sparse

        handle = ax._handle()
        self.inner_group = handle.inner_intra_layer_parallel_group
        self.outer_group = handle.outer_intra_layer_parallel_group
        self.depth_group = handle.depth_intra_layer_parallel_group
        self.inner_group_size = get_world_size(self.inner_group)
        self.outer_group_size = get_world_size(self.outer_group)
        self.depth_group_size = get_world_size(self.depth_group)

        self.out_features = embedding_dim
        self.in_features = num_embeddings
        if init_method is None:
            init_method = default_init_method

        # The embedding width is split over one of the two tensor-parallel groups; the
        # vocabulary is never split.
        if not transpose:
            assert self.inner_group_size == 1
            self._column_group, self._row_group = self.outer_group, self.inner_group
        else:
            assert self.outer_group_size == 1
            self._column_group, self._row_group = self.inner_group, self.outer_group
        columns = get_world_size(self._column_group)
        assert embedding_dim % columns == 0
        self.local_in_features = num_embeddings
        self.local_out_features = divide(embedding_dim, columns)
        initial_params = initialize_params(
            self.out_features, self.in_features, self._column_group, self._row_group,
            self.depth_group, init_method,
        )
        if self.padding_idx is not None:
            # The shard is row-major, so a row of the table is a run of the flat vector;
            # this rank zeroes the part of it that falls into its depth slice.  (The
            # reference indexes the 1-D parameter with the row number, :136-137, which
            # zeroes a single element; the whole row is what torch.nn.Embedding gives.)
            n = initial_params.numel()
            lo = (self.padding_idx * self.local_out_features
                  - handle.intra_layer_depth_parallel_rank * n)
            hi = lo + self.local_out_features
            initial_params[max(lo, 0):max(min(hi, n), 0)].fill_(0)

        self.weight = torch.nn.Parameter(initial_params, requires_grad=not _freeze)
        setattr(self.weight, "is_tensor_parallel", True)
        setattr(self.weight, "needs_depth_parallel_gradient_sync", False)
        setattr(self.weight, "process_group_for_norm_reduction", handle.intra_layer_group)

        self.expert_mode = expert_mode
        self.transpose = transpose
        self._old_load_from_state_dict = self._load_from_state_dict
        self._load_from_state_dict = self._modified_load_from_state_dict

    def get_output_feature_size(self):
        return self.local_out_features

    def forward(self, x):
        weight = ForwardGather_BackwardReduceScatter.apply(self.weight, self.depth_group).reshape(
            self.local_in_features, self.local_out_features
        )
        x = embedding(x, weight, self.padding_idx, self.max_norm, self.norm_type,
                      self.scale_grad_by_freq, self.sparse)
        if not self.expert_mode:
            x = Gather.apply(x, self._column_group)
        return x

    def _is_full_weight_matrix(self, weight):
        return (
            weight.ndim == 2
            and weight.size(0) == self.in_features
            and weight.size(1) == self.out_features
        )

    def _is_sharded_weight_matrix(self, weight):
        return weight.ndim == 1 and weight.size(0) == divide(
            self.local_out_features * self.local_in_features, self.depth_group_size
        )

    @torch.no_grad()
    def _modified_load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        weight = state_dict.get(prefix + "weight")
        if weight is not None:
            full = self._is_full_weight_matrix(weight)
            sharded = self._is_sharded_weight_matrix(weight)
            assert full or sharded, "This is neither a full checkpoint nor a sharded checkpoint"
            if full:
                weight = extract_local_params_from_full_params(
                    weight, self._column_group, self._row_group, self.depth_group
                )
            state_dict[prefix + "weight"] = weight
        self._old_load_from_state_dict(state_dict, prefix, *args, **kwargs)
