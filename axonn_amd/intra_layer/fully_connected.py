"""Tensor-parallel Linear layer on a one-GPU grid, with the reference's interface
(axonn/intra_layer/fully_connected.py) and its arithmetic in gfx950 kernels.

What is kept from the reference: the constructor and `forward` signatures, the
flat 1-D `weight` parameter (row-major [out, in], :263), the parameter tags the
gradient-sync and clipping code reads (:268-295), zero-initialised bias (:276-281),
`kaiming_uniform_(a=sqrt 5)` default init (:91-93), the state-dict loader that
accepts a full 2-D or a sharded 1-D weight (:350-400), the `AsyncLinear`
autograd function and its argument list (:96-108), autocast behaviour
(:32-54), and `skip_bias_add` (:345-346).

What differs: `Y = X W^T`, `dX = dY W` and `dW = dY^T X` (:118, :140, :147-151)
run as bf16 or fp16 MFMA kernels (fp32 kernels for fp32 layers); the bias add (:348)
and, on request, the GELU that callers place after the layer are fused into the
forward kernel's epilogue; with `optimize_communication(overlap_reduce_scatter=
True)` the weight gradient is accumulated into `weight.grad` by the wgrad kernel
itself instead of by a later pass (overlap_communication.py:38-47).
"""

import math
from typing import Optional, Sequence

import torch
from torch.autograd import Function

from .. import axonn as ax
from .. import ops
from ..axonn import get_world_size
from . import overlap_communication
from .communication import Drop, Gather, _gather, _reduce_scatter


def _flat_shard(full, outer_group, inner_group, depth_group):
    """This rank's part of a full [out_features, in_features] matrix as the flat vector
    the parameter holds: input columns of `inner_group`'s slice, output rows of
    `outer_group`'s, row-major, and of that vector the slice of `depth_group`
    (axonn/intra_layer/fully_connected.py:62-70 fixes this order; it is the checkpoint
    format).  On one GPU: the matrix, flattened."""
    with torch.no_grad():
        part = Drop.apply(full, inner_group)
        part = Drop.apply(part.t().contiguous(), outer_group).t().contiguous()
        return Drop.apply(part.reshape(-1), depth_group)


def default_init_method(weight):
    """torch.nn.Linear's own default, U(-1/sqrt(in), 1/sqrt(in)) (:91-93)."""
    with torch.no_grad():
        return torch.nn.init.kaiming_uniform_(weight, a=math.sqrt(5))


def _compute_dtype(*tensors):
    """dtype the kernels run in: the autocast dtype inside an autocast region
    (where the reference's matmul would be cast, :118), else the operands' own."""
    if torch.is_autocast_enabled("cuda"):
        return torch.get_autocast_dtype("cuda")
    dt = tensors[0].dtype
    for t in tensors[1:]:
        if t.dtype != dt:
            raise TypeError("operand dtypes differ: %s vs %s" % (dt, t.dtype))
    return dt


def _backward_products(grad_2d, w, input_2d, original_weight, need_input, need_weight):
    """dX = dY W and dW = dY^T X as AsyncLinear.backward needs them (:140, :147-151).  dW
    comes in the parameter's dtype, flat, either returned to autograd or - under
    overlap_reduce_scatter - accumulated straight into weight.grad.  When both are asked
    for they go through one entry point (ops.gemm_bwd).  Returns (dX, dW for autograd)."""
    if not need_weight:
        return (ops.gemm_dgrad(grad_2d, w) if need_input else None), None
    out_dtype = original_weight.dtype
    if out_dtype not in (torch.float32, grad_2d.dtype):
        out_dtype = grad_2d.dtype  # the kernels write dW in the operands' type or in fp32

    def products(**kw):
        if need_input:
            return ops.gemm_bwd(grad_2d, w, input_2d, **kw)
        return None, ops.gemm_wgrad(grad_2d, input_2d, **kw)

    if overlap_communication.OVERLAP_REDUCE_SCATTER:
        grad = original_weight.grad
        # the kernel writes 16-byte vectors: a gradient that is a view at an odd offset
        # of a flat buffer (axonn/utils.py:11-30 packs without padding) takes the later add
        fusable = (
            grad is not None and grad.is_contiguous() and grad.dtype == out_dtype
            and grad.numel() == original_weight.numel() and grad.data_ptr() % 16 == 0
        )
        if fusable:
            dx, _ = products(out=grad, accumulate=True)
        elif grad is None and out_dtype == original_weight.dtype:
            dx, dw = products(out_dtype=out_dtype)
            original_weight.grad = dw.reshape(original_weight.shape)
        else:
            dx, dw = products(out_dtype=out_dtype)
            overlap_communication.accumulate_later(original_weight, dw.reshape(-1))
        return dx, None
    dx, dw = products(out_dtype=out_dtype)
    return dx, _reduce_scatter(dw.reshape(-1), dim=0, process_group=None, overlap_comm=False)


def _weight_grad(grad_2d, input_2d, original_weight):
    """The weight gradient alone (callers that compute the input gradient by other means)."""
    return _backward_products(grad_2d, None, input_2d, original_weight, False, True)[1]


class AsyncLinear(Function):
    """Same call signature as the reference's AsyncLinear (:96-108)."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, input_, weight, forward_all_reduce_group, backward_all_reduce_group,
                depth_parallel_group, local_weight_shape, cache_weights):
        original_weight = weight
        weight = _gather(weight, dim=0, process_group=depth_parallel_group, cache=cache_weights)
        weight = weight.reshape(local_weight_shape)
        dt = _compute_dtype(input_, weight)
        x = input_.reshape(-1, input_.shape[-1]).to(dt)
        w = weight.to(dt)
        # A weight cast for this step (fp32 parameter under autocast) is kept for the
        # backward pass, as torch's autocast keeps its casts of parameters: one cast per
        # step, not one in forward and one more in backward.
        ctx.save_for_backward(x, original_weight, w if w.dtype != weight.dtype else None)
        ctx.backward_all_reduce_group = backward_all_reduce_group
        ctx.depth_parallel_group = depth_parallel_group
        ctx.shape = local_weight_shape
        ctx.input_shape = input_.shape
        ctx.compute_dtype = dt
        get_world_size(forward_all_reduce_group)  # one rank: the all-reduce is the identity
        output, _ = ops.gemm_fwd(x, w)
        return output.reshape(*input_.shape[:-1], local_weight_shape[0])

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        x, original_weight, w_cast = ctx.saved_tensors
        weight = _gather(original_weight, dim=0, process_group=ctx.depth_parallel_group,
                         cache=False)
        weight = weight.reshape(ctx.shape)
        dt = ctx.compute_dtype
        w = w_cast if w_cast is not None else weight.to(dt)
        g = grad_output.reshape(-1, grad_output.shape[-1]).to(dt)
        get_world_size(ctx.backward_all_reduce_group)
        grad_input, grad_weight = _backward_products(g, w, x, original_weight,
                                                     ctx.needs_input_grad[0], ctx.needs_input_grad[1])
        if grad_input is not None:
            grad_input = grad_input.reshape(ctx.input_shape)
        return grad_input, grad_weight, None, None, None, None, None


class FusedLinear(Function):
    """act(X W^T + b) with the bias add and the activation in the GEMM epilogue.
    The reference computes `x + bias` as a separate pass (:348) and leaves the
    activation to the caller; the backward here is what autograd would derive
    for that composition."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, input_, weight, bias, local_weight_shape, activation):
        original_weight = weight
        weight = weight.reshape(local_weight_shape)
        dt = _compute_dtype(input_, weight)
        x = input_.reshape(-1, input_.shape[-1]).to(dt)
        needs_grad = any(ctx.needs_input_grad[:3])
        w = weight.to(dt)
        # An fp32 bias on a 16-bit product (fp32 parameters under autocast) makes the
        # reference's `x + bias` an fp32 tensor by type promotion (:348): so it is here.
        out_f32 = bias is not None and bias.dtype == torch.float32 and dt != torch.float32
        output, z = ops.gemm_fwd(x, w, bias=bias, activation=activation, save_z=needs_grad,
                                 out_f32=out_f32)
        # the step's cast of an fp32 weight is kept for the backward pass (see AsyncLinear)
        ctx.save_for_backward(x, original_weight, z, w if w.dtype != weight.dtype else None)
        ctx.shape = local_weight_shape
        ctx.input_shape = input_.shape
        ctx.compute_dtype = dt
        ctx.has_bias = bias is not None
        return output.reshape(*input_.shape[:-1], local_weight_shape[0])

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        x, original_weight, z, w_cast = ctx.saved_tensors
        weight = original_weight.reshape(ctx.shape)
        dt = ctx.compute_dtype
        w = w_cast if w_cast is not None else weight.to(dt)
        g = grad_output.reshape(-1, grad_output.shape[-1]).to(dt)
        want_dbias = ctx.has_bias and ctx.needs_input_grad[2]
        grad_bias = None
        if z is not None or want_dbias:
            g, grad_bias = ops.dgelu_dbias(g, z, want_dbias=want_dbias)
        grad_input, grad_weight = _backward_products(g, w, x, original_weight,
                                                     ctx.needs_input_grad[0], ctx.needs_input_grad[1])
        if grad_input is not None:
            grad_input = grad_input.reshape(ctx.input_shape)
        return grad_input, grad_weight, grad_bias, None, None


class Linear(torch.nn.Module):
    """The reference's Linear (:190-301): `weight` is the flat shard of the row-major
    [out_features, in_features] matrix, `bias` this rank's output rows."""

    def __init__(
        self,
        in_features,
        out_features,
        *args,
        transpose=False,
        bias=True,
        skip_bias_add=False,
        init_method=None,
        expert_mode=False,
        tensor_parallel_dims: Optional[Sequence[int]] = None,
        fused_activation: Optional[str] = None,
        **kwargs,
    ):
        """Arguments as the reference's Linear (:191-203).  `fused_activation`
        (None or "gelu") is new: the exact-erf GELU applied in the forward
        kernel's epilogue, equal to `torch.nn.GELU()(layer(x))`."""
        super().__init__()
        if fused_activation not in (None, "gelu"):
            raise ValueError("fused_activation must be None or 'gelu', got %r" % (fused_activation,))
        handle = ax._handle()
        inner, outer, _ = handle.get_intra_layer_groups(tensor_parallel_dims)
        # input columns are split over the inner group and output rows over the outer one;
        # `transpose` swaps the roles (:218-219)
        self.inner_group, self.outer_group = (outer, inner) if transpose else (inner, outer)
        self.depth_group = handle.depth_intra_layer_parallel_group
        self.inner_group_size, self.outer_group_size, self.depth_group_size = (
            get_world_size(g) for g in (self.inner_group, self.outer_group, self.depth_group))
        assert in_features % self.inner_group_size == 0
        assert out_features % self.outer_group_size == 0

        self.in_features, self.out_features = in_features, out_features
        self.local_in_features = in_features // self.inner_group_size
        self.local_out_features = out_features // self.outer_group_size
        self.expert_mode, self.skip_bias_add = expert_mode, skip_bias_add
        self.fused_activation = fused_activation

        # Drawn as the full matrix on the device (as the reference does, :73-88), then cut.
        device = "cuda" if torch.cuda.is_available() else "cpu"
        full = torch.empty((out_features, in_features), device=device)
        (init_method or default_init_method)(full)
        shard = _flat_shard(full, self.outer_group, self.inner_group, self.depth_group).cpu()
        self.weight = torch.nn.Parameter(shard)
        # read by gradient sync and clipping (:268-295)
        self.weight.is_tensor_parallel = True
        self.weight.needs_depth_parallel_gradient_sync = False
        self.weight.process_group_for_norm_reduction = handle.intra_layer_group
        self.bias = None
        if bias:
            self.bias = torch.nn.Parameter(torch.zeros(self.local_out_features))
            self.bias.is_tensor_parallel = True
            self.bias.needs_depth_parallel_gradient_sync = True
            self.bias.process_group_for_norm_reduction = (
                handle.inner_intra_layer_parallel_group if transpose
                else handle.outer_intra_layer_parallel_group)
        # full tensors in a checkpoint are cut to this rank's shards on the way in (:350-400)
        self._register_load_state_dict_pre_hook(self._shard_incoming_state)

    def forward(self, x, cache_weights_in_all_gather=False):
        shape = (self.local_out_features, self.local_in_features)
        add_bias = self.bias is not None and not self.skip_bias_add
        if add_bias or self.fused_activation is not None:
            # bias and activation ride in the forward kernel's epilogue
            b = self.bias if add_bias else None
            if b is not None and not self.expert_mode:
                b = Gather.apply(b, self.outer_group)
            y = FusedLinear.apply(x, self.weight, b, shape, self.fused_activation)
            return (y, self.bias) if (self.bias is not None and self.skip_bias_add) else y
        y = AsyncLinear.apply(x, self.weight, self.inner_group, self.outer_group, self.depth_group,
                              shape, cache_weights_in_all_gather)
        if self.bias is None:
            return y
        # skip_bias_add: the caller adds (or fuses) the bias (:345-346)
        return y, (self.bias if self.expert_mode else Gather.apply(self.bias, self.outer_group))

    def _shard_incoming_state(self, state_dict, prefix, *unused):
        mismatch = "This is neither a full checkpoint nor a sharded checkpoint"
        w = state_dict.get(prefix + "weight")
        if w is not None:
            shard_len = self.local_out_features * self.local_in_features // self.depth_group_size
            if w.dim() == 2 and tuple(w.shape) == (self.out_features, self.in_features):
                state_dict[prefix + "weight"] = _flat_shard(w, self.outer_group, self.inner_group,
                                                            self.depth_group)
            else:
                assert w.dim() == 1 and w.numel() == shard_len, mismatch
        b = state_dict.get(prefix + "bias") if self.bias is not None else None
        if b is not None:
            if b.shape[0] == self.out_features:
                with torch.no_grad():
                    state_dict[prefix + "bias"] = Drop.apply(b, self.outer_group)
            else:
                assert b.shape[0] == self.local_out_features, mismatch
