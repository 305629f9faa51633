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


def divide(a, b):
    assert a % b == 0
    return a // b


@torch.no_grad()
def extract_local_params_from_full_params(params, out_features_group, in_features_group,
                                          depth_group):
    params = Drop.apply(params, in_features_group)
    params = Drop.apply(torch.t(params).contiguous(), out_features_group)
    params = torch.t(params).contiguous()
    params = Drop.apply(params.reshape(-1), depth_group)  # 1-D view
    return params


@torch.no_grad()
def initialize_params(out_features, in_features, out_features_group, in_features_group,
                      depth_group, init_method, init_device=None):
    if init_device is None:
        init_device = "cuda" if torch.cuda.is_available() else "cpu"
    params = torch.empty((out_features, in_features), device=init_device)
    init_method(params)
    params = extract_local_params_from_full_params(
        params, out_features_group, in_features_group, depth_group
    ).cpu()
    return params


@torch.no_grad()
def default_init_method(weight):
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


def _weight_grad(grad_2d, input_2d, original_weight):
    """dW = dY^T X in the parameter's dtype, flat, either returned to autograd or
    - under overlap_reduce_scatter - accumulated straight into weight.grad."""
    out_dtype = original_weight.dtype
    if out_dtype not in (torch.float32, grad_2d.dtype):
        out_dtype = grad_2d.dtype  # the kernels write dW in the operands' type or in fp32
    if overlap_communication.OVERLAP_REDUCE_SCATTER:
        grad = original_weight.grad
        fusable = (
            grad is not None and grad.is_contiguous() and grad.dtype == out_dtype
            and grad.numel() == original_weight.numel()
        )
        if fusable:
            ops.gemm_wgrad(grad_2d, input_2d, out=grad, accumulate=True)
        elif grad is None and out_dtype == original_weight.dtype:
            original_weight.grad = ops.gemm_wgrad(
                grad_2d, input_2d, out_dtype=out_dtype
            ).reshape(original_weight.shape)
        else:
            dw = ops.gemm_wgrad(grad_2d, input_2d, out_dtype=out_dtype).reshape(-1)
            overlap_communication.accumulate_later(original_weight, dw)
        return None
    dw = ops.gemm_wgrad(grad_2d, input_2d, out_dtype=out_dtype).reshape(-1)
    return _reduce_scatter(dw, dim=0, process_group=None, overlap_comm=False)


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
        ctx.save_for_backward(x, original_weight)
        ctx.backward_all_reduce_group = backward_all_reduce_group
        ctx.depth_parallel_group = depth_parallel_group
        ctx.shape = local_weight_shape
        ctx.input_shape = input_.shape
        ctx.compute_dtype = dt
        get_world_size(forward_all_reduce_group)  # one rank: the all-reduce is the identity
        output, _ = ops.gemm_fwd(x, weight.to(dt))
        return output.reshape(*input_.shape[:-1], local_weight_shape[0])

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        x, original_weight = ctx.saved_tensors
        weight = _gather(original_weight, dim=0, process_group=ctx.depth_parallel_group,
                         cache=False)
        weight = weight.reshape(ctx.shape)
        dt = ctx.compute_dtype
        g = grad_output.reshape(-1, grad_output.shape[-1]).to(dt)
        grad_input, grad_weight = None, None
        get_world_size(ctx.backward_all_reduce_group)
        if ctx.needs_input_grad[0]:
            grad_input = ops.gemm_dgrad(g, weight.to(dt)).reshape(ctx.input_shape)
        if ctx.needs_input_grad[1]:
            grad_weight = _weight_grad(g, x, original_weight)
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
        output, z = ops.gemm_fwd(x, weight.to(dt), bias=bias, activation=activation,
                                 save_z=needs_grad)
        ctx.save_for_backward(x, original_weight, z)
        ctx.shape = local_weight_shape
        ctx.input_shape = input_.shape
        ctx.compute_dtype = dt
        ctx.has_bias = bias is not None
        return output.reshape(*input_.shape[:-1], local_weight_shape[0])

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        x, original_weight, z = ctx.saved_tensors
        weight = original_weight.reshape(ctx.shape)
        dt = ctx.compute_dtype
        g = grad_output.reshape(-1, grad_output.shape[-1]).to(dt)
        want_dbias = ctx.has_bias and ctx.needs_input_grad[2]
        grad_bias = None
        if z is not None or want_dbias:
            g, grad_bias = ops.dgelu_dbias(g, z, want_dbias=want_dbias)
        grad_input, grad_weight = None, None
        if ctx.needs_input_grad[0]:
            grad_input = ops.gemm_dgrad(g, weight.to(dt)).reshape(ctx.input_shape)
        if ctx.needs_input_grad[1]:
            grad_weight = _weight_grad(g, x, original_weight)
        return grad_input, grad_weight, grad_bias, None, None


class Linear(torch.nn.Module):
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
        super(Linear, self).__init__()
        handle = ax._handle()
        self.inner_group, self.outer_group, self.depth_group = handle.get_intra_layer_groups(
            tensor_parallel_dims
        )
        if transpose:
            self.inner_group, self.outer_group = self.outer_group, self.inner_group
        self.depth_group = handle.depth_intra_layer_parallel_group

        self.inner_group_size = get_world_size(self.inner_group)
        self.outer_group_size = get_world_size(self.outer_group)
        self.depth_group_size = get_world_size(self.depth_group)

        self.in_features = in_features
        self.out_features = out_features
        self.expert_mode = expert_mode
        if fused_activation not in (None, "gelu"):
            raise ValueError("fused_activation must be None or 'gelu', got %r" % (fused_activation,))
        self.fused_activation = fused_activation

        if init_method is None:
            init_method = default_init_method

        assert in_features % self.inner_group_size == 0
        assert out_features % self.outer_group_size == 0
        self.local_in_features = divide(in_features, self.inner_group_size)
        self.local_out_features = divide(out_features, self.outer_group_size)

        initial_params = initialize_params(
            out_features, in_features, self.outer_group, self.inner_group, self.depth_group,
            init_method,
        )
        self.weight = torch.nn.Parameter(initial_params, requires_grad=True)
        setattr(self.weight, "is_tensor_parallel", True)
        setattr(self.weight, "needs_depth_parallel_gradient_sync", False)
        setattr(self.weight, "process_group_for_norm_reduction", handle.intra_layer_group)

        if bias:
            self.bias = torch.nn.Parameter(torch.zeros(self.local_out_features))
            setattr(self.bias, "is_tensor_parallel", True)
            setattr(self.bias, "needs_depth_parallel_gradient_sync", True)
            if not transpose:
                setattr(self.bias, "process_group_for_norm_reduction",
                        handle.outer_intra_layer_parallel_group)
            else:
                setattr(self.bias, "process_group_for_norm_reduction",
                        handle.inner_intra_layer_parallel_group)
        else:
            self.bias = None

        self.skip_bias_add = skip_bias_add
        self._old_load_from_state_dict = self._load_from_state_dict
        self._load_from_state_dict = self._modified_load_from_state_dict

    def forward(self, x, cache_weights_in_all_gather=False):
        weight = self.weight
        shape = (self.local_out_features, self.local_in_features)
        fuse_bias = self.bias is not None and not self.skip_bias_add
        if fuse_bias or self.fused_activation is not None:
            bias = self.bias if fuse_bias else None
            if bias is not None and not self.expert_mode:
                bias = Gather.apply(bias, self.outer_group)
            y = FusedLinear.apply(x, weight, bias, shape, self.fused_activation)
            if self.bias is not None and self.skip_bias_add:
                return y, self.bias
            return y
        y = AsyncLinear.apply(
            x, weight, self.inner_group, self.outer_group, self.depth_group, shape,
            cache_weights_in_all_gather,
        )
        if self.bias is None:
            return y
        bias = self.bias
        if not self.expert_mode:
            bias = Gather.apply(bias, self.outer_group)
        return y, bias  # skip_bias_add

    def _is_full_weight_matrix(self, weight):
        return (
            weight.ndim == 2
            and weight.size(0) == self.out_features
            and weight.size(1) == self.in_features
        )

    def _is_sharded_weight_matrix(self, weight):
        return weight.ndim == 1 and weight.size(0) == divide(
            self.local_out_features * self.local_in_features, self.depth_group_size
        )

    @torch.no_grad()
    def _modified_load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        weight = state_dict[prefix + "weight"] if prefix + "weight" in state_dict else None
        if weight is not None:
            is_full_weight_matrix = self._is_full_weight_matrix(weight)
            is_sharded_weight_matrix = self._is_sharded_weight_matrix(weight)
            assert (
                is_full_weight_matrix or is_sharded_weight_matrix
            ), "This is neither a full checkpoint nor a sharded checkpoint"
            if is_full_weight_matrix:
                weight = extract_local_params_from_full_params(
                    weight, self.outer_group, self.inner_group, self.depth_group
                )
            state_dict[prefix + "weight"] = weight

        if self.bias is not None:
            bias = state_dict[prefix + "bias"] if prefix + "bias" in state_dict else None
            if bias is not None:
                if bias.size(0) == self.out_features:
                    bias = Drop.apply(bias, self.outer_group)
                    state_dict[prefix + "bias"] = bias
                else:
                    assert (
                        bias.size(0) == self.local_out_features
                    ), "This is neither a full checkpoint nor a sharded checkpoint"

        self._old_load_from_state_dict(state_dict, prefix, *args, **kwargs)
