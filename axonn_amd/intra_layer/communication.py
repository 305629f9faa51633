"""Intra-layer communication primitives on a one-rank grid.

Same names and call signatures as axonn/intra_layer/communication.py:11-215.
With one rank per group each of them returns its input, exactly as the
reference's own size-1 short circuits do (:24-25, :37-38, :71-72); a group with
more than one rank is outside what this build covers and raises.
"""

import torch

from ..axonn import get_world_size


def _single(process_group):
    if get_world_size(process_group) != 1:
        raise NotImplementedError("axonn_amd runs on one GPU")


def _all_reduce(input_, process_group=None, overlap_comm=False):
    _single(process_group)
    return input_.contiguous()


def _drop(input_, dim, process_group=None):
    _single(process_group)
    return input_


def _gather(input_, dim, process_group=None, cache=False):
    _single(process_group)
    return input_


def _reduce_scatter(input_, dim, process_group=None, overlap_comm=False):
    assert dim == 0, "reduce scatter only implemented for dim=0"
    _single(process_group)
    return input_


class ForwardAllReduce(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_, process_group=None):
        return _all_reduce(input_, process_group)

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None


class BackwardAllReduce(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_, process_group=None):
        ctx.process_group = process_group
        return input_

    @staticmethod
    def backward(ctx, grad_output):
        return _all_reduce(grad_output, ctx.process_group), None


class Drop(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_, process_group=None, dim=-1):
        ctx.process_group, ctx.dim = process_group, dim
        return _drop(input_, dim=dim, process_group=process_group)

    @staticmethod
    def backward(ctx, grad_output):
        return _gather(grad_output, dim=ctx.dim, process_group=ctx.process_group), None, None


class Gather(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_, process_group=None, dim=-1):
        ctx.process_group, ctx.dim = process_group, dim
        return _gather(input_, dim=dim, process_group=process_group)

    @staticmethod
    def backward(ctx, grad_output):
        return _drop(grad_output, dim=ctx.dim, process_group=ctx.process_group), None, None


class ForwardGather_BackwardReduceScatter(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_, process_group=None, dim=0):
        assert dim == 0
        ctx.process_group, ctx.dim = process_group, dim
        return _gather(input_, dim=dim, process_group=process_group)

    @staticmethod
    def backward(ctx, grad_output):
        return _reduce_scatter(grad_output, dim=ctx.dim, process_group=ctx.process_group), None, None
