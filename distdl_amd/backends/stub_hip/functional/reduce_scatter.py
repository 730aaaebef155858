"""Reduce-scatter along one partitioned axis and its adjoint (reference:
backends/mpi_numpy/functional/reduce_scatter.py:86-127, :130-200): every worker
holds a full-length tensor and keeps its balanced slab of the sum.  The adjoint
is the all-gather.  Local work: strided slab reads with accumulating box
copies, resp. one unpack launch of the box kernel; see all_gather.py."""

__all__ = ["ReduceScatterFunction"]

import torch

from .all_gather import gather_slabs
from .all_gather import reduce_scatter_slabs


class ReduceScatterFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, P_reducescatter, axis=None, tag=None):
        if not P_reducescatter.active or P_reducescatter.size == 1:
            ctx.identity = True
            return input
        ctx.identity = False
        ctx.P, ctx.axis, ctx.tag = P_reducescatter, int(axis), tag
        return reduce_scatter_slabs(P_reducescatter, input.detach(), int(axis), ("reduce_scatter", tag))

    @staticmethod
    def backward(ctx, grad_output):
        if ctx.identity:
            return grad_output, None, None, None
        dx = gather_slabs(ctx.P, grad_output.detach(), ctx.axis, ("reduce_scatter_adjoint", ctx.tag))
        return dx, None, None, None
