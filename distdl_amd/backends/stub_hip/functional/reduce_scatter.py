"""Reduce-scatter along one partitioned axis and its adjoint (reference:
backends/mpi_numpy/functional/reduce_scatter.py:86-127, :130-200): every worker
holds a full-length tensor and keeps its balanced slab of the sum.  The adjoint
is the all-gather.  Local work: one launch of the sum kernel over the P slabs,
resp. one unpack launch of the box kernel; see all_gather.py."""

__all__ = ["ReduceScatterFunction"]

import torch

from .all_gather import gather_slabs
from .all_gather import reduce_scatter_slabs
from .all_gather import single_axis


class ReduceScatterFunction(torch.autograd.Function):
    """Positional arguments as in the reference
    (backends/mpi_numpy/functional/reduce_scatter.py:35-37); the tensor
    structures are accepted and not needed."""

    @staticmethod
    def forward(ctx, input, P_reducescatter, input_tensor_structure, output_tensor_structure, axes):
        if not P_reducescatter.active or P_reducescatter.size == 1:
            ctx.identity = True
            return input
        ctx.identity = False
        ctx.P, ctx.axis = P_reducescatter, single_axis(axes, "ReduceScatter")
        return reduce_scatter_slabs(P_reducescatter, input.detach(), ctx.axis, ("reduce_scatter", None))

    @staticmethod
    def backward(ctx, grad_output):
        if ctx.identity:
            return grad_output, None, None, None, None
        dx = gather_slabs(ctx.P, grad_output.detach(), ctx.axis, ("reduce_scatter_adjoint", None))
        return dx, None, None, None, None
