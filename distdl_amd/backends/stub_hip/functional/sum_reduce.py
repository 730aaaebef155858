"""Sum-reduce stand-in (reference: backends/mpi_numpy/functional/sum_reduce.py:13-122,
:125-206).  The reduction is the adjoint of the broadcast and is delegated to
the transport the same way: the partial tensors of the workers of ``P_send``
are added, in rank order, onto the worker of ``P_recv`` they would receive a
broadcast from; the adjoint hands that worker's gradient back to every one of
them.  Workers outside the receiving partition get the reference's zero-volume
tensor."""

__all__ = ["SumReduceFunction"]

import torch

from ....utilities.torch import zero_volume_tensor
from .broadcast import route_of


def _world_of(P_send, P_recv):
    return P_send._world if P_send._world is not None else P_recv._world


class SumReduceFunction(torch.autograd.Function):
    """Positional arguments as in the reference (:32-34).  ``P_send`` and
    ``P_recv`` come from ``P_x.create_reduction_partition_to(P_y, ...)``; the
    tensor structures are accepted and not needed."""

    @staticmethod
    def forward(ctx, input, P_send, P_recv, preserve_batch, input_tensor_structure, output_tensor_structure):
        if not (P_send.active or P_recv.active):
            return input
        route = route_of(P_send, P_recv, "reduction")
        P_send, P_recv, tag = route.P_src, route.P_dest, None
        transpose_src, transpose_dest = route.transpose_src, route.transpose_dest
        ctx.P_send, ctx.P_recv, ctx.tag = P_send, P_recv, tag
        ctx.transposes = (transpose_src, transpose_dest)
        ctx.input_like = (tuple(input.shape), input.dtype, input.device)
        # The receiving partition is the smaller one, the "source" of the
        # broadcast this reduction is the adjoint of.
        out = _world_of(P_send, P_recv).transport.broadcast_adjoint(
            P_recv, P_send, input.detach(), transpose_src=transpose_dest, transpose_dst=transpose_src,
            tag=("sum-reduce", tag))
        if out is None:
            batch = int(input.shape[0]) if (preserve_batch and input.dim() > 0) else None
            out = zero_volume_tensor(batch, dtype=input.dtype, device=input.device)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        P_send, P_recv = ctx.P_send, ctx.P_recv
        transpose_src, transpose_dest = ctx.transposes
        shape, dtype, device = ctx.input_like
        grad = _world_of(P_send, P_recv).transport.broadcast(
            P_recv, P_send, grad_output.detach(), transpose_src=transpose_dest, transpose_dst=transpose_src,
            tag=("sum-reduce-adjoint", ctx.tag))
        if not P_send.active:
            grad = torch.zeros(shape, dtype=dtype, device=device)
        return grad, None, None, None, None, None
