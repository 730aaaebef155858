"""Broadcast stand-in.  The reference's broadcast and its sum-reduce adjoint
(backends/mpi_numpy/functional/broadcast.py:116-128, :213-221) are collectives
and therefore outside this build; both directions are delegated to the
transport (identity for a solo rank that owns the data; copies between rank
threads, summed with the box kernel, under loopback) so that layers storing
weights on a sub-grid work end to end, gradients included."""

__all__ = ["BroadcastFunction", "route_of"]

import torch

from .... import hip_ops
from ....utilities.torch import zero_volume_tensor


def route_of(P_send, P_recv, kind):
    """The two Cartesian partitions and transposes behind a (P_send, P_recv)
    pair made by ``create_broadcast_partition_to`` / ``create_reduction_partition_to``."""
    route = getattr(P_send, "_route", None) or getattr(P_recv, "_route", None)
    if route is None or route.kind != kind:
        raise ValueError(f"P_send / P_recv were not made by this backend's create_{kind}_partition_to")
    return route


class BroadcastFunction(torch.autograd.Function):
    """Positional arguments as in the reference (:32-34).  ``P_send`` and
    ``P_recv`` come from ``P_x.create_broadcast_partition_to(P_y, ...)`` and carry
    the partitions and transposes the transport needs; the tensor structures
    are accepted and not needed."""

    @staticmethod
    def forward(ctx, input, P_send, P_recv, preserve_batch, input_tensor_structure, output_tensor_structure,
                scale_backward):
        if not (P_send.active or P_recv.active):
            return input
        route = route_of(P_send, P_recv, "broadcast")
        P_send, P_recv, tag = route.P_src, route.P_dest, None
        transpose_src, transpose_dest = route.transpose_src, route.transpose_dest
        ctx.P_send, ctx.P_recv, ctx.tag = P_send, P_recv, tag
        ctx.transposes = (transpose_src, transpose_dest)
        ctx.scale_backward = scale_backward
        ctx.input_like = (tuple(input.shape), input.dtype, input.device)
        world = P_send._world if P_send._world is not None else P_recv._world
        out = world.transport.broadcast(P_send, P_recv, input.detach(), transpose_src=transpose_src,
                                        transpose_dst=transpose_dest, tag=tag)
        if not P_recv.active:
            # A worker that only sends holds nothing afterwards (reference :50-54, :116-128).
            batch = int(input.shape[0]) if (preserve_batch and input.dim() > 0) else None
            out = zero_volume_tensor(batch, dtype=input.dtype, device=input.device)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        P_send, P_recv = ctx.P_send, ctx.P_recv
        world = P_send._world if P_send._world is not None else P_recv._world
        transpose_src, transpose_dest = ctx.transposes
        grad_output = grad_output.detach()
        if ctx.scale_backward is not None and P_recv.active:
            # Every receiver's gradient is divided before the sum (reference :208-209).
            grad_output = hip_ops.scaled(grad_output, ctx.scale_backward)
        grad = world.transport.broadcast_adjoint(P_send, P_recv, grad_output, transpose_src=transpose_src,
                                                 transpose_dst=transpose_dest, tag=ctx.tag)
        if grad is None:
            shape, dtype, device = ctx.input_like
            grad = torch.zeros(shape, dtype=dtype, device=device)
        return grad, None, None, None, None, None, None
