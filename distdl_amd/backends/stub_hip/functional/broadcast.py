"""Broadcast stand-in.  The reference's broadcast (and its sum-reduce adjoint,
backends/mpi_numpy/functional/broadcast.py:116-128, :213-221) is a collective
and therefore outside this build; the forward is delegated to the transport
(identity for a solo rank that owns the data, a copy from the owning rank thread
under loopback) so that layers storing weights on a sub-grid work end to end."""

__all__ = ["BroadcastFunction"]

import torch


class BroadcastFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, P_send, P_recv, preserve_batch=False, tag=None):
        if not (P_send.active or P_recv.active):
            return input
        world = P_send._world if P_send._world is not None else P_recv._world
        return world.transport.broadcast(P_send, P_recv, input.detach(), tag=tag)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("the adjoint of Broadcast is a sum-reduce collective, not part of this build")
