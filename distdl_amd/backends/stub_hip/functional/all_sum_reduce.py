"""All-sum-reduce stand-in (reference: backends/mpi_numpy/functional/all_sum_reduce.py:77-92).
A collective, hence outside this build: contributions are gathered through the
transport and summed in rank order."""

__all__ = ["AllSumReduceFunction"]

import torch


class AllSumReduceFunction(torch.autograd.Function):
    """Positional arguments as in the reference (:32-33); the tensor structures
    are accepted and not needed."""

    @staticmethod
    def forward(ctx, input, P_allreduce, input_tensor_structure, output_tensor_structure, scale_backward):
        P_reduce = P_allreduce
        ctx.P_reduce, ctx.tag, ctx.scale_backward = P_reduce, None, scale_backward
        tag = None
        if not P_reduce.active or P_reduce.size == 1:
            return input
        parts = P_reduce._world.transport.allgather(P_reduce, input.detach(), tag=tag)
        return parts.sum(dim=0)

    @staticmethod
    def backward(ctx, grad_output):
        # The all-sum-reduce is its own adjoint (reference :95-161).
        P_reduce = ctx.P_reduce
        grad_output = grad_output.detach()
        if ctx.scale_backward is not None:
            grad_output = grad_output / ctx.scale_backward      # before the sum (reference :127-128)
        if not P_reduce.active or P_reduce.size == 1:
            return grad_output, None, None, None, None
        parts = P_reduce._world.transport.allgather(P_reduce, grad_output.contiguous(), tag=("adjoint", ctx.tag))
        return parts.sum(dim=0), None, None, None, None
