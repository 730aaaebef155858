"""All-sum-reduce stand-in (reference: backends/mpi_numpy/functional/all_sum_reduce.py:77-92).
A collective, hence outside this build: the workers' tensors are handed over by
the transport and summed in rank order by one launch of the sum kernel."""

__all__ = ["AllSumReduceFunction"]

import torch

from .... import hip_ops


def _sum_over(P, tensor, tag, divisor=1):
    """Sum of ``tensor / divisor`` over the workers of ``P``, in rank order."""
    transport = P._world.transport
    mine = hip_ops.contiguous(tensor)
    parts = transport.gather_list(P, mine, tag=tag)
    out = torch.empty_like(mine)
    if out.numel():
        full = [slice(0, int(n)) for n in mine.shape]
        hip_ops.sum_boxes(parts, full, out, full, divisor)
    transport.release(P, tag=tag)
    return out


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
        return _sum_over(P_reduce, input.detach(), ("all_sum_reduce", tag))

    @staticmethod
    def backward(ctx, grad_output):
        # The all-sum-reduce is its own adjoint (reference :95-161).
        P_reduce = ctx.P_reduce
        grad_output = grad_output.detach()
        # Every worker's gradient is divided before the sum (reference :127-128): the sum kernel divides as it reads.
        divisor = 1 if ctx.scale_backward is None else ctx.scale_backward
        if not P_reduce.active or P_reduce.size == 1:
            return (grad_output if divisor == 1 else hip_ops.scaled(grad_output, divisor)), None, None, None, None
        return _sum_over(P_reduce, grad_output, ("all_sum_reduce_adjoint", ctx.tag), divisor), None, None, None, None
