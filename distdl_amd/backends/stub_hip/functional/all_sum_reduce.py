"""All-sum-reduce stand-in (reference: backends/mpi_numpy/functional/all_sum_reduce.py:77-92).
A collective, hence outside this build: contributions are gathered through the
transport and summed in rank order."""

__all__ = ["AllSumReduceFunction"]

import torch


class AllSumReduceFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, P_reduce, tag=None):
        if not P_reduce.active or P_reduce.size == 1:
            return input
        parts = P_reduce._world.transport.allgather(P_reduce, input.detach(), tag=tag)
        return parts.sum(dim=0)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("the adjoint of AllSumReduce is a collective, not part of this build")
