"""Sum-reduce stand-in (reference: backends/mpi_numpy/functional/sum_reduce.py:115-122).
A collective, hence outside this build; only the trivial one-source case is
answered, everything else raises."""

__all__ = ["SumReduceFunction"]

import torch


class SumReduceFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, P_send, P_recv, preserve_batch=True, tag=None):
        if P_send.active and P_send.size == 1 and P_recv.active:
            return input
        raise NotImplementedError("SumReduce over more than one source is a collective, not part of this build")

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("the adjoint of SumReduce is a collective, not part of this build")
