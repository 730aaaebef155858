"""All-gather stand-in (reference: backends/mpi_numpy/functional/all_gather.py:88-149).
A collective followed by a local re-layout; outside this build."""

__all__ = ["AllGatherFunction"]

import torch


class AllGatherFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, P_allgather, axis=None, tag=None):
        if not P_allgather.active or P_allgather.size == 1:
            return input
        raise NotImplementedError("AllGather is a collective, not part of this build")

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("the adjoint of AllGather is a collective, not part of this build")
