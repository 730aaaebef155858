"""Reduce-scatter stand-in (reference: backends/mpi_numpy/functional/reduce_scatter.py:86-127).
A collective preceded by a local re-layout; outside this build."""

__all__ = ["ReduceScatterFunction"]

import torch


class ReduceScatterFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, P_reducescatter, axis=None, tag=None):
        if not P_reducescatter.active or P_reducescatter.size == 1:
            return input
        raise NotImplementedError("ReduceScatter is a collective, not part of this build")

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("the adjoint of ReduceScatter is a collective, not part of this build")
