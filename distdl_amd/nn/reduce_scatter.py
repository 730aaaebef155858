"""ReduceScatter layer (reference: nn/reduce_scatter.py): sums the tensors of
the workers that differ along ``axes_reduce_scatter`` and leaves every worker
its balanced slab of the sum.  Under the solo transport the absent workers
hold what the live one holds unless a gather provider supplies their tensors, so
without one the result is the live worker's slab of its own tensor times the
number of workers."""

import numpy as np

from ..utilities.torch import TensorStructure
from .module import Module


class ReduceScatter(Module):

    def __init__(self, P_x, axes_reduce_scatter=None, axes_keep=None):
        super().__init__()
        self.P_x = P_x
        if not P_x.active:
            return
        if axes_reduce_scatter is None:
            axes_reduce_scatter = [d for d in range(P_x.dim) if d not in [int(a) for a in axes_keep]]
        self.axes = tuple(int(a) for a in axes_reduce_scatter)
        self.axes_reduce_scatter = self.axes
        self.P_reducescatter = P_x.create_allreduction_partition(self.axes)
        self.identity = int(np.prod(self.P_reducescatter.shape)) == 1

    def forward(self, input):
        if not self.P_x.active or self.identity:
            return input
        Function = self._distdl_backend.functional.reduce_scatter.ReduceScatterFunction
        # Positional arguments as in the reference (nn/reduce_scatter.py:177-182).
        return Function.apply(input, self.P_reducescatter, TensorStructure(input), None, self.axes)
