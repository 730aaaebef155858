"""AllSumReduce layer stand-in (reference: nn/all_sum_reduce.py:36-178): sums a
tensor over the workers that share every Cartesian index outside ``axes_reduce``."""

import numpy as np

from ..utilities.torch import TensorStructure
from .module import Module


class AllSumReduce(Module):

    def __init__(self, P_x, axes_reduce=None, axes_keep=None, scale_backward=None):
        super().__init__()
        self.P_x = P_x
        self.scale_backward = scale_backward
        if not P_x.active:
            self.P_allreduce = None
            return
        if axes_reduce is None and axes_keep is None:
            raise ValueError("One of `axes_reduce` or `axes_keep` must be given.")
        if axes_reduce is not None and axes_keep is not None:
            raise ValueError("Only one of `axes_reduce` or `axes_keep` may be given.")
        dims = range(P_x.dim)
        if axes_reduce is None:
            axes_reduce = [d for d in dims if d not in [int(a) for a in axes_keep]]
        self.axes_reduce = tuple(int(a) for a in axes_reduce)
        # The workers this worker reduces with, row-major over the reduced axes.
        self.P_allreduce = P_x.create_allreduction_partition(self.axes_reduce)
        self.identity = int(np.prod(self.P_allreduce.shape)) == 1

    def forward(self, input):
        if not self.P_x.active or self.identity:
            return input
        Function = self._distdl_backend.functional.all_sum_reduce.AllSumReduceFunction
        # Positional arguments as in the reference (nn/all_sum_reduce.py:174-178).
        structure = TensorStructure(input)
        return Function.apply(input, self.P_allreduce, structure, structure, self.scale_backward)
