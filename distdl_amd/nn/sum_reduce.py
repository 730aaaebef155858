"""SumReduce layer stand-in (reference: nn/sum_reduce.py): the partial tensors
held on ``P_x`` are summed onto ``P_y`` along the dimensions in which ``P_y`` has
one worker, by the reference's broadcast rules read backwards.  The collective
itself is outside this build; see backends/stub_hip/functional/sum_reduce.py."""

from ..utilities.torch import TensorStructure
from .module import Module


class SumReduce(Module):

    def __init__(self, P_x, P_y, transpose_src=False, transpose_dest=False, preserve_batch=True):
        super().__init__()
        self.P_x = P_x
        self.P_y = P_y
        self.transpose_src = transpose_src
        self.transpose_dest = transpose_dest
        self.preserve_batch = preserve_batch
        # Source and destination are the same team: nothing is added.
        self.identity = (P_x == P_y)
        self.P_send = self.P_recv = None
        if not self.identity and (P_x.active or P_y.active):
            self.P_send, self.P_recv = P_x.create_reduction_partition_to(P_y, transpose_src, transpose_dest)

    def forward(self, input):
        if self.identity or not (self.P_x.active or self.P_y.active):
            return input
        Function = self._distdl_backend.functional.sum_reduce.SumReduceFunction
        # Positional arguments as in the reference (nn/sum_reduce.py:205-211).
        return Function.apply(input, self.P_send, self.P_recv, self.preserve_batch, TensorStructure(input), None)
