"""Broadcast layer stand-in (reference: nn/broadcast.py).  The collective itself
is outside this build; see backends/stub_hip/functional/broadcast.py."""

from ..utilities.torch import TensorStructure
from .module import Module


class Broadcast(Module):

    def __init__(self, P_x, P_y, transpose_src=False, transpose_dest=False, preserve_batch=True,
                 scale_backward=None):
        super().__init__()
        self.P_x = P_x
        self.P_y = P_y
        self.transpose_src = transpose_src
        self.transpose_dest = transpose_dest
        self.preserve_batch = preserve_batch
        self.scale_backward = scale_backward
        # Source and destination are the same team: nothing moves.
        self.identity = (P_x == P_y)
        self.P_send = self.P_recv = None
        if not self.identity and (P_x.active or P_y.active):
            self.P_send, self.P_recv = P_x.create_broadcast_partition_to(P_y, transpose_src, transpose_dest)

    def forward(self, input):
        if self.identity or not (self.P_x.active or self.P_y.active):
            return input
        Function = self._distdl_backend.functional.broadcast.BroadcastFunction
        # Positional arguments as in the reference (nn/broadcast.py:215-221).
        return Function.apply(input, self.P_send, self.P_recv, self.preserve_batch, TensorStructure(input), None,
                              self.scale_backward)
