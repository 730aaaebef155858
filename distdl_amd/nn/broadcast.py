"""Broadcast layer stand-in (reference: nn/broadcast.py).  The collective itself
is outside this build; see backends/stub_hip/functional/broadcast.py."""

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

    def forward(self, input):
        if self.identity or not (self.P_x.active or self.P_y.active):
            return input
        Function = self._distdl_backend.functional.broadcast.BroadcastFunction
        return Function.apply(input, self.P_x, self.P_y, self.preserve_batch, None,
                              self.transpose_src, self.transpose_dest, self.scale_backward)
