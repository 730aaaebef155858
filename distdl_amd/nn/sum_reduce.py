"""SumReduce layer stand-in (reference: nn/sum_reduce.py).  Only the case in
which every destination worker has a single source is answered (no arithmetic
is needed then); a true reduction is a collective outside this build."""

from .module import Module


class SumReduce(Module):

    def __init__(self, P_x, P_y, transpose_src=False, transpose_dest=False, preserve_batch=True):
        super().__init__()
        self.P_x = P_x
        self.P_y = P_y
        self.preserve_batch = preserve_batch

    def forward(self, input):
        if not (self.P_x.active or self.P_y.active):
            return input
        sources = max(int(self.P_x.size), 1) // max(int(self.P_y.size), 1)
        if self.P_x.active and self.P_y.active and sources == 1:
            return input
        raise NotImplementedError("SumReduce with more than one source per destination is a collective, "
                                  "not part of this build")
