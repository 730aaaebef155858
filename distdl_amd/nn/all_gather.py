"""AllGather layer (reference: nn/all_gather.py): concatenates the shards of
the workers that differ along ``axes_all_gather``.  Under the solo transport the
caller supplies the already gathered activation and the layer is the identity;
otherwise the backend's AllGatherFunction runs (box-kernel re-layout forward,
reduce-scatter adjoint)."""

import numpy as np

from ..utilities.torch import TensorStructure
from .module import Module


class AllGather(Module):

    def __init__(self, P_x, axes_all_gather=None, axes_keep=None, scale_backward=None):
        super().__init__()
        self.P_x = P_x
        if not P_x.active:
            return
        self.scale_backward = scale_backward
        if axes_all_gather is None:
            axes_all_gather = [d for d in range(P_x.dim) if d not in [int(a) for a in axes_keep]]
        self.axes = tuple(int(a) for a in axes_all_gather)
        self.axes_all_gather = self.axes
        self.P_allgather = P_x.create_allreduction_partition(self.axes)
        self.identity = int(np.prod(self.P_allgather.shape)) == 1

    def forward(self, input):
        if not self.P_x.active or self.identity:
            return input
        transport = self.P_x._world.transport
        Function = self._distdl_backend.functional.all_gather.AllGatherFunction
        if getattr(transport, "ghosts_preloaded", False):
            # solo: the input already is the gathered tensor; only the scaling of the gradient remains
            if self.scale_backward is None:
                return input
            return Function.apply(input, None, TensorStructure(input), TensorStructure(input), self.axes, self.scale_backward)
        # Positional arguments as in the reference (nn/all_gather.py:182-187).
        return Function.apply(input, self.P_allgather, TensorStructure(input), None, self.axes, self.scale_backward)
