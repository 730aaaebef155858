"""AllGather layer (reference: nn/all_gather.py): concatenates the shards of
the workers that differ along ``axes_all_gather``.  Under the solo transport the
caller supplies the already gathered activation and the layer is the identity;
otherwise the backend's AllGatherFunction runs (box-kernel re-layout forward,
reduce-scatter adjoint)."""

import numpy as np

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
        keep = [d in self.axes for d in range(P_x.dim)]
        self.P_allgather = P_x.create_cartesian_subtopology_partition(keep)
        self.identity = int(np.prod(self.P_allgather.shape)) == 1

    def forward(self, input):
        if not self.P_x.active or self.identity:
            return input
        transport = self.P_x._world.transport
        Function = self._distdl_backend.functional.all_gather.AllGatherFunction
        if getattr(transport, "ghosts_preloaded", False):
            # solo: the input already is the gathered tensor; only the scaling of the gradient remains
            return input if self.scale_backward is None else Function.apply(input, None, None, None, self.scale_backward)
        if len(self.axes) != 1:
            raise NotImplementedError("AllGather along several axes is not part of this build")
        return Function.apply(input, self.P_allgather, self.axes[0], None, self.scale_backward)
