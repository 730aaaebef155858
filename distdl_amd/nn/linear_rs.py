"""DistributedLinearReduceScatter (reference: nn/linear_rs.py:18-364): every
worker applies its weight shard ``[out, in/P]`` to its slice of the input
features (reference :361, ``F.linear``, here the MFMA kernel of the operands'
type) and the partial outputs are summed and scattered along the feature (or
token) axis (reference :364).  The bias is added by one worker of each group
that is summed, so that the sum counts it once."""

import math

import numpy as np
import torch

from ..utilities.slicing import compute_subshape
from ..utilities.slicing import worker_layout
from ..utilities.torch import zero_volume_tensor
from .broadcast import Broadcast
from .linear import linear_shard
from .module import Module
from .reduce_scatter import ReduceScatter


def _sub_partition(P, pick, shape):
    """Cartesian partition of ``shape`` over the workers of ``P`` selected by the
    index expression ``pick`` (row-major order)."""
    workers = worker_layout(P.shape)[tuple(pick)].reshape(-1).tolist()
    base = P.create_partition_inclusive(workers)
    part = base.create_cartesian_topology_partition(shape)
    base.deactivate()
    return part


class DistributedLinearReduceScatter(Module):
    r"""Signature of the reference.  ``P_x`` has the form ``[D, ..., 1, M]``;
    weights ``[out_features, in_features / M]`` live on the first data-parallel
    worker of every model-parallel column and are broadcast from there; the
    output is partitioned like ``P_x``, or like ``P_y = [D, ..., M, 1]`` when
    given.  ``collect_state=True`` (the state-dict re-layout) is not part of this
    build."""

    def __init__(self, P_x, in_features, out_features, bias=True, device=None, dtype=None,
                 P_y=None, P_weight=None, P_store_bias=None, P_apply_bias=None,
                 collect_state=False, scale_backward=None):
        super().__init__()
        self.P_x = P_x
        if not self.P_x.active:
            return
        assert P_x.shape[-2] == 1 or P_x.shape[-1] == 1
        if collect_state:
            raise NotImplementedError("collect_state=True is not part of this build")
        if P_y is None:
            self.P_y = P_x
        else:
            assert P_y.dim == P_x.dim
            assert P_y.shape[-2] == P_x.shape[-1]
            assert P_y.shape[-1] == 1
            self.P_y = P_y
        if device is None:
            device = P_x.device
        self.in_features = in_features
        self.out_features = out_features
        self.collect_state = collect_state
        self.use_bias = bias
        dim, M = P_x.dim, int(P_x.shape[-1])

        if P_weight is None:
            pick = [slice(0, 1)] * dim
            pick[-1] = slice(0, M)
            P_weight = _sub_partition(P_x, pick, [1] * (dim - 1) + [M])
        else:
            assert P_x.dim == P_weight.dim
            assert P_weight.shape[-1] == P_x.shape[-1]
            assert np.prod(P_weight.shape[:dim - 1]) == 1
        if P_store_bias is not None:
            assert P_x.dim == P_store_bias.dim
            assert np.prod(P_store_bias.shape) == 1
        elif bias:
            P_store_bias = _sub_partition(P_x, [slice(0, 1)] * dim, [1] * dim)
        if P_apply_bias is not None:
            assert P_x.dim == P_apply_bias.dim
            assert np.prod(P_apply_bias.shape[-2:]) == 1
            for i in range(dim - 2):
                assert P_apply_bias.shape[i] == P_x.shape[i]
        elif bias:
            pick = [slice(0, 1)] * dim
            for i in range(dim - 2):
                pick[i] = slice(0, int(P_x.shape[i]))
            P_apply_bias = _sub_partition(P_x, pick, [int(n) for n in P_x.shape[:dim - 2]] + [1, 1])
        self.P_weight = P_weight
        if bias:
            self.P_store_bias = P_store_bias
            self.P_apply_bias = P_apply_bias

        self.broadcast_weight = Broadcast(P_weight, P_x, scale_backward=scale_backward)
        if bias and self.P_apply_bias.active:
            self.broadcast_bias = Broadcast(P_store_bias, P_apply_bias, scale_backward=scale_backward)

        if P_weight.active:
            in_local = int(compute_subshape(P_weight.shape[-1], P_weight.index[-1], [in_features])[0])
            weight_shape = [1] * dim
            weight_shape[-1] = in_local
            weight_shape[-2] = out_features
            self.weight = torch.nn.Parameter(torch.empty(tuple(weight_shape), device=device, dtype=dtype))
        else:
            self.register_buffer('weight', zero_volume_tensor(device=device, requires_grad=True))
        if self.use_bias and self.P_store_bias.active:
            bias_shape = [1] * dim
            bias_shape[-2] = out_features
            self.bias = torch.nn.Parameter(torch.empty(tuple(bias_shape), device=device, dtype=dtype))
        elif self.use_bias and self.P_apply_bias.active:
            self.register_buffer('bias', zero_volume_tensor(device=device, requires_grad=True))
        else:
            self.register_parameter('bias', None)
        self.reset_parameters()

        scatter_dim = int(np.argmax(np.asarray(self.P_y.shape[-2:]))) + self.P_y.dim - 2
        self.reduce_scatter = ReduceScatter(self.P_y, axes_reduce_scatter=(scatter_dim,))
        self.weight_buffer = None
        if self.use_bias:
            self.bias_buffer = None

    def reset_parameters(self) -> None:
        """Kaiming-uniform weight shards; the bias uniform within the bound of
        the GLOBAL fan-in, as the reference computes it (:228-231)."""
        if self.P_weight.active:
            with torch.no_grad():
                torch.nn.init.kaiming_uniform_(self.weight.view(self.out_features, -1), a=math.sqrt(5))
        if self.use_bias and self.P_store_bias.active:
            bound = 1 / math.sqrt(self.in_features) if self.in_features > 0 else 0
            with torch.no_grad():
                torch.nn.init.uniform_(self.bias, -bound, bound)

    def extra_repr(self) -> str:
        return f'in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}'

    def prefetch_weights(self):
        if self.P_x.size == 1:
            return
        self.weight_buffer = self.broadcast_weight(self.weight).view(self.out_features, -1)
        if self.bias is not None:
            self.bias_buffer = self.broadcast_bias(self.bias).view(self.out_features)

    def forward(self, input):
        if not self.P_x.active:
            return input
        if self.weight_buffer is None:
            weight = self.broadcast_weight(self.weight).view(self.out_features, -1)
        else:
            weight = self.weight_buffer
            self.weight_buffer = None
        if self.bias is not None:
            if self.bias_buffer is None:
                bias = self.broadcast_bias(self.bias).view(self.out_features)
            else:
                bias = self.bias_buffer
                self.bias_buffer = None
        else:
            bias = None
        return self.reduce_scatter(linear_shard(input, weight, bias))
