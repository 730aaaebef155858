"""DistributedLinearAllGather (reference: nn/linear_ag.py:22-486): all-gather
the input along the partitioned feature (or token) axis, then apply the weight
shard ``[out/P, in]`` (reference :486, ``F.linear``) with the bf16 MFMA kernel.
The output stays partitioned along the feature axis."""

import math

import numpy as np
import torch

from ..utilities.slicing import compute_subshape
from ..utilities.slicing import worker_layout
from ..utilities.torch import zero_volume_tensor
from .all_gather import AllGather
from .broadcast import Broadcast
from .linear import linear_shard
from .module import Module


class DistributedLinearAllGather(Module):
    r"""Signature of the reference.  ``collect_state``, ``num_heads``,
    ``num_heads_kv``, ``num_vars`` and ``geglu`` only steer the state-dict
    re-layout, which is not part of this build (``collect_state=True`` raises)."""

    def __init__(self, P_y, in_features, out_features, bias=True, device=None, dtype=None,
                 P_x=None, P_store_weight=None, P_apply_weight=None, collect_state=False, num_heads=None,
                 num_heads_kv=None, num_vars=3, geglu=False, scale_backward=None):
        super().__init__()
        self.P_y = P_y
        if not self.P_y.active:
            return
        assert P_y.shape[-2] == 1 or P_y.shape[-1] == 1
        if collect_state:
            raise NotImplementedError("collect_state=True is not part of this build")
        if P_x is None:
            self.P_x = P_y
        else:
            assert P_x.dim == P_y.dim
            assert P_x.shape[-2] == P_y.shape[-1]
            assert P_x.shape[-1] == 1
            self.P_x = P_x
        if device is None:
            device = P_y.device
        self.in_features = in_features
        self.out_features = out_features
        self.collect_state = collect_state
        self.num_heads, self.num_heads_kv, self.num_vars, self.geglu = num_heads, num_heads_kv, num_vars, geglu
        self.use_bias = bias

        # Weights are stored on the workers of the last partition axis (index 0
        # elsewhere), laid out as a column of workers; they are applied on a
        # partition shaped like P_y with its last two axes swapped.
        if P_store_weight is None:
            store_shape = [1] * P_y.dim
            store_shape[-2] = int(P_y.shape[-1])
            pick = [slice(0, 1)] * P_y.dim
            pick[-1] = slice(0, int(P_y.shape[-1]))
            workers = worker_layout(P_y.shape)[tuple(pick)].reshape(-1).tolist()
            base = P_y.create_partition_inclusive(workers)
            P_store_weight = base.create_cartesian_topology_partition(store_shape)
            base.deactivate()
        else:
            assert P_y.dim == P_store_weight.dim
            assert P_store_weight.shape[-2] == P_y.shape[-1]
            assert P_store_weight.shape[-1] == 1
        if P_apply_weight is None:
            apply_shape = np.asarray(P_y.shape).astype(int).copy()
            apply_shape[-1] = 1
            apply_shape[-2] = int(P_y.shape[-1])
            base = P_y.create_partition_inclusive(range(P_y.size))
            P_apply_weight = base.create_cartesian_topology_partition(apply_shape)
            base.deactivate()
        else:
            assert P_y.dim == P_apply_weight.dim
            assert P_apply_weight.shape[-1] == 1
            assert P_apply_weight.shape[-2] == P_y.shape[-1]
        self.P_store_weight = P_store_weight
        self.P_apply_weight = P_apply_weight
        self.broadcast_weight = Broadcast(P_store_weight, P_apply_weight, scale_backward=scale_backward)
        if bias:
            self.broadcast_bias = Broadcast(P_store_weight, P_apply_weight, scale_backward=scale_backward)

        if P_store_weight.active:
            out_local = int(compute_subshape(P_store_weight.shape[-2], P_store_weight.index[-2], [out_features])[0])
            weight_shape = [1] * P_y.dim
            weight_shape[-1] = in_features
            weight_shape[-2] = out_local
            self.weight = torch.nn.Parameter(torch.empty(tuple(weight_shape), device=device, dtype=dtype))
        else:
            self.register_buffer('weight', zero_volume_tensor(device=device, requires_grad=True))
        if self.use_bias and P_store_weight.active:
            bias_shape = [1] * P_y.dim
            bias_shape[-2] = out_local
            self.bias = torch.nn.Parameter(torch.empty(tuple(bias_shape), device=device, dtype=dtype))
        elif self.use_bias:
            self.register_buffer('bias', zero_volume_tensor(device=device, requires_grad=True))
        else:
            self.register_parameter('bias', None)
        self.reset_parameters()

        gather_dim = int(np.argmax(np.asarray(self.P_x.shape[-2:]))) + self.P_x.dim - 2
        self.all_gather = AllGather(self.P_x, axes_all_gather=(gather_dim,))
        self.weight_buffer = None
        if self.use_bias:
            self.bias_buffer = None

    def reset_parameters(self) -> None:
        """Kaiming-uniform weights and the matching uniform bias, as ``torch.nn.Linear``."""
        if self.P_store_weight.active:
            with torch.no_grad():
                torch.nn.init.kaiming_uniform_(self.weight.view(-1, self.in_features), a=math.sqrt(5))
                if self.use_bias:
                    bound = 1 / math.sqrt(self.in_features) if self.in_features > 0 else 0
                    torch.nn.init.uniform_(self.bias, -bound, bound)

    def prefetch_weights(self):
        if self.P_x.size == 1:
            return
        self.weight_buffer = self.broadcast_weight(self.weight).view(-1, self.in_features)
        if self.bias is not None:
            self.bias_buffer = self.broadcast_bias(self.bias).view(-1)

    def forward(self, input):
        if not self.P_y.active:
            return input
        input = self.all_gather(input)
        if self.weight_buffer is None:
            weight = self.broadcast_weight(self.weight).view(-1, self.in_features)
        else:
            weight = self.weight_buffer
            self.weight_buffer = None
        if self.bias is not None:
            if self.bias_buffer is None:
                bias = self.broadcast_bias(self.bias).view(weight.shape[-2])
            else:
                bias = self.bias_buffer
                self.bias_buffer = None
        else:
            bias = None
        return linear_shard(input, weight, bias)
