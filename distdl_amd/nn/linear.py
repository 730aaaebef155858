"""DistributedLinear (reference: nn/linear.py:11-108): broadcast x over the rows
of the weight partition, apply the local ``[out/P_fo, in/P_fi]`` shard, sum-reduce
the partial outputs.  The local apply (reference :103, ``self.sublinear(x)``) is
the MFMA kernel of the operands' type."""

__all__ = ["DistributedLinear"]

import torch

from .. import hip_ops
from ..utilities.slicing import compute_subshape
from .broadcast import Broadcast
from .module import Module
from .sum_reduce import SumReduce


class _LinearShard(torch.autograd.Function):
    """``F.linear`` and its adjoint (dx = dy w, dw = dy^T x, db = column sums of
    dy) on the HIP kernels."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        return hip_ops.linear(x.detach(), weight.detach(), None if bias is None else bias.detach())

    @staticmethod
    def backward(ctx, grad_output):
        x, weight = ctx.saved_tensors
        need_x, need_w, need_b = ctx.needs_input_grad
        dx, dw, db = hip_ops.linear_backward(x.detach(), weight.detach(), grad_output.detach().to(x.dtype),
                                             need_x, need_w, need_b and ctx.has_bias)
        return dx, dw, db


def linear_shard(x, weight, bias):
    """``x @ weight.T + bias`` on the HIP kernels: bfloat16 and float16 on the
    tuned MFMA kernel, float32 (the layers' default) on the fp32 one."""
    if x.dtype not in (torch.bfloat16, torch.float16, torch.float32) or weight.dtype != x.dtype:
        raise NotImplementedError(f"the linear shard kernels take bfloat16, float16 or float32 operands of one type "
                                  f"(got x {x.dtype}, weight {weight.dtype})")
    return _LinearShard.apply(x, weight, bias)


class DistributedLinear(Module):
    r"""Affine layer with ``P_x ~ 1 x P_fi``, ``P_y ~ 1 x P_fo`` and
    ``P_w ~ P_fo x P_fi``; ``in_features`` / ``out_features`` are global."""

    def __init__(self, P_x, P_y, P_w, in_features, out_features, bias=True):
        super().__init__()
        self.P_x = P_x
        self.P_y = P_y
        self.P_w = P_w
        self.bias = bias
        self.x_broadcast = Broadcast(self.P_x, self.P_w, preserve_batch=True)
        if self.P_w.active:
            local_in_features = compute_subshape(P_w.shape[1], P_w.index[1], in_features)
            local_out_features = compute_subshape(P_w.shape[0], P_w.index[0], out_features)
            # Only column 0 of the weight partition adds the bias, so that the
            # sum-reduce counts it once.
            bias = self.bias if (self.P_w.index[-1] == 0) else False
            self.sublinear = torch.nn.Linear(int(local_in_features[0]), int(local_out_features[0]), bias=bias,
                                             device=P_w.device)
        self.y_sum_reduce = SumReduce(self.P_w, self.P_y, transpose_src=True, preserve_batch=True)

    def forward(self, input):
        if not (self.P_x.active or self.P_y.active or self.P_w.active):
            return input
        x = self.x_broadcast(input)
        if self.P_w.active:
            x = linear_shard(x, self.sublinear.weight, self.sublinear.bias)
        return self.y_sum_reduce(x)
