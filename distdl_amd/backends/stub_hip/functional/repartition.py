"""Repartition forward / adjoint on one GPU.

Order of operations follows the reference
(backends/mpi_numpy/functional/repartition.py:142-213 forward, :285-355
adjoint): pack every outgoing overlap into its contiguous buffer, hand the
buffers to the transport, create the output, copy the self overlap directly,
unpack every incoming buffer.  The differences are where the work runs: all
outgoing boxes are packed by ONE kernel launch and all incoming boxes unpacked
by ONE launch (``ddl_pack_boxes`` / ``ddl_unpack_boxes``) instead of one strided
copy per peer, and the output is not zero-filled first when the incoming boxes
tile it completely (they always do for a valid pair of partitions).
"""

__all__ = ["RepartitionFunction"]

import numpy as np
import torch

from .... import hip_ops
from ....utilities.torch import zero_volume_tensor

_FWD_TAG = 111
_ADJ_TAG = 113


class OverlapList(list):
    """List of ``(slices, shape, partner)`` that also carries the C descriptors
    derived from it, so that they are built once per input structure."""

    def __init__(self, *args):
        super().__init__(*args)
        self.plans = {}


def _plan(overlaps, tensor, which):
    """Box plan of the non-self (``which='remote'``) overlaps of ``tensor``."""
    cache = getattr(overlaps, "plans", None)
    key = (which, tuple(tensor.shape), tuple(tensor.stride()))
    if cache is not None and key in cache:
        return cache[key]
    boxes = []
    for sl, sh, partner in overlaps:
        if sl is None or partner == "self":
            boxes.append(None)
        else:
            boxes.append(sl)
    plan = hip_ops.BoxPlan.from_slices(tensor, boxes)
    if cache is not None:
        cache[key] = plan
    return plan


def _views(overlaps, buffers):
    out = []
    for (sl, sh, partner), buff in zip(overlaps, buffers):
        out.append(None if buff is None else buff.get_view(sh))
    return out


def _self_slices(overlaps):
    for sl, sh, partner in overlaps:
        if partner == "self":
            return sl
    return None


def _covered(overlaps, shape):
    """Do the (disjoint) overlaps tile a tensor of this shape completely?"""
    cache = getattr(overlaps, "plans", None)
    key = ("covered", shape)
    if cache is not None and key in cache:
        return cache[key]
    volume = 0
    for sl, sh, partner in overlaps:
        if sl is not None:
            volume += int(np.prod(sh, dtype=np.int64))
    covered = volume == int(np.prod(shape, dtype=np.int64))
    if cache is not None:
        cache[key] = covered
    return covered


def _move(src, P_union, dtype, P_src, src_overlaps, src_buffers, P_dst, dst_overlaps, dst_buffers, dst_shape,
          preserve_batch, tag):
    """Shared body of forward (x -> y) and adjoint (dy -> dx)."""
    device = src.device
    if preserve_batch:
        out = zero_volume_tensor(src.shape[0], dtype=dtype, device=device)
    else:
        out = zero_volume_tensor(dtype=dtype, device=device)

    sends, recvs = [], []
    if P_dst.active:
        recv_views = _views(dst_overlaps, dst_buffers)
        for (sl, sh, partner), view in zip(dst_overlaps, recv_views):
            if view is not None:
                recvs.append((partner, view, tag))
    if P_src.active:
        send_views = _views(src_overlaps, src_buffers)
        if any(v is not None for v in send_views):
            _plan(src_overlaps, src, "remote").pack(src, send_views)
        for (sl, sh, partner), view in zip(src_overlaps, send_views):
            if view is not None:
                sends.append((partner, view, tag))

    if P_union.active and (sends or recvs):
        P_union._world.transport.exchange(P_union, sends, recvs)

    if P_dst.active:
        shape = tuple(int(s) for s in dst_shape)
        if _covered(dst_overlaps, shape):
            out = torch.empty(shape, dtype=dtype, device=device)
        else:
            out = torch.zeros(shape, dtype=dtype, device=device)
        if P_src.active:
            s_self, d_self = _self_slices(src_overlaps), _self_slices(dst_overlaps)
            if s_self is not None and d_self is not None:
                hip_ops.copy_box(src, s_self, out, d_self)
        if any(v is not None for v in recv_views):
            _plan(dst_overlaps, out, "remote").unpack(out, recv_views)
    return out


class RepartitionFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, P_union, x_global_structure,
                x_local_structure, y_local_structure,
                P_x, P_x_to_y_overlaps, P_x_to_y_buffers,
                P_y, P_y_to_x_overlaps, P_y_to_x_buffers, preserve_batch):
        ctx.P_union = P_union
        ctx.x_global_structure = x_global_structure
        ctx.x_local_structure = x_local_structure
        ctx.P_x = P_x
        ctx.P_x_to_y_overlaps = P_x_to_y_overlaps
        ctx.P_x_to_y_buffers = P_x_to_y_buffers
        ctx.P_y = P_y
        ctx.P_y_to_x_overlaps = P_y_to_x_overlaps
        ctx.P_y_to_x_buffers = P_y_to_x_buffers
        ctx.preserve_batch = preserve_batch
        ctx.device = input.device

        # The reference shares requires_grad of the first input worker with the
        # whole union on every call (repartition.py:111-127).
        rg = input.requires_grad
        if P_union.active:
            rg = bool(P_union.broadcast_data(bool(input.requires_grad) if P_x.active else None, root=0))
        ctx.input_requires_grad = rg

        return _move(input.detach(), P_union, x_global_structure.dtype,
                     P_x, P_x_to_y_overlaps, P_x_to_y_buffers,
                     P_y, P_y_to_x_overlaps, P_y_to_x_buffers,
                     y_local_structure.shape if P_y.active else None, preserve_batch, _FWD_TAG)

    @staticmethod
    def backward(ctx, grad_output):
        """Adjoint: the same movement with the two overlap lists exchanged; the
        boxes are disjoint, so it copies and never adds (reference :344-346)."""
        grad_input = _move(grad_output.detach(), ctx.P_union, ctx.x_global_structure.dtype,
                           ctx.P_y, ctx.P_y_to_x_overlaps, ctx.P_y_to_x_buffers,
                           ctx.P_x, ctx.P_x_to_y_overlaps, ctx.P_x_to_y_buffers,
                           ctx.x_local_structure.shape if ctx.P_x.active else None, ctx.preserve_batch, _ADJ_TAG)
        return grad_input, None, None, None, None, None, None, None, None, None, None, None
