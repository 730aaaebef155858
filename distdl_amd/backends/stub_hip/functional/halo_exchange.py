"""HaloExchange forward / adjoint on one GPU.

Dimension-ordered exchange of the reference
(backends/mpi_numpy/functional/halo_exchange.py:13-78 forward, :81-144
adjoint).  Per exchange dimension the two bulk slabs are packed by one launch,
the transport swaps them with the neighbours, and the two ghost slabs are
unpacked by one launch; dimension i sees the ghosts of dimensions < i, which is
what makes the corners right.  The adjoint walks the dimensions backwards:
pack the ghosts, clear them, swap, ADD what arrives into the bulk.
"""

__all__ = ["HaloExchangeFunction"]

import torch

from .... import hip_ops
from ....utilities.slicing import compute_nd_slice_shape
from ....utilities.torch import zero_volume_tensor
from ..partition import PROC_NULL

_LTAG = 0
_RTAG = 1


class SliceTable(list):
    """The per-dimension ``[left bulk, left ghost, right bulk, right ghost]``
    slices plus the C descriptors derived from them."""

    def __init__(self, *args):
        super().__init__(*args)
        self.plans = {}


def _plans(slices, tensor, i):
    """(bulk plan, ghost plan) of exchange dimension ``i``; each plan holds the
    left and the right box."""
    cache = getattr(slices, "plans", None)
    key = (i, tuple(tensor.shape), tuple(tensor.stride()))
    if cache is not None and key in cache:
        return cache[key]
    lbs, lgs, rbs, rgs = slices[i]
    plans = (hip_ops.BoxPlan.from_slices(tensor, [lbs, rbs]), hip_ops.BoxPlan.from_slices(tensor, [lgs, rgs]))
    if cache is not None:
        cache[key] = plans
    return plans


def _dim_views(slices_i, buffers_i):
    return [None if b is None else b.get_view(compute_nd_slice_shape(s)) for s, b in zip(slices_i, buffers_i)]


def _swap(P_x, neighbor_ranks_i, out_left, out_right, in_left, in_right):
    """Left message travels with tag 0, right message with tag 1; the receiver
    matches the opposite tag (reference :55-61)."""
    lrank, rrank = neighbor_ranks_i
    sends, recvs = [], []
    if in_left is not None and lrank != PROC_NULL:
        recvs.append((lrank, in_left, _RTAG))
    if in_right is not None and rrank != PROC_NULL:
        recvs.append((rrank, in_right, _LTAG))
    if out_left is not None and lrank != PROC_NULL:
        sends.append((lrank, out_left, _LTAG))
    if out_right is not None and rrank != PROC_NULL:
        sends.append((rrank, out_right, _RTAG))
    if sends or recvs:
        P_x._world.transport.exchange(P_x, sends, recvs)


class HaloExchangeFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, P_x, slices, buffers, neighbor_ranks):
        ctx.slices = slices
        ctx.buffers = buffers
        ctx.neighbor_ranks = neighbor_ranks
        ctx.P_x = P_x
        ctx.device = input.device

        if not P_x.active:
            return zero_volume_tensor(input.shape[0], device=input.device)
        if P_x.size == 1:
            return input

        # The reference works on a copy because marking the input dirty breaks
        # some downstream layers (halo_exchange.py:26-30); the copy runs on the
        # box kernel as one contiguous box.
        src = input.detach()
        output = torch.empty_like(src, memory_format=torch.contiguous_format)
        full = tuple(slice(0, int(s)) for s in src.shape)
        hip_ops.copy_box(src, full, output, full)

        for i in range(P_x.dim):
            lbb, lgb, rbb, rgb = _dim_views(slices[i], buffers[i])
            bulk_plan, ghost_plan = _plans(slices, output, i)
            if lbb is not None or rbb is not None:
                bulk_plan.pack(output, [lbb, rbb])
            _swap(P_x, neighbor_ranks[i], lbb, rbb, lgb, rgb)
            if lgb is not None or rgb is not None:
                ghost_plan.unpack(output, [lgb, rgb])
        return output

    @staticmethod
    def backward(ctx, grad_output):
        P_x, slices, buffers = ctx.P_x, ctx.slices, ctx.buffers
        if not P_x.active:
            return zero_volume_tensor(grad_output.shape[0], device=ctx.device), None, None, None, None
        if P_x.size == 1:
            return grad_output, None, None, None, None

        # In place on the incoming gradient, as the reference (:98).
        ctx.mark_dirty(grad_output)
        if not grad_output.is_contiguous():
            raise ValueError("HaloExchange adjoint needs a contiguous gradient")

        for i in reversed(range(P_x.dim)):
            lbb, lgb, rbb, rgb = _dim_views(slices[i], buffers[i])
            bulk_plan, ghost_plan = _plans(slices, grad_output, i)
            if lgb is not None or rgb is not None:
                ghost_plan.pack(grad_output, [lgb, rgb])
                ghost_plan.zero(grad_output)
            _swap(P_x, ctx.neighbor_ranks[i], lgb, rgb, lbb, rbb)
            if lbb is not None and rbb is not None and slices[i][0][i].stop > slices[i][2][i].start:
                # Narrow shards: the left and right bulk strips share elements, so
                # the two accumulations must not run in one launch.
                bulk_plan.unpack(grad_output, [lbb, None], accumulate=True)
                bulk_plan.unpack(grad_output, [None, rbb], accumulate=True)
            elif lbb is not None or rbb is not None:
                bulk_plan.unpack(grad_output, [lbb, rbb], accumulate=True)
        return grad_output, None, None, None, None
