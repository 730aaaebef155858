"""Repartition forward / adjoint on one GPU.

Order of operations follows the reference
(backends/mpi_numpy/functional/repartition.py:142-213 forward, :285-355
adjoint): pack every outgoing overlap into its contiguous buffer, hand the
buffers to the transport, create the output, copy the self overlap directly,
unpack every incoming buffer.  The differences are where the work runs: all
outgoing boxes are packed by ONE kernel launch, which also makes the self copy,
and all incoming boxes are unpacked by ONE launch (``ddl_copy_boxes`` on box
descriptors that are built once per input structure, where the reference
builds its overlap lists) instead of one strided copy per peer, and the output
is not zero-filled first when the incoming boxes tile it completely (they
always do for a valid pair of partitions).
"""

__all__ = ["RepartitionFunction"]

import ctypes

import numpy as np
import torch

from .... import _lib
from .... import hip_ops
from ....utilities.torch import zero_volume_tensor
from .. import buffer as _buffer

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


def _contiguous_strides(shape):
    strides, run = [], 1
    for n in reversed(shape):
        strides.append(run)
        run *= int(n)
    return strides[::-1]


_BOX_WORDS = ctypes.sizeof(_lib.ddl_box_t) // 8     # a box descriptor as 8-byte words; words 0 and 1 are src and dst


class _MovePlan:
    """One direction of a Repartition (x -> y, or dy -> dx) for one input
    structure, lowered once to the two launches it takes:

      first   every outgoing box packed into its send buffer, and the box this
              worker keeps copied straight into the output
      second  every receive buffer unpacked into the output

    The box descriptors are built here; a call only writes the addresses that
    change (the source tensor, the fresh output) into them.  Buffer views have
    fixed addresses until some pooled buffer is reallocated, which invalidates
    the plan (``stale``).
    """

    def __init__(self, src, dtype, src_active, src_overlaps, src_buffers, dst_active, dst_overlaps, dst_buffers, dst_shape):
        self.reallocations = _buffer.reallocations()
        self.elem_size = torch.empty((), dtype=dtype).element_size()
        if src_active and src.dtype != dtype:
            raise ValueError(f"Repartition was set up for {dtype}, got a tensor of {src.dtype}")
        self.send_views = _views(src_overlaps, src_buffers) if src_active else []
        self.recv_views = _views(dst_overlaps, dst_buffers) if dst_active else []
        self.keep = (src_overlaps, src_buffers, dst_overlaps, dst_buffers)     # ids of these are part of the cache key
        self.out_shape = None if dst_shape is None else tuple(int(n) for n in dst_shape)
        self.zero_fill = dst_active and not _covered(dst_overlaps, self.out_shape)
        es = self.elem_size
        src_strides = [int(v) for v in src.stride()]
        out_strides = _contiguous_strides(self.out_shape) if dst_active else None

        def offset(slices, strides):
            return sum(int(sl.start) * st for sl, st in zip(slices, strides)) * es

        first, second = [], []      # (src address or None, src offset, dst address or None, dst offset, shape, sstr, dstr)
        if src_active:
            for (sl, sh, partner), view in zip(src_overlaps, self.send_views):
                if view is not None and view.numel() > 0:
                    shape = [int(n) for n in sh]
                    first.append((None, offset(sl, src_strides), view.data_ptr(), 0, shape, src_strides,
                                  _contiguous_strides(shape)))
            s_self, d_self = _self_slices(src_overlaps), (_self_slices(dst_overlaps) if dst_active else None)
            if s_self is not None and d_self is not None:
                shape = [int(sl.stop) - int(sl.start) for sl in s_self]
                if int(np.prod(shape, dtype=np.int64)) > 0:
                    first.append((None, offset(s_self, src_strides), None, offset(d_self, out_strides), shape, src_strides,
                                  out_strides))
        if dst_active:
            for (sl, sh, partner), view in zip(dst_overlaps, self.recv_views):
                if view is not None and view.numel() > 0:
                    shape = [int(n) for n in sh]
                    second.append((view.data_ptr(), 0, None, offset(sl, out_strides), shape, _contiguous_strides(shape),
                                   out_strides))
        self.first = self._lower(first)
        self.second = self._lower(second)
        self.sends = [(partner, view) for (sl, sh, partner), view in zip(src_overlaps, self.send_views) if view is not None] \
            if src_active else []
        self.recvs = [(partner, view) for (sl, sh, partner), view in zip(dst_overlaps, self.recv_views) if view is not None] \
            if dst_active else []

    @staticmethod
    def _lower(entries):
        """(box array, its words as a NumPy table, rows / offsets of the
        addresses that follow the source tensor, the same for the output)."""
        n = len(entries)
        if n == 0:
            return None
        boxes = (_lib.ddl_box_t * n)()
        words = np.frombuffer(boxes, dtype=np.int64).reshape(n, _BOX_WORDS)
        from_src, from_out = ([], []), ([], [])
        for i, (sa, so, da, do, shape, sstr, dstr) in enumerate(entries):
            box = boxes[i]
            box.ndim = len(shape)
            for d, (nd, s1, s2) in enumerate(zip(shape, sstr, dstr)):
                box.shape[d], box.src_stride[d], box.dst_stride[d] = nd, s1, s2
            if sa is None:
                from_src[0].append(i)
                from_src[1].append(so)
            else:
                box.src = sa
            if da is None:
                from_out[0].append(i)
                from_out[1].append(do)
            else:
                box.dst = da
        return (boxes, words, n,
                (np.asarray(from_src[0], dtype=np.intp), np.asarray(from_src[1], dtype=np.int64)),
                (np.asarray(from_out[0], dtype=np.intp), np.asarray(from_out[1], dtype=np.int64)))

    def stale(self):
        return self.reallocations != _buffer.reallocations()

    def launch(self, which, src_ptr, out_ptr, stream):
        if which is None:
            return
        boxes, words, n, (src_rows, src_offs), (out_rows, out_offs) = which
        if len(src_rows):
            words[src_rows, 0] = src_offs + src_ptr
        if len(out_rows):
            words[out_rows, 1] = out_offs + out_ptr
        rc = _lib.load().ddl_copy_boxes(boxes, n, self.elem_size, _lib.DDL_OP_COPY, _lib.DDL_DT_BITS, stream)
        if rc:
            _lib.check(rc, "ddl_copy_boxes")


def _move_plan(src, dtype, P_src, src_overlaps, src_buffers, P_dst, dst_overlaps, dst_buffers, dst_shape):
    cache = getattr(src_overlaps, "plans", None)
    if cache is None:
        cache = getattr(dst_overlaps, "plans", None)
    key = ("move", src.shape, src.stride(), src.dtype, dtype, id(src_overlaps), id(src_buffers), id(dst_overlaps),
           id(dst_buffers), None if dst_shape is None else tuple(int(n) for n in dst_shape))
    plan = None if cache is None else cache.get(key)
    if plan is None or plan.stale():
        plan = _MovePlan(src, dtype, P_src.active, src_overlaps, src_buffers, P_dst.active, dst_overlaps, dst_buffers, dst_shape)
        if cache is not None:
            cache[key] = plan
    return plan


def _move(src, P_union, dtype, P_src, src_overlaps, src_buffers, P_dst, dst_overlaps, dst_buffers, dst_shape,
          preserve_batch, tag):
    """Shared body of forward (x -> y) and adjoint (dy -> dx)."""
    device = src.device
    if not (P_src.active or P_dst.active):
        if preserve_batch:
            return zero_volume_tensor(src.shape[0], dtype=dtype, device=device)
        return zero_volume_tensor(dtype=dtype, device=device)
    if P_src.active and not src.is_cuda:
        raise RuntimeError(f"distdl_amd: tensor on {src.device}; the HIP path only accepts GPU tensors and there is "
                           "no CPU fallback")

    plan = _move_plan(src, dtype, P_src, src_overlaps, src_buffers, P_dst, dst_overlaps, dst_buffers, dst_shape)
    if P_dst.active:
        alloc = torch.zeros if plan.zero_fill else torch.empty
        out = alloc(plan.out_shape, dtype=dtype, device=device)
        out_ptr = out.data_ptr()
    else:
        out = zero_volume_tensor(src.shape[0], dtype=dtype, device=device) if preserve_batch else \
            zero_volume_tensor(dtype=dtype, device=device)
        out_ptr = 0
    stream = hip_ops._stream()
    plan.launch(plan.first, src.data_ptr() if P_src.active else 0, out_ptr, stream)
    if P_union.active and (plan.sends or plan.recvs):
        P_union._world.transport.exchange(P_union, [(p, v, tag) for p, v in plan.sends],
                                          [(p, v, tag) for p, v in plan.recvs])
    plan.launch(plan.second, 0, out_ptr, stream)
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
