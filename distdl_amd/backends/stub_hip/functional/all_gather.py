"""All-gather along one partitioned axis and its adjoint (reference:
backends/mpi_numpy/functional/all_gather.py:88-149, :152-230).  The collective
itself belongs to the transport; what runs here is the local re-layout the
reference does with einops (``p a b c -> a (p b) c``, zero-padding and stripping
uneven shards): the P received pieces are unpacked into their slabs of the
output by one launch of the box kernel, uneven pieces included.  The adjoint is
a reduce-scatter: every worker sums its slab of all workers' gradients in one
launch of the sum kernel (strided reads of the P slabs, one write)."""

__all__ = ["AllGatherFunction", "gather_slabs", "reduce_scatter_slabs", "single_axis"]

import numpy as np
import torch

from .... import hip_ops
from ....utilities.slicing import compute_subshape


def gather_slabs(P, local, axis, tag):
    """``local`` of every worker of ``P``, concatenated along ``axis`` in rank order."""
    transport = P._world.transport
    x = hip_ops.contiguous(local)
    parts = transport.gather_list(P, x, tag=tag)
    extent = sum(int(p.shape[axis]) for p in parts)
    shape = list(x.shape)
    shape[axis] = extent
    out = torch.empty(shape, dtype=x.dtype, device=x.device)
    boxes, start = [], 0
    for p in parts:
        origin = [0] * out.dim()
        origin[axis] = start
        boxes.append((origin, list(p.shape)))
        start += int(p.shape[axis])
    hip_ops.BoxPlan(out.shape, out.stride(), boxes).unpack(out, parts)
    transport.release(P, tag=tag)
    return out


def reduce_scatter_slabs(P, full, axis, tag, divisor=1):
    """Sum over the workers of ``P``, in rank order, of their ``full`` tensors
    (each divided by ``divisor`` first), of which this worker keeps its balanced
    slab along ``axis``: one launch that reads the P slabs where they lie and
    writes the result once."""
    transport = P._world.transport
    g = hip_ops.contiguous(full)
    grads = transport.gather_list(P, g, tag=tag)
    me = int(P.rank)
    extent = int(g.shape[axis])
    sizes = [int(np.asarray(compute_subshape(P.size, r, extent)).reshape(-1)[0]) for r in range(P.size)]
    start = sum(sizes[:me])
    shape = list(g.shape)
    shape[axis] = sizes[me]
    out = torch.empty(shape, dtype=g.dtype, device=g.device)
    src = [slice(0, int(n)) for n in g.shape]
    src[axis] = slice(start, start + sizes[me])
    dst = [slice(0, int(n)) for n in shape]
    if out.numel():
        hip_ops.sum_boxes(grads, src, out, dst, divisor)
    transport.release(P, tag=tag)
    return out


def single_axis(axes, who):
    """The one tensor axis a re-layout runs along (the reference's layers pass
    a tuple of axes; its einops pattern handles one, all_gather.py:126-149)."""
    axes = [int(a) for a in np.atleast_1d(np.asarray(axes))]
    if len(axes) != 1:
        raise NotImplementedError(f"{who} along several axes is not part of this build")
    return axes[0]


class AllGatherFunction(torch.autograd.Function):
    """Positional arguments as in the reference
    (backends/mpi_numpy/functional/all_gather.py:36-37).  The tensor structures
    are accepted and not needed: the output shape follows from the gathered
    pieces.  ``P_allgather`` None stands for a gather already done by the
    caller (solo transport): only the scaling of the gradient remains."""

    @staticmethod
    def forward(ctx, input, P_allgather, input_tensor_structure, output_tensor_structure, axes, scale_backward):
        ctx.scale_backward = scale_backward
        if P_allgather is None or not P_allgather.active or P_allgather.size == 1:
            ctx.identity = True
            return input
        ctx.identity = False
        ctx.P, ctx.axis = P_allgather, single_axis(axes, "AllGather")
        return gather_slabs(P_allgather, input.detach(), ctx.axis, ("all_gather", None))

    @staticmethod
    def backward(ctx, grad_output):
        grad_output = grad_output.detach()
        # Every worker's gradient is divided before the sum (reference :188-190): the sum kernel divides as it reads.
        divisor = 1 if ctx.scale_backward is None else ctx.scale_backward
        if ctx.identity:
            return (grad_output if divisor == 1 else hip_ops.scaled(grad_output, divisor)), None, None, None, None, None
        dx = reduce_scatter_slabs(ctx.P, grad_output, ctx.axis, ("all_gather_adjoint", None), divisor)
        return dx, None, None, None, None, None
