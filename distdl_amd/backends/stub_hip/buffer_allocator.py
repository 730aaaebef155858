"""Buffer layout of the two data-movement layers (reference:
backends/common/buffer_allocator.py:7-60 and :63-94)."""

import numpy as np

from ...utilities.slicing import compute_nd_slice_shape


def _needs_buffer(overlap):
    sl, sh, partner = overlap
    return sl is not None and partner != "self"


def allocate_repartition_buffers(buffer_manager, P_x_to_y_overlaps, P_y_to_x_overlaps, dtype):
    """One pooled buffer per overlap with another worker: all send buffers
    first, then all receive buffers; ``None`` for empty and self overlaps."""
    count = sum(_needs_buffer(o) for o in P_x_to_y_overlaps) + sum(_needs_buffer(o) for o in P_y_to_x_overlaps)
    pool = iter(buffer_manager.request_buffers(count, dtype=dtype))
    out = []
    for overlaps in (P_x_to_y_overlaps, P_y_to_x_overlaps):
        side = []
        for overlap in overlaps:
            buff = None
            if _needs_buffer(overlap):
                buff = next(pool)
                buff.allocate_view(overlap[1])
            side.append(buff)
        out.append(side)
    return out[0], out[1]


def allocate_halo_exchange_buffers(buffer_manager, slices, recv_buffer_shape, send_buffer_shape, dtype):
    """Exactly four pooled buffers (left bulk, left ghost, right bulk, right
    ghost) shared by every exchange dimension, since dimensions are processed
    one after the other."""
    pool = buffer_manager.request_buffers(4, dtype=dtype)
    out = []
    for i in range(len(slices)):
        widths = (send_buffer_shape[i, 0], recv_buffer_shape[i, 0], send_buffer_shape[i, 1], recv_buffer_shape[i, 1])
        per_dim = []
        for j in range(4):
            buff = None
            if widths[j] > 0:
                shape = compute_nd_slice_shape(slices[i][j])
                if np.prod(shape) > 0:
                    buff = pool[j]
                    buff.allocate_view(shape)
            per_dim.append(buff)
        out.append(per_dim)
    return out
