"""Halo geometry of sliding-window layers on a partitioned tensor (reference:
nn/mixins/halo_mixin.py:9-207).

For every dimension a worker owns the global input indices
``[start, start + n)`` and must produce the global output indices of its
balanced output block.  The first and last of those outputs read inputs from
``stride*o - padding`` up to ``stride*o + dilation*(k-1) - padding`` (clamped
to the tensor); whatever lies outside the owned range is halo.  What a worker
sends to a neighbour is that neighbour's halo on the facing side.
"""

import numpy as np

from ...utilities.slicing import compute_start_index
from ...utilities.slicing import compute_subshape


def _left_pad_to(values, length, fill):
    values = np.atleast_1d(values)
    return np.concatenate([np.full(length - len(values), fill, dtype=values.dtype), values])


class HaloMixin:

    def _compute_exchange_info(self, x_global_shape, kernel_size, stride, padding, dilation,
                               partition_active, partition_shape, partition_index, subtensor_shapes=None):
        """Returns ``(halo_shape, recv_buffer_shape, send_buffer_shape,
        needed_ranges)``, each ``[dim, 2]`` (left, right) (reference :9-111)."""
        if not partition_active:
            return None, None, None, None

        x_global_shape = np.atleast_1d(x_global_shape)
        nd = len(x_global_shape)
        kernel_size = _left_pad_to(kernel_size, nd, 1)
        stride = _left_pad_to(stride, nd, 1)
        padding = _left_pad_to(padding, nd, 0)
        dilation = _left_pad_to(dilation, nd, 1)
        window = (x_global_shape, kernel_size, stride, padding, dilation)

        def halo_of(index, nonneg=True):
            return self._compute_halo_shape(partition_shape, index, *window, require_nonnegative=nonneg,
                                            subtensor_shapes=subtensor_shapes)

        halo_shape = halo_of(partition_index)
        recv_buffer_shape = halo_shape.copy()
        send_buffer_shape = np.zeros_like(halo_shape, dtype=int)
        for i in range(len(partition_shape)):
            for side, step in ((0, -1), (1, +1)):
                neighbour = [int(v) for v in partition_index]
                neighbour[i] += step
                if 0 <= neighbour[i] < partition_shape[i]:
                    # my left send width is my left neighbour's right halo, and vice versa
                    send_buffer_shape[i, side] = halo_of(neighbour)[i, 1 - side]

        if subtensor_shapes is not None:
            x_local_shape = subtensor_shapes[tuple(partition_index)]
        else:
            x_local_shape = compute_subshape(partition_shape, partition_index, x_global_shape)
        needed_ranges = self._compute_needed_ranges(x_local_shape, halo_of(partition_index, nonneg=False))
        return halo_shape.astype(int), recv_buffer_shape, send_buffer_shape, needed_ranges.astype(int)

    def _compute_local_start_index(self, index, subtensor_shapes, x_local_shape):
        """Global start of an unbalanced shard: sum of the extents of the shards
        before it along each axis (reference :113-124)."""
        nd = len(x_local_shape)
        start = np.zeros(nd, dtype=int)
        for d in range(nd):
            for i in range(int(index[d])):
                probe = tuple(i if j == d else 0 for j in range(nd))
                start[d] += subtensor_shapes[probe][d]
        return start

    def _compute_needed_ranges(self, tensor_shape, halo_shape):
        """Slice of the exchanged tensor the local kernel must see: a negative
        left halo is skipped, the stop is owned extent plus positive halos
        (reference :126-141)."""
        ranges = np.zeros_like(halo_shape, dtype=int)
        ranges[:, 0] = -np.minimum(0, halo_shape[:, 0])
        ranges[:, 1] = np.asarray(tensor_shape) + np.maximum(0, halo_shape[:, 0]) + np.maximum(0, halo_shape[:, 1])
        return ranges

    def _compute_out_shape(self, in_shape, kernel_size, stride, padding, dilation):
        """Output extent of a sliding window (reference :143-145)."""
        return np.floor((in_shape + 2 * padding - dilation * (kernel_size - 1) - 1) / stride + 1).astype(in_shape.dtype)

    def _compute_halo_shape(self, shape, index, x_global_shape, kernel_size, stride, padding, dilation,
                            require_nonnegative=True, subtensor_shapes=None):
        """``[dim, 2]`` halo widths of the worker at ``index`` (reference :147-207)."""
        x_global_shape = np.asarray(x_global_shape)
        if subtensor_shapes is not None:
            x_n = subtensor_shapes[tuple(index)]
            x_lo = self._compute_local_start_index(index, subtensor_shapes, x_n)
        else:
            x_n = compute_subshape(shape, index, x_global_shape)
            x_lo = compute_start_index(shape, index, x_global_shape)
        x_hi = x_lo + x_n - 1                                  # last owned index

        y_global_shape = self._compute_out_shape(x_global_shape, kernel_size, stride, padding, dilation)
        y_n = compute_subshape(shape, index, y_global_shape)
        y_lo = compute_start_index(shape, index, y_global_shape)
        y_hi = y_lo + y_n - 1

        need_lo = self._compute_min_input_range(y_lo, kernel_size, stride, padding, dilation)
        need_lo = np.maximum(np.zeros_like(x_global_shape), need_lo)
        need_hi = self._compute_max_input_range(y_hi, kernel_size, stride, padding, dilation)
        need_hi = np.minimum(x_global_shape - 1, need_hi)

        left, right = x_lo - need_lo, need_hi - x_hi
        if require_nonnegative:
            left, right = np.maximum(left, 0), np.maximum(right, 0)
        return np.stack([left, right], axis=1)
