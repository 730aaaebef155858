"""Pooled communication buffers living in device memory.

Behaviour follows the reference's expandable buffers
(backends/common/buffer.py:74-108, backends/nccl_cupy/buffer_cupy.py:36-85,
108-136): a buffer is a 1-D raw allocation from which C-contiguous views of any
shape are carved at offset zero -- the wire layout of a packed box -- and which
grows by reallocate-and-copy; a manager hands out the first ``n`` buffers of a
dtype so that layers sharing a manager share memory.
"""

import numpy as np
import torch

from . import device as _device


# Number of times any buffer has been reallocated.  Whoever caches device
# addresses of buffer views compares this against the value it saw.
_reallocations = 0


def reallocations():
    return _reallocations


class ExpandableBuffer:

    def __init__(self, dtype, initial_capacity=0, device=None):
        self.dtype = dtype
        self.capacity = int(initial_capacity)
        self.device = _device.get_device() if device is None else device
        self.raw_buffer = torch.zeros(self.capacity, dtype=dtype, device=self.device)
        self.views = dict()

    def expand(self, new_capacity):
        new_capacity = int(new_capacity)
        if new_capacity <= self.capacity:
            return
        global _reallocations
        _reallocations += 1
        grown = torch.zeros(new_capacity, dtype=self.dtype, device=self.device)
        grown[:self.capacity].copy_(self.raw_buffer)
        self.raw_buffer = grown
        self.capacity = new_capacity
        self.views = {shape: self._carve(shape) for shape in self.views}

    def _carve(self, view_shape):
        volume = int(np.prod(view_shape, dtype=np.int64))
        return self.raw_buffer[:volume].view(view_shape)

    def allocate_view(self, view_shape):
        self.get_view(tuple(view_shape))

    def get_view(self, view_shape):
        view_shape = tuple(int(s) for s in view_shape)
        view = self.views.get(view_shape)
        if view is None:
            volume = int(np.prod(view_shape, dtype=np.int64))
            if volume > self.capacity:
                self.expand(volume)
            view = self.views[view_shape] = self._carve(view_shape)
        return view


class BufferManager:

    def __init__(self, device=None):
        self.buffers_map = dict()
        self.device = device

    def request_buffers(self, n_buffers, dtype, **kwargs):
        pool = self.buffers_map.setdefault(dtype, [])
        while len(pool) < n_buffers:
            pool.append(ExpandableBuffer(dtype, device=self.device, **kwargs))
        return pool[:n_buffers]
