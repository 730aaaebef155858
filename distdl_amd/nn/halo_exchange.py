"""HaloExchange layer (reference: nn/halo_exchange.py:5-151)."""

import numpy as np

from ..utilities.torch import TensorStructure
from .module import Module


def assemble_halo_slices(x_local_shape, recv_buffer_shape, send_buffer_shape):
    """Four boxes per exchange dimension ``i`` -- left bulk, left ghost, right
    bulk, right ghost -- of a tensor that already contains its ghost regions
    (reference nn/halo_exchange.py:37-99).

    Along ``i`` itself a box is the strip in question.  Dimensions before ``i``
    span the whole tensor, ghosts included, because they have already been
    exchanged; dimensions after ``i`` span the bulk only.  This nesting is what
    carries corner values across two hops.
    """
    recv = np.asarray(recv_buffer_shape).astype(int)
    send = np.asarray(send_buffer_shape).astype(int)
    dim = len(x_local_shape)
    size = [int(s) for s in x_local_shape]
    whole = [slice(0, size[j], None) for j in range(dim)]
    bulk = [slice(int(recv[j, 0]), size[j] - int(recv[j, 1]), None) for j in range(dim)]
    table = []
    for i in range(dim):
        lrecv, rrecv = int(recv[i, 0]), int(recv[i, 1])
        lsend, rsend = int(send[i, 0]), int(send[i, 1])
        strips = (slice(lrecv, lrecv + lsend, None),                        # left bulk
                  slice(0, lrecv, None),                                    # left ghost
                  slice(size[i] - rrecv - rsend, size[i] - rrecv, None),    # right bulk
                  slice(size[i] - rrecv, size[i], None))                    # right ghost
        table.append([tuple(whole[:i] + [strip] + bulk[i + 1:]) for strip in strips])
    return table


class HaloExchange(Module):

    def __init__(self, P_x, halo_shape, recv_buffer_shape, send_buffer_shape, buffer_manager=None):
        super().__init__()
        self.P_x = P_x
        self.halo_shape = halo_shape
        self.recv_buffer_shape = recv_buffer_shape
        self.send_buffer_shape = send_buffer_shape

        self.neighbor_ranks = None
        if self.P_x.active:
            self.neighbor_ranks = self.P_x.neighbor_ranks(self.P_x.rank)

        self.slices = None
        self.buffers = None

        if buffer_manager is None:
            buffer_manager = self._distdl_backend.BufferManager()
        elif type(buffer_manager) is not self._distdl_backend.BufferManager:
            raise ValueError("Buffer manager type does not match backend.")
        self.buffer_manager = buffer_manager

        self._distdl_is_setup = False
        self._input_tensor_structure = TensorStructure()
        self.allocate_halo_exchange_buffers = self._distdl_backend.buffer_allocator.allocate_halo_exchange_buffers

    def _assemble_slices(self, x_local_shape, recv_buffer_shape, send_buffer_shape):
        return assemble_halo_slices(x_local_shape, recv_buffer_shape, send_buffer_shape)

    def _distdl_module_setup(self, input):
        if self.P_x.active:
            SliceTable = self._distdl_backend.functional.halo_exchange.SliceTable
            self.slices = SliceTable(self._assemble_slices(input[0].shape, self.recv_buffer_shape,
                                                           self.send_buffer_shape))
            self.buffers = self.allocate_halo_exchange_buffers(self.buffer_manager,
                                                               self.slices,
                                                               self.recv_buffer_shape,
                                                               self.send_buffer_shape,
                                                               input[0].dtype)
            self.P_x.initialize_backend_comm()
        self._distdl_is_setup = True
        self._input_tensor_structure = TensorStructure(input[0])

    def _distdl_module_teardown(self, input):
        self.slices = None
        self.buffers = None
        self._distdl_is_setup = False
        self._input_tensor_structure = TensorStructure()

    def _distdl_input_changed(self, input):
        return self._input_tensor_structure != TensorStructure(input[0])

    def forward(self, input):
        Function = self._distdl_backend.functional.halo_exchange.HaloExchangeFunction
        if not self.P_x.active:
            return input
        return Function.apply(input, self.P_x, self.slices, self.buffers, self.neighbor_ranks)
