"""Repartition layer (reference: nn/repartition.py:14-370)."""

import numpy as np

from ..utilities.slicing import compute_nd_slice_shape
from ..utilities.slicing import compute_subshape
from ..utilities.slicing import range_index
from ..utilities.tensor_decomposition import compute_subtensor_intersection_slice
from ..utilities.tensor_decomposition import compute_subtensor_shapes_balanced
from ..utilities.tensor_decomposition import compute_subtensor_start_indices
from ..utilities.tensor_decomposition import compute_subtensor_stop_indices
from ..utilities.torch import TensorStructure
from .module import Module


def compute_overlaps(my_index, my_start_table, my_stop_table, peer_partition_shape, peer_start_table,
                     peer_stop_table, self_index, peer_union_ranks):
    """Overlap of this worker's box with the box of every worker of the peer
    partition, in row-major order of the peer partition (reference
    nn/repartition.py:218-253 for the send side, :257-288 for the receive side).

    Returns a list of ``(slices, shape, partner)``: slices relative to this
    worker's box, ``partner`` the peer's rank in the union partition or
    ``"self"`` when the peer is this very worker; ``(None, None, None)`` for an
    empty overlap.
    """
    mine = tuple(int(i) for i in my_index)
    lo, hi = my_start_table[mine], my_stop_table[mine]
    out = []
    for rank, peer_index in enumerate(range_index(peer_partition_shape)):
        sl = compute_subtensor_intersection_slice(lo, hi, peer_start_table[peer_index], peer_stop_table[peer_index])
        if sl is None:
            out.append((None, None, None))
            continue
        if self_index is not None and np.all(np.asarray(peer_index) == np.asarray(self_index)):
            partner = "self"
        else:
            partner = int(np.where(peer_union_ranks == rank)[0][0])
        out.append((sl, compute_nd_slice_shape(sl), partner))
    return out


def _ranks_within(P_union, P):
    """For every worker of the union, its rank in ``P`` or -1 (what the
    reference all-gathers, nn/repartition.py:121-128)."""
    group = P._ranks if P._ranks is not None else ()
    return np.array([group.index(w) if w in group else -1 for w in P_union._ranks], dtype=int)


class Repartition(Module):
    """Moves a tensor from partition ``P_x`` to partition ``P_y`` without
    changing its values (a generalised all-to-all).

    Parameters as in the reference: ``P_x``, ``P_y``, ``preserve_batch=True``
    (keep the batch size of zero-volume outputs) and an optional
    ``buffer_manager`` shared with other layers.
    """

    def __init__(self, P_x, P_y, preserve_batch=True, buffer_manager=None):
        super().__init__()
        self.global_input_tensor_structure = TensorStructure()
        self.input_tensor_structure = TensorStructure()
        self.output_tensor_structure = TensorStructure()
        self.P_x = P_x
        self.P_y = P_y
        self.preserve_batch = preserve_batch
        self.P_x_to_y_overlaps = []
        self.P_y_to_x_overlaps = []

        if buffer_manager is None:
            buffer_manager = self._distdl_backend.BufferManager()
        elif not isinstance(buffer_manager, self._distdl_backend.BufferManager):
            raise ValueError("Buffer manager type does not match backend.")
        self.buffer_manager = buffer_manager
        self.P_x_to_y_buffers = None
        self.P_y_to_x_buffers = None

        self._distdl_is_setup = False
        self._input_tensor_structure = TensorStructure()

        P_union = self._distdl_backend.Partition()
        if P_x.active or P_y.active:
            P_union = P_x.create_partition_union(P_y, initialize_backend_comm=True)
        self.P_union = P_union

        self.P_x_shape = None
        self.P_y_shape = None
        self.union_indices = None
        if not P_union.active:
            return

        # Partition shapes survive on workers outside the partition, so no
        # exchange is needed to know them (the reference broadcasts them,
        # nn/repartition.py:103-113).
        self.P_x_shape = np.asarray(P_x.shape).astype(int)
        self.P_y_shape = np.asarray(P_y.shape).astype(int)
        if len(self.P_x_shape) != len(self.P_y_shape):
            raise ValueError("Input and output partition must be same dimension.")

        self.P_x_ranks = _ranks_within(P_union, P_x)
        self.P_y_ranks = _ranks_within(P_union, P_y)
        self.allocate_repartition_buffers = self._distdl_backend.buffer_allocator.allocate_repartition_buffers

    def extra_repr(self) -> str:
        return f'P_x.shape={self.P_x.shape}, P_y.shape={self.P_y.shape}'

    def _distdl_module_setup(self, input):
        """Builds the send / receive overlap lists and their buffers for the
        structure of ``input[0]`` (reference nn/repartition.py:135-295)."""
        self._distdl_is_setup = True
        self._input_tensor_structure.fill_from_tensor(input[0])
        if not self.P_union.active:
            return

        backend = self._distdl_backend
        self.input_tensor_structure = TensorStructure(input[0])
        if self.P_x.active and len(input[0].shape) != len(self.P_x_shape):
            raise ValueError(f"Input partition mush have same dimension "
                             f"({len(self.P_x_shape)}) as input tensor rank ({len(input[0].shape)}).")
        self.global_input_tensor_structure = backend.assemble_global_tensor_structure(
            self.input_tensor_structure, self.P_x, self.P_union)
        x_global_shape = np.asarray(self.global_input_tensor_structure.shape).astype(int)

        if self.P_y.active:
            self.output_tensor_structure.shape = compute_subshape(self.P_y.shape, self.P_y.index, x_global_shape)

        tensor_dim = len(x_global_shape)
        if len(self.P_x_shape) != tensor_dim:
            raise ValueError(f"Input partition mush have same dimension "
                             f"({len(self.P_x_shape)}) as input tensor rank ({tensor_dim}).")
        if len(self.P_y_shape) != tensor_dim:
            raise ValueError(f"Output partition mush have same dimension "
                             f"({len(self.P_y_shape)}) as input tensor rank ({tensor_dim}).")
        if 1 in x_global_shape[x_global_shape != self.P_y_shape]:
            raise ValueError(f"Input tensor must not be size 1 "
                             f"({x_global_shape}) in a dimension where "
                             f"output partition is other than 1 ({self.P_y_shape}).")

        # Input shards may be unbalanced, so their shapes are collected; output
        # shards are balanced by construction.
        x_shapes = backend.tensor_decomposition.compute_subtensor_shapes_unbalanced(
            self.input_tensor_structure, self.P_x, self.P_union)
        y_shapes = compute_subtensor_shapes_balanced(self.global_input_tensor_structure, self.P_y_shape)
        x_lo, x_hi = compute_subtensor_start_indices(x_shapes), compute_subtensor_stop_indices(x_shapes)
        y_lo, y_hi = compute_subtensor_start_indices(y_shapes), compute_subtensor_stop_indices(y_shapes)

        OverlapList = backend.functional.repartition.OverlapList
        self.P_x_to_y_overlaps = OverlapList()
        self.P_y_to_x_overlaps = OverlapList()
        if self.P_x.active:
            self.P_x_to_y_overlaps.extend(compute_overlaps(
                self.P_x.index, x_lo, x_hi, self.P_y_shape, y_lo, y_hi,
                self.P_y.index if self.P_y.active else None, self.P_y_ranks))
        if self.P_y.active:
            self.P_y_to_x_overlaps.extend(compute_overlaps(
                self.P_y.index, y_lo, y_hi, self.P_x_shape, x_lo, x_hi,
                self.P_x.index if self.P_x.active else None, self.P_x_ranks))

        buffs = self.allocate_repartition_buffers(self.buffer_manager,
                                                  self.P_x_to_y_overlaps,
                                                  self.P_y_to_x_overlaps,
                                                  self.global_input_tensor_structure.dtype)
        self.P_x_to_y_buffers, self.P_y_to_x_buffers = buffs

    def _distdl_module_teardown(self, input):
        self.P_x_to_y_overlaps = []
        self.P_y_to_x_overlaps = []
        self.P_x_to_y_buffers = None
        self.P_y_to_x_buffers = None
        self._distdl_is_setup = False
        self._input_tensor_structure = TensorStructure()

    def _distdl_input_changed(self, input):
        return self._input_tensor_structure != TensorStructure(input[0])

    def forward(self, input):
        Function = self._distdl_backend.functional.repartition.RepartitionFunction
        if not (self.P_x.active or self.P_y.active):
            return input
        return Function.apply(input,
                              self.P_union,
                              self.global_input_tensor_structure,
                              self.input_tensor_structure,
                              self.output_tensor_structure,
                              self.P_x,
                              self.P_x_to_y_overlaps,
                              self.P_x_to_y_buffers,
                              self.P_y,
                              self.P_y_to_x_overlaps,
                              self.P_y_to_x_buffers,
                              self.preserve_batch)
