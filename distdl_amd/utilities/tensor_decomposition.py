"""Per-worker shape / start / stop tables of a partitioned tensor.

Counterpart of the reference's ``utilities/tensor_decomposition.py``.  A table
for a D-dimensional tensor over a partition of shape ``P`` is an integer array of
shape ``P + (D,)``: entry ``[i_0, ..., i_{D-1}, d]`` is the value for dimension
``d`` of the worker at Cartesian index ``(i_0, ..., i_{D-1})``.
"""

import numpy as np

from .slicing import assemble_slices
from .slicing import compute_intersection


def compute_subtensor_shapes_balanced(global_tensor_structure, P_tensor_shape):
    """Shape table of a perfectly balanced decomposition
    (utilities/tensor_decomposition.py:8-49)."""
    P = np.atleast_1d(P_tensor_shape).astype(int)
    n = np.atleast_1d(global_tensor_structure.shape).astype(int)
    D = len(P)
    table = np.zeros(list(P) + [D], dtype=int)
    for d in range(D):
        # Along dimension d the extent depends on the worker's d-th index only.
        per_index = n[d] // P[d] + (np.arange(P[d]) < n[d] % P[d]).astype(int)
        view = [1] * D
        view[d] = P[d]
        table[..., d] = per_index.reshape(view)
    return table


def compute_subtensor_stop_indices(shapes):
    """Stop (exclusive) global index table: running sum of the extents along
    each partition dimension (utilities/tensor_decomposition.py:103-133)."""
    D = shapes.ndim - 1
    stops = np.empty_like(shapes)
    for d in range(D):
        stops[..., d] = np.cumsum(shapes[..., d], axis=d)
    return stops


def compute_subtensor_start_indices(shapes):
    """Start global index table: the previous worker's stop, zero for the first
    (utilities/tensor_decomposition.py:52-100)."""
    return compute_subtensor_stop_indices(shapes) - shapes


def compute_subtensor_intersection_slice(x_start_index, x_stop_index, y_start_index, y_stop_index):
    """Overlap of box x with box y as slices relative to x, ``None`` if empty
    (utilities/tensor_decomposition.py:136-190)."""
    bounds = [np.atleast_1d(v) for v in (x_start_index, x_stop_index, y_start_index, y_stop_index)]
    if any(b.ndim != 1 for b in bounds):
        raise ValueError("Index lists must be convertible to 1-dimensional arrays.")
    x_lo, x_hi, y_lo, y_hi = bounds
    lo, _, extent = compute_intersection(x_lo, x_hi, y_lo, y_hi)
    if np.prod(extent) == 0:
        return None
    rel = lo - x_lo
    return assemble_slices(rel, rel + extent)
