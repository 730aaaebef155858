"""Integer geometry of balanced Cartesian tensor partitions.

Host-side counterpart of the reference's ``utilities/slicing.py``: the same
function names and results (reference lines are cited per function), written as
plain vectorised integer arithmetic.  Everything here runs once per input
structure, where the reference's forward pre-hook runs it; the results feed the
box descriptors of the HIP copy kernels.
"""

import itertools

import numpy as np

INDEX_DTYPE = np.int64
MAX_INT = np.iinfo(INDEX_DTYPE).max
MIN_INT = np.iinfo(INDEX_DTYPE).min


def _ivec(v):
    return np.atleast_1d(np.asarray(v)).astype(INDEX_DTYPE)


def compute_subshape(P_shape, index, shape):
    """Extent of worker ``index``'s block: ``shape // P`` everywhere and one more
    for the first ``shape % P`` workers of each dimension (utilities/slicing.py:8-16)."""
    P, i, n = _ivec(P_shape), _ivec(index), _ivec(shape)
    return n // P + (i < n % P).astype(INDEX_DTYPE)


def compute_subshape_along_axis(P_shape, index, shape, axis):
    """As :func:`compute_subshape`, but only ``axis`` is divided (utilities/slicing.py:19-31)."""
    P, i, n = _ivec(P_shape), _ivec(index), _ivec(shape)
    out = n.copy()
    for a in np.atleast_1d(axis):
        out[a] = n[a] // P[a] + (1 if i[a] < n[a] % P[a] else 0)
    return out


def compute_start_index(P_shape, index, shape):
    """First global index owned by worker ``index`` (utilities/slicing.py:34-42):
    ``(shape // P) * index + min(index, shape % P)``."""
    P, i, n = _ivec(P_shape), _ivec(index), _ivec(shape)
    return (n // P) * i + np.minimum(i, n % P)


def compute_stop_index(P_shape, index, shape):
    """One past the last global index owned by worker ``index`` (utilities/slicing.py:45-51)."""
    return compute_start_index(P_shape, index, shape) + compute_subshape(P_shape, index, shape)


def compute_intersection(r0_start_index, r0_stop_index, r1_start_index, r1_stop_index):
    """Overlap of two index boxes: (start, stop, shape), shape clamped at zero
    (utilities/slicing.py:54-62)."""
    lo = np.maximum(r0_start_index, r1_start_index)
    hi = np.minimum(r0_stop_index, r1_stop_index)
    return lo, hi, np.maximum(hi - lo, 0)


def assemble_slices(start_index, stop_index):
    """Tuple of ``slice(start, stop)`` per dimension (utilities/slicing.py:65-72)."""
    return tuple(slice(a, b, None) for a, b in zip(start_index, stop_index))


def compute_partition_intersection(P_x_r_shape, P_x_r_index, P_x_s_shape, P_x_s_index, x_shape):
    """Overlap of two workers' blocks of one global tensor under two balanced
    partitions, as slices relative to the first block; ``None`` when empty
    (utilities/slicing.py:75-108)."""
    r_lo = compute_start_index(P_x_r_shape, P_x_r_index, x_shape)
    r_hi = compute_stop_index(P_x_r_shape, P_x_r_index, x_shape)
    s_lo = compute_start_index(P_x_s_shape, P_x_s_index, x_shape)
    s_hi = compute_stop_index(P_x_s_shape, P_x_s_index, x_shape)
    lo, _, extent = compute_intersection(r_lo, r_hi, s_lo, s_hi)
    if np.prod(extent) == 0:
        return None
    rel = lo - r_lo
    return assemble_slices(rel, rel + extent)


def compute_nd_slice_volume(slices):
    """Number of elements a tuple of slices selects (utilities/slicing.py:111-113)."""
    return np.prod([s.stop - s.start for s in slices])


def compute_nd_slice_shape(slices):
    """Shape a tuple of slices selects (utilities/slicing.py:116-134)."""
    return tuple(s.stop - s.start for s in slices)


def range_index(shape):
    """Cartesian indices of a partition of the given shape in row-major order,
    last index fastest (utilities/slicing.py:137-160)."""
    return itertools.product(*(range(int(n)) for n in shape))


def worker_layout(shape):
    """Array of the given shape holding each worker's row-major rank
    (utilities/slicing.py:163-171)."""
    shape = [int(n) for n in np.atleast_1d(shape)]
    return np.arange(int(np.prod(shape)), dtype=int).reshape(shape)


def filtered_range_index(shape, filter):
    """Cartesian indices matching ``filter`` where it is not ``None``
    (utilities/slicing.py:174-205)."""
    for idx in range_index(shape):
        if all(f is None or i == f for i, f in zip(idx, filter)):
            yield idx


def assemble_index_filter(index, dims, invert=False):
    """Filter keeping ``index`` in ``dims`` (or outside them when ``invert``)
    and ``None`` elsewhere (utilities/slicing.py:208-243)."""
    return tuple(index[k] if ((k in dims) != invert) else None for k in range(len(index)))
