"""ORACLE -- test infrastructure, not product code.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import it.

Scalar restatement of the reference's balanced-partition arithmetic, written
with plain Python integers so that it shares no code (and no vectorisation
trick) with ``distdl_amd.utilities``:

  subshape / start / stop   utilities/slicing.py:8-51
  shape and index tables    utilities/tensor_decomposition.py:8-133
  box intersection          utilities/slicing.py:54-62,
                            utilities/tensor_decomposition.py:136-190

Pinned by tests/test_oracle_golden.py against the reference's own known
answers (tests/utilities/test_buffer.py:171-190, :276-281;
examples/primitives/ex_repartition.py:51-124), against brute force over every
element of small tensors, and against the tiling invariant (the boxes of a
partition are disjoint and cover the tensor).
"""

import itertools


def subshape_1d(P, i, n):
    """Extent of block ``i`` of ``n`` elements over ``P`` workers."""
    return n // P + (1 if i < n % P else 0)


def start_1d(P, i, n):
    return (n // P) * i + min(i, n % P)


def subshape(P_shape, index, shape):
    return [subshape_1d(P, i, n) for P, i, n in zip(P_shape, index, shape)]


def start_index(P_shape, index, shape):
    return [start_1d(P, i, n) for P, i, n in zip(P_shape, index, shape)]


def stop_index(P_shape, index, shape):
    return [a + b for a, b in zip(start_index(P_shape, index, shape), subshape(P_shape, index, shape))]


def indices(P_shape):
    """Row-major Cartesian indices of a partition (utilities/slicing.py:137-160)."""
    return list(itertools.product(*[range(int(p)) for p in P_shape]))


def boxes_balanced(P_shape, shape):
    """{index: (start, stop)} of every worker's block under a balanced split."""
    return {idx: (start_index(P_shape, idx, shape), stop_index(P_shape, idx, shape)) for idx in indices(P_shape)}


def boxes_from_shapes(P_shape, shapes):
    """{index: (start, stop)} from explicit (possibly unbalanced) per-worker
    shapes: the start along a dimension is the sum of the extents of the
    workers before it on that axis (utilities/tensor_decomposition.py:52-133)."""
    out = {}
    for idx in indices(P_shape):
        lo = []
        for d in range(len(P_shape)):
            acc = 0
            for i in range(idx[d]):
                probe = list(idx)
                probe[d] = i
                acc += shapes[tuple(probe)][d]
            lo.append(acc)
        out[idx] = (lo, [a + b for a, b in zip(lo, shapes[idx])])
    return out


def intersect(lo0, hi0, lo1, hi1):
    """Overlap of box 0 with box 1 as ``(start, stop)`` relative to box 0, or
    ``None`` when it is empty."""
    lo = [max(a, b) for a, b in zip(lo0, lo1)]
    hi = [min(a, b) for a, b in zip(hi0, hi1)]
    if any(h <= l for l, h in zip(lo, hi)):
        return None
    return [l - o for l, o in zip(lo, lo0)], [h - o for h, o in zip(hi, lo0)]


def as_slices(lo, hi):
    return tuple(slice(int(a), int(b)) for a, b in zip(lo, hi))
