"""CPU restatement of the local re-layouts of AllGather and ReduceScatter.

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py, never by the product.

Reference (paths under src/distdl/):
  backends/mpi_numpy/functional/all_gather.py:88-149   forward (zero-pad, gather, `p a b c -> a (p b) c`, strip)
  backends/mpi_numpy/functional/all_gather.py:185-250  adjoint (divide by scale_backward, reduce-scatter)
  backends/mpi_numpy/functional/reduce_scatter.py:86-143  forward (split, zero-pad, MPI.SUM, strip)
  backends/mpi_numpy/functional/reduce_scatter.py:176-240 adjoint (all-gather)
  utilities/slicing.py:240-275  get_rearrange_ordering (the gather axis moved to the front / merged back)

All workers of the team are simulated at once: functions take the list of the
workers' tensors in rank order and return the list of what each ends up with.

What the reference leaves open: MPI.SUM does not fix the order of the
additions.  This restatement adds in rank order with a rounding to the element
type after every addition; on data whose sums are exact (small integers) every
order gives the same bits, and that is what the parity tests use.

Pinned by tests/test_oracle_golden.py without running the reference (its own
tests of these layers, tests/primitives/test_all_gather.py and
test_reduce_scatter.py, hold no fixtures: they check adjoint consistency only):
the closed form (a gather of a balanced split is the tensor, a reduce-scatter of
P copies of it is P times the split), an element-by-element brute force on
small uneven cases, and the adjoint identity <A x, y> = <x, A* y> on integers.
"""
import numpy as np


def shard_extents(n, P):
    """Extents of the P shards of an axis of length n: n // P, the first n % P
    one larger (reduce_scatter.py:96-101, the balanced split of slicing.py:8-16)."""
    base, rem = divmod(int(n), int(P))
    return [base + (1 if r < rem else 0) for r in range(P)]


def _pad_one(a, axis):
    pad = [(0, 0)] * a.ndim
    pad[axis] = (0, 1)
    return np.pad(a, pad, mode="constant", constant_values=0)


def _strip_one(a, axis):
    sl = [slice(None)] * a.ndim
    sl[axis] = slice(0, -1)
    return a[tuple(sl)]


def all_gather(parts, axis):
    """parts[r]: worker r's shard, extents along `axis` as shard_extents gives
    them.  Returns the gathered tensor (every worker receives the same one).

    Follows all_gather.py:88-149: workers r >= remainder zero-pad their shard by
    one along the axis so that all messages have one size (:90-96); Iallgather
    concatenates them in rank order into [P, *padded_shape] (:103-123); the
    padding is cut off the pieces of workers r >= remainder and the pieces are
    joined along the axis, `p a b c -> a (p b) c` (:125-147)."""
    P = len(parts)
    n = sum(p.shape[axis] for p in parts)
    remainder = n % P
    if [p.shape[axis] for p in parts] != shard_extents(n, P):
        raise ValueError("all_gather: shards are not the balanced split of their total")
    padded = [_pad_one(p, axis) if remainder and r >= remainder else p for r, p in enumerate(parts)]
    gathered = np.stack(padded)                                   # p a b c
    pieces = [(_strip_one(gathered[r], axis) if remainder and r >= remainder else gathered[r]) for r in range(P)]
    return np.concatenate(pieces, axis=axis)


def _sum_in_rank_order(arrays):
    acc = arrays[0].copy()
    for a in arrays[1:]:
        acc = (acc + a).astype(arrays[0].dtype)
    return acc


def reduce_scatter(fulls, axis):
    """fulls[r]: worker r's tensor (all of one shape).  Returns the list of what
    each worker receives: its slab, along `axis`, of the sum over the workers.

    Follows reduce_scatter.py:86-143: the tensor is split into P slabs of
    shard_extents (:96-101), each moved to `p a b c` with p = 1 (:103-105), the
    slabs of workers r >= remainder zero-padded by one along the axis (:107-112),
    all joined and flattened (:115); Ireduce_scatter with MPI.SUM hands worker r
    the sum of the r-th equal chunk (:127-128), which is reshaped to the padded
    slab shape (:118-121) and stripped of the padding again (:138-143)."""
    P = len(fulls)
    n = fulls[0].shape[axis]
    remainder = n % P
    extents = shard_extents(n, P)
    starts = np.concatenate([[0], np.cumsum(extents)])
    flat = []
    for full in fulls:
        slabs = []
        for r in range(P):
            sl = [slice(None)] * full.ndim
            sl[axis] = slice(int(starts[r]), int(starts[r + 1]))
            slab = full[tuple(sl)]
            if remainder and r >= remainder:
                slab = _pad_one(slab, axis)
            slabs.append(slab.reshape(-1))
        flat.append(np.concatenate(slabs))
    chunk = flat[0].size // P
    out = []
    for r in range(P):
        summed = _sum_in_rank_order([f[r * chunk:(r + 1) * chunk] for f in flat])
        shape = list(fulls[0].shape)
        shape[axis] = extents[r] + (1 if remainder and r >= remainder else 0)
        slab = summed.reshape(shape)
        out.append(_strip_one(slab, axis) if remainder and r >= remainder else slab)
    return out


def all_gather_adjoint(grads, axis, scale_backward=None):
    """Adjoint of all_gather (all_gather.py:185-250): every worker's gradient of
    the gathered tensor is divided by scale_backward (:192-193) and the quotients
    are reduce-scattered.  grads[r]: worker r's gradient; returns the list of
    shard gradients."""
    if scale_backward is not None:
        grads = [(g / scale_backward).astype(g.dtype) for g in grads]
    return reduce_scatter(grads, axis)


def reduce_scatter_adjoint(grads, axis):
    """Adjoint of reduce_scatter (reduce_scatter.py:176-240): the all-gather of
    the workers' slab gradients; returns the list of what each worker receives
    (the same tensor for all)."""
    full = all_gather(grads, axis)
    return [full.copy() for _ in grads]
