"""ORACLE -- test infrastructure, not product code.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import it.

NumPy restatement of the reference's halo machinery:

  halo widths      nn/mixins/halo_mixin.py:9-207 with the kernel ranges of
                   nn/mixins/conv_mixin.py:34-91 (scalar, one dimension at a time)
  explicit padding nn/conv_feature.py:367-377, :399-407 (np.pad constant 0)
  slab slices      nn/halo_exchange.py:37-99
  forward          backends/mpi_numpy/functional/halo_exchange.py:30-76
  adjoint          same file :100-142

Pinned by: the kernel-2 / stride-2 table of tests/utilities/test_halo_mixin.py:46-87;
the forward and adjoint matrices of examples/primitives/ex_halo_exchange.py:67-140;
brute force (the set of input indices a worker's outputs read, enumerated);
pad -> exchange -> crop -> torch conv equals the sequential torch conv on the
geometries of tests/layers/test_conv_feature.py:9-247.
"""

import numpy as np

from . import partition_math as pm


# ------------------------------------------------------------------ widths --

def out_extent(n, k, s, p, d):
    return (n + 2 * p - d * (k - 1) - 1) // s + 1


def halo_1d(P, i, n, k, s, p, d, x_start=None, x_len=None, nonneg=True):
    """(left, right) halo of worker ``i`` along one dimension."""
    if x_start is None:
        x_start, x_len = pm.start_1d(P, i, n), pm.subshape_1d(P, i, n)
    ny = out_extent(n, k, s, p, d)
    y_start, y_len = pm.start_1d(P, i, ny), pm.subshape_1d(P, i, ny)
    need_lo = max(0, s * y_start - p)
    need_hi = min(n - 1, s * (y_start + y_len - 1) + d * (k - 1) - p)
    left = x_start - need_lo
    right = need_hi - (x_start + x_len - 1)
    if nonneg:
        left, right = max(left, 0), max(right, 0)
    return left, right


def exchange_info(global_shape, kernel, stride, padding, dilation, P_shape, index, shapes=None):
    """halo, recv, send, needed ranges ([dim][2] lists) of the worker at
    ``index``.  Window parameters are right-aligned with the tensor dimensions
    (missing leading ones are kernel 1 / stride 1 / padding 0 / dilation 1).
    ``shapes``: optional {index: local shape} for unbalanced shards."""
    nd = len(global_shape)

    def lead(v, fill):
        v = list(np.atleast_1d(v))
        return [fill] * (nd - len(v)) + [int(a) for a in v]

    k, s, p, dl = lead(kernel, 1), lead(stride, 1), lead(padding, 0), lead(dilation, 1)

    def local_box(idx, dim):
        if shapes is None:
            return None, None
        start = 0
        for i in range(idx[dim]):
            probe = [0] * nd
            probe[dim] = i
            start += shapes[tuple(probe)][dim]
        return start, shapes[tuple(idx)][dim]

    def halo_of(idx, nonneg=True):
        out = []
        for dim in range(nd):
            xs, xl = local_box(idx, dim)
            out.append(list(halo_1d(P_shape[dim], idx[dim], global_shape[dim], k[dim], s[dim], p[dim], dl[dim],
                                    xs, xl, nonneg)))
        return out

    index = [int(i) for i in index]
    halo = halo_of(index)
    recv = [list(h) for h in halo]
    send = [[0, 0] for _ in range(nd)]
    for dim in range(nd):
        if index[dim] - 1 >= 0:
            nb = list(index)
            nb[dim] -= 1
            send[dim][0] = halo_of(nb)[dim][1]
        if index[dim] + 1 < P_shape[dim]:
            nb = list(index)
            nb[dim] += 1
            send[dim][1] = halo_of(nb)[dim][0]
    raw = halo_of(index, nonneg=False)
    local = [shapes[tuple(index)][d] if shapes is not None else pm.subshape_1d(P_shape[d], index[d], global_shape[d])
             for d in range(nd)]
    needed = [[-min(0, raw[d][0]), local[d] + max(0, raw[d][0]) + max(0, raw[d][1])] for d in range(nd)]
    return halo, recv, send, needed


def local_padding(P_shape, index, global_padding):
    """Explicit zero padding only on global-boundary sides."""
    return [[gp if i == 0 else 0, gp if i == P - 1 else 0] for P, i, gp in zip(P_shape, index, global_padding)]


# ------------------------------------------------------------------ slices --

def slab_slices(shape, recv, send):
    """[dim] -> (left bulk, left ghost, right bulk, right ghost) slice tuples."""
    nd = len(shape)
    out = []
    for i in range(nd):
        four = [[], [], [], []]
        for j in range(nd):
            n = shape[j]
            lr, ls, rr, rs = recv[j][0], send[j][0], recv[j][1], send[j][1]
            if j < i:
                four_j = [slice(0, n)] * 4
            elif j == i:
                four_j = [slice(lr, lr + ls), slice(0, lr), slice(n - rr - rs, n - rr), slice(n - rr, n)]
            else:
                four_j = [slice(lr, n - rr)] * 4
            for q in range(4):
                four[q].append(four_j[q])
        out.append([tuple(f) for f in four])
    return out


def _shape_of(sl):
    return tuple(s.stop - s.start for s in sl)


# ---------------------------------------------------------------- one rank --

def pad_exchange_single(x, pad, recv, send, ghost_bufs):
    """What one worker ends up with when its neighbours deliver ``ghost_bufs``
    ([dim][side] arrays or None): np.pad, then per dimension pack the bulk slabs
    and unpack the ghosts.  Returns (exchanged tensor, bulk slabs [dim][side])."""
    out = np.pad(x, [(int(a), int(b)) for a, b in pad], mode="constant", constant_values=0)
    slices = slab_slices(out.shape, recv, send)
    bulks = []
    for i in range(x.ndim):
        lbs, lgs, rbs, rgs = slices[i]
        lb = np.ascontiguousarray(out[lbs]) if send[i][0] > 0 else None
        rb = np.ascontiguousarray(out[rbs]) if send[i][1] > 0 else None
        bulks.append([lb, rb])
        if recv[i][0] > 0:
            out[lgs] = ghost_bufs[i][0].reshape(_shape_of(lgs))
        if recv[i][1] > 0:
            out[rgs] = ghost_bufs[i][1].reshape(_shape_of(rgs))
    return out, bulks


# --------------------------------------------------------------- all ranks --

def _neighbours(P_shape, idx, dim):
    left = right = None
    if idx[dim] - 1 >= 0:
        nb = list(idx)
        nb[dim] -= 1
        left = tuple(nb)
    if idx[dim] + 1 < P_shape[dim]:
        nb = list(idx)
        nb[dim] += 1
        right = tuple(nb)
    return left, right


def forward_all(padded, P_shape, recv, send):
    """Halo exchange over every worker.  ``padded``/``recv``/``send``: dicts
    keyed by Cartesian index.  Returns new dict of exchanged tensors."""
    out = {idx: a.copy() for idx, a in padded.items()}
    slices = {idx: slab_slices(out[idx].shape, recv[idx], send[idx]) for idx in out}
    for dim in range(len(P_shape)):
        packed = {}
        for idx in out:
            lbs, lgs, rbs, rgs = slices[idx][dim]
            packed[idx] = (np.ascontiguousarray(out[idx][lbs]), np.ascontiguousarray(out[idx][rbs]))
        for idx in out:
            lbs, lgs, rbs, rgs = slices[idx][dim]
            left, right = _neighbours(P_shape, idx, dim)
            if left is not None and recv[idx][dim][0] > 0:
                out[idx][lgs] = packed[left][1].reshape(_shape_of(lgs))
            if right is not None and recv[idx][dim][1] > 0:
                out[idx][rgs] = packed[right][0].reshape(_shape_of(rgs))
    return out


def adjoint_all(grads, P_shape, recv, send):
    """Adjoint over every worker: dimensions reversed, ghosts are sent and
    zeroed, what arrives is added into the bulk."""
    out = {idx: a.copy() for idx, a in grads.items()}
    slices = {idx: slab_slices(out[idx].shape, recv[idx], send[idx]) for idx in out}
    for dim in reversed(range(len(P_shape))):
        packed = {}
        for idx in out:
            lbs, lgs, rbs, rgs = slices[idx][dim]
            packed[idx] = (out[idx][lgs].copy(), out[idx][rgs].copy())
            if recv[idx][dim][0] > 0:
                out[idx][lgs] = 0
            if recv[idx][dim][1] > 0:
                out[idx][rgs] = 0
        for idx in out:
            lbs, lgs, rbs, rgs = slices[idx][dim]
            left, right = _neighbours(P_shape, idx, dim)
            if left is not None and send[idx][dim][0] > 0:
                out[idx][lbs] += packed[left][1].reshape(_shape_of(lbs))
            if right is not None and send[idx][dim][1] > 0:
                out[idx][rbs] += packed[right][0].reshape(_shape_of(rbs))
    return out
