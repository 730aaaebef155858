"""ORACLE -- test infrastructure, not product code.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import it.

NumPy restatement of the reference's Repartition:

  overlap lists   nn/repartition.py:135-295 (send side :218-253, receive :257-288)
  forward         backends/mpi_numpy/functional/repartition.py:142-213
                  (pack np.copyto :164, zeros :176-177, self copy :179-190,
                  unpack np.copyto :206)
  adjoint         same file :285-355 (lists swapped, copies not adds)

Workers are identified by their row-major rank inside their own partition; the
wire is a dict keyed by (source rank, destination rank).  bf16 payloads are
handled as uint16 bit patterns: the reference's CPU backend has no bf16 mapping
(utilities/dtype.py:54,61-73) and the operation is a pure move.

Pinned by: ex_repartition.py forward and adjoint matrices; identity
repartition has only self overlaps (tests/primitives/test_repartition.py:643-647);
scatter-then-gather returns the global tensor; element-by-element brute force
over the global index space.
"""

import numpy as np

from . import partition_math as pm


def overlaps(my_box, peer_boxes, peer_order, same_worker):
    """Overlap of ``my_box`` with each peer box in row-major peer order.
    Returns [(slices rel. to my box, shape, peer rank or "self")] with
    (None, None, None) for empty overlaps."""
    out = []
    for rank, idx in enumerate(peer_order):
        hit = pm.intersect(my_box[0], my_box[1], peer_boxes[idx][0], peer_boxes[idx][1])
        if hit is None:
            out.append((None, None, None))
            continue
        lo, hi = hit
        out.append((pm.as_slices(lo, hi), tuple(h - l for l, h in zip(lo, hi)), "self" if same_worker(rank) else rank))
    return out


def plan(global_shape, P_x_shape, P_y_shape, x_shapes=None, shared_workers=True):
    """Send and receive overlap lists of every worker.

    ``shared_workers``: x rank r and y rank r are the same process (the two
    partitions are laid over the same team), so that pair's overlap is a self
    copy.  Returns (send[x_rank], recv[y_rank], x_boxes, y_boxes)."""
    x_order, y_order = pm.indices(P_x_shape), pm.indices(P_y_shape)
    x_boxes = pm.boxes_balanced(P_x_shape, global_shape) if x_shapes is None else pm.boxes_from_shapes(P_x_shape, x_shapes)
    y_boxes = pm.boxes_balanced(P_y_shape, global_shape)
    send, recv = [], []
    for xr, xi in enumerate(x_order):
        send.append(overlaps(x_boxes[xi], y_boxes, y_order, lambda r, xr=xr: shared_workers and r == xr))
    for yr, yi in enumerate(y_order):
        recv.append(overlaps(y_boxes[yi], x_boxes, x_order, lambda r, yr=yr: shared_workers and r == yr))
    return send, recv, x_boxes, y_boxes


def pack(x_local, send_list):
    """One contiguous buffer per non-self overlap: np.copyto(buf, x[sl])."""
    bufs = []
    for sl, sh, partner in send_list:
        if sl is None or partner == "self":
            bufs.append(None)
            continue
        buf = np.empty(sh, dtype=x_local.dtype)
        np.copyto(buf, x_local[sl])
        bufs.append(buf)
    return bufs


def unpack(recv_list, bufs, y_shape, dtype, x_local=None, send_list=None):
    """zeros -> self copy -> np.copyto(y[sl], buf) for every received buffer."""
    y = np.zeros(y_shape, dtype=dtype)
    if x_local is not None and send_list is not None:
        src = [sl for sl, sh, p in send_list if p == "self"]
        dst = [sl for sl, sh, p in recv_list if p == "self"]
        if src and dst:
            np.copyto(y[dst[0]], x_local[src[0]])
    for (sl, sh, partner), buf in zip(recv_list, bufs):
        if sl is None or partner == "self" or buf is None:
            continue
        np.copyto(y[sl], buf)
    return y


def forward_all(x_locals, global_shape, P_x_shape, P_y_shape, x_shapes=None, shared_workers=True):
    """Every worker's output shard, moving data through an in-memory wire."""
    send, recv, x_boxes, y_boxes = plan(global_shape, P_x_shape, P_y_shape, x_shapes, shared_workers)
    wire = {}
    for xr, x in enumerate(x_locals):
        for (sl, sh, partner), buf in zip(send[xr], pack(x, send[xr])):
            if buf is not None:
                wire[(xr, partner)] = buf
    outs = []
    y_order = pm.indices(P_y_shape)
    for yr, yi in enumerate(y_order):
        lo, hi = y_boxes[yi]
        bufs = [None if (sl is None or p == "self") else wire[(p, yr)] for sl, sh, p in recv[yr]]
        has_self = shared_workers and yr < len(x_locals)
        outs.append(unpack(recv[yr], bufs, tuple(h - l for l, h in zip(lo, hi)), x_locals[0].dtype,
                           x_locals[yr] if has_self else None, send[yr] if has_self else None))
    return outs


def adjoint_all(dy_locals, global_shape, P_x_shape, P_y_shape, x_shapes=None, shared_workers=True):
    """Adjoint: the same movement from P_y back to P_x with the lists swapped."""
    send, recv, x_boxes, y_boxes = plan(global_shape, P_x_shape, P_y_shape, x_shapes, shared_workers)
    wire = {}
    for yr, dy in enumerate(dy_locals):
        for (sl, sh, partner), buf in zip(recv[yr], pack(dy, recv[yr])):
            if buf is not None:
                wire[(yr, partner)] = buf
    outs = []
    x_order = pm.indices(P_x_shape)
    for xr, xi in enumerate(x_order):
        lo, hi = x_boxes[xi]
        bufs = [None if (sl is None or p == "self") else wire[(p, xr)] for sl, sh, p in send[xr]]
        has_self = shared_workers and xr < len(dy_locals)
        outs.append(unpack(send[xr], bufs, tuple(h - l for l, h in zip(lo, hi)), dy_locals[0].dtype,
                           dy_locals[xr] if has_self else None, recv[xr] if has_self else None))
    return outs


def scatter(global_x, P_shape):
    """Balanced shards of a global array, in row-major rank order."""
    boxes = pm.boxes_balanced(P_shape, global_x.shape)
    return [np.ascontiguousarray(global_x[pm.as_slices(*boxes[idx])]) for idx in pm.indices(P_shape)]
