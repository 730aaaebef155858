"""Tensor metadata shared between workers (reference:
backends/common/tensor_comm.py:11-188).  The reference moves these few integers
with MPI collectives; here the shape table of the partition comes from the
world's transport and everything else is local."""

import numpy as np
import torch

from ...utilities.torch import TensorStructure


def _as_structure(local):
    if isinstance(local, TensorStructure):
        return local
    return TensorStructure(local)


def assemble_global_tensor_structure(local_tensor_structure, P_in, P_out=None):
    """Global shape = per dimension, the sum of the shard extents along that
    dimension of the partition (reference :98-148)."""
    local = _as_structure(local_tensor_structure)
    out = TensorStructure()
    if P_in.active:
        table = P_in._world.transport.subtensor_shapes(P_in, local.shape)
        shape = np.zeros(P_in.dim, dtype=int)
        for d in range(P_in.dim):
            line = [0] * P_in.dim + [d]
            line[d] = slice(None)
            shape[d] = int(np.sum(table[tuple(line)]))
        out.shape = shape
        out.dtype = local.dtype
        out.requires_grad = local.requires_grad
    if P_out is not None and P_out.active:
        payload = (out.shape, out.dtype, out.requires_grad) if P_in.active else None
        shape, dtype, rg = P_out.broadcast_data(payload, P_data=P_in)
        out.shape, out.dtype, out.requires_grad = np.asarray(shape, dtype=int), dtype, bool(rg)
    return out


def assemble_global_tensor_structure_along_axis(local_tensor_structure, P_x, axis):
    """As above, summing only along ``axis`` (reference :151-188)."""
    local = _as_structure(local_tensor_structure)
    out = TensorStructure()
    if P_x.active:
        axis = np.atleast_1d(axis)
        table = P_x._world.transport.subtensor_shapes(P_x, local.shape)
        shape = [int(s) for s in local.shape]
        a = int(axis[0])
        line = [int(i) for i in P_x.index] + [a]
        line[a] = slice(None)
        shape[a] = int(np.sum(table[tuple(line)]))
        out.shape = torch.Size(shape)
        out.dtype = local.dtype
        out.requires_grad = local.requires_grad
    return out


def broadcast_tensor_structure(input_tensor_structure, P_send, P_recv):
    """Structure of the sender's tensor on every receiver (reference :11-95)."""
    out = TensorStructure()
    if not P_send.active and not P_recv.active:
        return out
    if P_send.active and (P_send == P_recv or not P_recv.active):
        src = input_tensor_structure
        out.shape, out.dtype, out.requires_grad = src.shape, src.dtype, src.requires_grad
        if P_send == P_recv:
            return out
    union = P_send.create_partition_union(P_recv)
    payload = None
    if P_send.active:
        s = input_tensor_structure
        payload = (tuple(int(v) for v in s.shape), s.dtype, bool(s.requires_grad))
    shape, dtype, rg = union.broadcast_data(payload, P_data=P_send)
    if P_recv.active and not P_send.active:
        out.shape, out.dtype, out.requires_grad = torch.Size(shape), dtype, rg
    return out
