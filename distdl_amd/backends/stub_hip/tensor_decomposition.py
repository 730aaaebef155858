"""Shape table of a partition whose shards need not be balanced (reference:
backends/common/tensor_decomposition.py:4-53)."""


def compute_subtensor_shapes_unbalanced(local_tensor_structure, P_in, P_out=None):
    shapes = None
    if P_in.active:
        shapes = P_in._world.transport.subtensor_shapes(P_in, local_tensor_structure.shape)
    if P_out is not None and P_out.active:
        shapes = P_out.broadcast_data(shapes, P_data=P_in)
    return shapes
