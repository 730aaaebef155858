"""Host-side logic of the package on the CPU: index math against the oracle and
the golden vectors, overlap lists and buffer pools of the layers, the loopback
transport, error behaviour, and the C-ABI surface.  No kernel is launched here."""

import ctypes
import os
import re

import numpy as np
import pytest
import torch

from distdl_amd import _lib
from distdl_amd.backends.stub_hip import BufferManager
from distdl_amd.backends.stub_hip import ExpandableBuffer
from distdl_amd.backends.stub_hip import SimWorld
from distdl_amd.nn import DistributedConv2d
from distdl_amd.nn import DistributedConv3d
from distdl_amd.nn import HaloExchange
from distdl_amd.nn import Repartition
from distdl_amd.nn.halo_exchange import assemble_halo_slices
from distdl_amd.nn.mixins.conv_mixin import ConvMixin
from distdl_amd.nn.mixins.halo_mixin import HaloMixin
from distdl_amd.nn.mixins.pooling_mixin import PoolingMixin
from distdl_amd.utilities import slicing
from distdl_amd.utilities import tensor_decomposition as td
from distdl_amd.utilities.torch import TensorStructure
from distdl_amd.utilities.torch import distdl_padding_to_torch_padding
from distdl_amd.utilities.torch import zero_volume_tensor
from oracle import halo as o_halo
from oracle import partition_math as pm
from oracle import repartition as o_rep

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class MockPoolLayer(HaloMixin, PoolingMixin):
    pass


class MockConvLayer(HaloMixin, ConvMixin):
    pass


# ------------------------------------------------------------- utilities ----

@pytest.mark.parametrize("P_shape,shape", [([4], [10]), ([2, 2], [7, 5]), ([1, 8, 1], [8, 4096, 8192]),
                                          ([3, 1, 5], [2, 9, 11]), ([5], [3])])
def test_slicing_matches_oracle(P_shape, shape):
    class S:
        pass
    S.shape = shape
    table = td.compute_subtensor_shapes_balanced(S, P_shape)
    lo_t, hi_t = td.compute_subtensor_start_indices(table), td.compute_subtensor_stop_indices(table)
    for idx in pm.indices(P_shape):
        assert slicing.compute_subshape(P_shape, idx, shape).tolist() == pm.subshape(P_shape, idx, shape)
        assert slicing.compute_start_index(P_shape, idx, shape).tolist() == pm.start_index(P_shape, idx, shape)
        assert slicing.compute_stop_index(P_shape, idx, shape).tolist() == pm.stop_index(P_shape, idx, shape)
        assert table[idx].tolist() == pm.subshape(P_shape, idx, shape)
        assert lo_t[idx].tolist() == pm.start_index(P_shape, idx, shape)
        assert hi_t[idx].tolist() == pm.stop_index(P_shape, idx, shape)


def test_unbalanced_tables_match_oracle():
    shapes = np.zeros((1, 4, 2), dtype=int)
    for i, n in enumerate([3, 3, 2, 2]):
        shapes[0, i] = [1, n]
    lo, hi = td.compute_subtensor_start_indices(shapes), td.compute_subtensor_stop_indices(shapes)
    boxes = pm.boxes_from_shapes([1, 4], {(0, i): (1, n) for i, n in enumerate([3, 3, 2, 2])})
    for idx, (blo, bhi) in boxes.items():
        assert lo[idx].tolist() == blo and hi[idx].tolist() == bhi


def test_intersection_slices_match_oracle():
    rng = np.random.default_rng(0)
    for _ in range(100):
        lo0, lo1 = rng.integers(0, 6, 3), rng.integers(0, 6, 3)
        hi0, hi1 = lo0 + rng.integers(1, 5, 3), lo1 + rng.integers(1, 5, 3)
        got = td.compute_subtensor_intersection_slice(lo0, hi0, lo1, hi1)
        want = pm.intersect(list(lo0), list(hi0), list(lo1), list(hi1))
        if want is None:
            assert got is None
        else:
            assert [(s.start, s.stop) for s in got] == list(zip(*want))
    with pytest.raises(ValueError):
        td.compute_subtensor_intersection_slice(np.zeros((2, 2)), [1, 1], [0, 0], [1, 1])


def test_small_helpers():
    assert list(slicing.range_index([2, 3])) == [(0, 0), (0, 1), (0, 2), (1, 0), (1, 1), (1, 2)]
    assert slicing.worker_layout(np.array([2, 3])).tolist() == [[0, 1, 2], [3, 4, 5]]
    assert list(slicing.filtered_range_index([2, 3], (1, None))) == [(1, 0), (1, 1), (1, 2)]
    assert slicing.assemble_index_filter((4, 3, 2), (1,)) == (None, 3, None)
    assert slicing.assemble_index_filter((4, 3, 2), (1,), invert=True) == (4, None, 2)
    assert slicing.compute_nd_slice_shape((slice(1, 4), slice(0, 2))) == (3, 2)
    assert slicing.compute_subshape_along_axis([2, 3], [0, 1], [7, 10], [1]).tolist() == [7, 3]
    assert distdl_padding_to_torch_padding(np.array([[0, 0], [1, 2], [3, 4]])) == (3, 4, 1, 2, 0, 0)
    assert zero_volume_tensor().shape == (0,) and zero_volume_tensor(3).shape == (3, 0)
    a, b = TensorStructure(torch.zeros(2, 3)), TensorStructure(torch.zeros(2, 3))
    assert a == b
    b.requires_grad = True
    assert a != b


# ------------------------------------------------------------ halo widths ----

def test_halo_mixin_known_answers(golden):
    g = golden("halo_mixin_k2s2.json")
    layer = MockPoolLayer()
    for entry in g["ranks"]:
        got = layer._compute_exchange_info(np.array(g["x_global_shape"]), np.array(g["kernel_size"]),
                                           np.array(g["stride"]), np.array(g["padding"]), np.array(g["dilation"]),
                                           True, np.array(g["partition_shape"]), np.array(entry["index"]))
        for arr, key in zip(got, ("halo", "recv", "send", "needed")):
            assert arr.tolist() == entry[key]
    assert layer._compute_exchange_info(None, None, None, None, None, False, None, None) == (None,) * 4


def test_halo_mixin_matches_oracle_on_reference_geometries(golden):
    layer = MockConvLayer()
    for geom in golden("layer_geometries.json")["conv_feature"]:
        P, g = geom["P_x_shape"], geom["x_global_shape"]
        nd = len(g)
        gpad = [0] * (nd - len(geom["padding"])) + geom["padding"]
        padded_global = [n + 2 * q for n, q in zip(g, gpad)]
        shapes = {i: tuple(n + a + b for n, (a, b) in zip(pm.subshape(P, i, g), o_halo.local_padding(P, i, gpad)))
                  for i in pm.indices(P)}
        table = np.zeros(list(P) + [nd], dtype=int)
        for i, s in shapes.items():
            table[i] = s
        for idx in pm.indices(P):
            want = o_halo.exchange_info(padded_global, geom["kernel_size"], geom["stride"],
                                        [0] * len(geom["kernel_size"]), geom["dilation"], P, idx, shapes=shapes)
            got = layer._compute_exchange_info(np.array(padded_global), np.array(geom["kernel_size"]),
                                               np.array(geom["stride"]), np.zeros(len(geom["kernel_size"]), dtype=int),
                                               np.array(geom["dilation"]), True, np.array(P), np.array(idx),
                                               subtensor_shapes=table)
            for arr, w in zip(got, want):
                assert arr.tolist() == w, (geom["id"], idx)


def test_halo_slices_match_oracle():
    rng = np.random.default_rng(2)
    for _ in range(50):
        nd = int(rng.integers(1, 6))
        recv = rng.integers(0, 3, (nd, 2))
        send = rng.integers(0, 3, (nd, 2))
        shape = [int(recv[j].sum() + send[j].sum() + rng.integers(1, 5)) for j in range(nd)]
        got = assemble_halo_slices(shape, recv, send)
        want = o_halo.slab_slices(shape, recv.tolist(), send.tolist())
        for i in range(nd):
            for q in range(4):
                assert [(s.start, s.stop) for s in got[i][q]] == [(s.start, s.stop) for s in want[i][q]]


# ---------------------------------------------------- partitions and world ----

def test_partition_algebra():
    world = SimWorld(6, device=torch.device("cpu"))
    P = world.partition(2)
    assert P.active and P.rank == 2 and P.size == 6 and P.shape.tolist() == [6]
    sub = P.create_partition_inclusive([4, 2, 0])
    assert sub.active and sub.rank == 1 and sub.size == 3
    other = P.create_partition_inclusive([1, 3])
    assert not other.active and other.size == -1 and other.index is None
    cart = sub.create_cartesian_topology_partition([3, 1])
    assert cart.index.tolist() == [1, 0] and cart.dim == 2
    assert cart.neighbor_ranks(1) == [(0, 2), (-1, -1)]
    inactive_cart = other.create_cartesian_topology_partition([1, 2])
    assert not inactive_cart.active and inactive_cart.shape.tolist() == [1, 2]     # the shape survives
    union = sub.create_partition_union(other)
    assert union._ranks == (4, 2, 0, 1, 3) and union.rank == 1
    assert cart == sub.create_cartesian_topology_partition([3, 1])
    assert not (cart == inactive_cart) and cart != union
    with pytest.raises(Exception):
        sub.create_cartesian_topology_partition([2, 2])
    grid = P.create_partition_inclusive(range(6)).create_cartesian_topology_partition([2, 3])
    assert grid.index.tolist() == [0, 2]
    row = grid.create_cartesian_subtopology_partition([False, True])
    assert row._ranks == (0, 1, 2) and row.rank == 2
    col = grid.create_cartesian_subtopology_partition([True, False])
    assert col._ranks == (2, 5) and col.rank == 0
    cart.deactivate()
    assert not cart.active and cart.shape.tolist() == [3, 1]


def test_loopback_transport_moves_data_between_rank_threads():
    world = SimWorld(4, device=torch.device("cpu"))

    def body(P):
        t = world.transport
        right, left = (P.rank + 1) % 4, (P.rank - 1) % 4
        out = torch.full((3,), float(P.rank))
        inbox = torch.empty(3)
        t.exchange(P, [(right, out, 7)], [(left, inbox, 7)])
        gathered = t.allgather(P, torch.tensor([P.rank * 1.0]), tag="g")
        shapes = t.subtensor_shapes(P.create_cartesian_topology_partition([2, 2]), (P.rank + 1, 5))
        summed = P.allreduce_data(np.array([P.rank]))
        root = P.broadcast_data("hello" if P.rank == 0 else None, root=0)
        return inbox.tolist(), gathered.flatten().tolist(), shapes[..., 0].tolist(), int(summed[0]), root

    for rank, (inbox, gathered, shapes, summed, root) in enumerate(world.run(body)):
        assert inbox == [float((rank - 1) % 4)] * 3
        assert gathered == [0.0, 1.0, 2.0, 3.0]
        assert shapes == [[1, 2], [3, 4]]
        assert summed == 6 and root == "hello"


def test_allgather_into_fills_the_other_slots_in_place():
    """In-place all-gather: every worker writes its own slot, the transport fills
    the rest (loopback); solo, the absent workers mirror the live one unless a
    provider speaks for them, on every call or -- declared constant -- once per
    buffer object."""
    world = SimWorld(3, device=torch.device("cpu"))

    def body(P):
        results = []
        buf = torch.full((3, 2), -1.0)
        for step in range(2):                       # the same buffer on consecutive calls
            buf[P.rank] = torch.tensor([10.0 * step + P.rank, 0.5])
            world.transport.allgather_into(P, buf, tag="s")
            results.append(buf.clone())
        return results

    for rank, results in enumerate(world.run(body)):
        for step, got in enumerate(results):
            assert got[:, 0].tolist() == [10.0 * step, 10.0 * step + 1, 10.0 * step + 2] and got[:, 1].tolist() == [0.5] * 3

    solo = SimWorld(3, device=torch.device("cpu"))
    P = solo.partition(1)
    buf = torch.zeros(3, 2)
    buf[0], buf[2] = torch.tensor([7.0, 7.0]), torch.tensor([9.0, 9.0])
    buf[1] = 1.0
    assert not solo.transport.peers_gathered_ahead(P, buf, tag="s")
    assert solo.transport.allgather_into(P, buf, tag="s") is buf and buf.tolist() == [[1, 1], [1, 1], [1, 1]]
    assert torch.equal(solo.transport.allgather(P, buf[1], tag="s"), buf)      # the two gathers agree about the peers
    calls = []

    def provider(P_, mine):
        calls.append(1)
        return [mine + 2.0, None, mine + 3.0]
    solo.transport.set_gather_provider("s", provider)
    solo.transport.allgather_into(P, buf, tag="s")
    buf[1] = 2.0
    assert not solo.transport.peers_gathered_ahead(P, buf, tag="s")
    solo.transport.allgather_into(P, buf, tag="s")
    assert buf.tolist() == [[4, 4], [2, 2], [5, 5]] and len(calls) == 2      # asked on every gather
    solo.transport.set_gather_provider("s", provider, constant=True)
    assert not solo.transport.peers_gathered_ahead(P, buf, tag="s")
    solo.transport.allgather_into(P, buf, tag="s")
    buf[1] = 6.0
    assert solo.transport.peers_gathered_ahead(P, buf, tag="s")
    solo.transport.allgather_into(P, buf, tag="s")
    assert buf.tolist() == [[4, 4], [6, 6], [5, 5]] and len(calls) == 3      # once per buffer
    other = torch.zeros(3, 2)                                                # another buffer object: asked again
    assert not solo.transport.peers_gathered_ahead(P, other, tag="s")


def test_loopback_transport_propagates_failures():
    world = SimWorld(2, device=torch.device("cpu"))

    def body(P):
        if P.rank == 1:
            raise ValueError("boom")
        world.transport.allgather(P, torch.zeros(1))

    with pytest.raises(ValueError, match="boom"):
        world.run(body, timeout=5.0)


# ------------------------------------------------------- Repartition setup ----

def _setup_world(world_size, make_layer_and_input):
    """Runs layer setup (no forward: that needs the GPU) on every rank thread."""
    world = SimWorld(world_size, device=torch.device("cpu"))

    def body(P_world):
        layer, x = make_layer_and_input(P_world)
        layer._distdl_forward_pre_hook(layer, (x,))
        return layer

    return world.run(body)


def _as_tuples(overlaps):
    out = []
    for sl, sh, partner in overlaps:
        if sl is None:
            out.append((None, None, None))
        else:
            out.append((tuple((int(s.start), int(s.stop)) for s in sl), tuple(int(v) for v in sh), partner))
    return out


@pytest.mark.parametrize("shape,P_x,P_y", [([7, 5], [4, 1], [2, 2]), ([3, 10, 11], [1, 4, 1], [1, 1, 4]),
                                          ([5, 6, 7], [2, 3, 1], [1, 2, 2]), ([8, 64, 128], [1, 8, 1], [1, 1, 8])])
def test_repartition_overlaps_match_oracle(shape, P_x, P_y):
    nx, ny = int(np.prod(P_x)), int(np.prod(P_y))
    x_shards = o_rep.scatter(np.zeros(shape, dtype=np.float32), P_x)

    def make(P_world):
        Px = P_world.create_partition_inclusive(range(nx)).create_cartesian_topology_partition(P_x)
        Py = P_world.create_partition_inclusive(range(ny)).create_cartesian_topology_partition(P_y)
        x = torch.from_numpy(x_shards[Px.rank]) if Px.active else zero_volume_tensor()
        return Repartition(Px, Py, preserve_batch=False), x

    layers = _setup_world(max(nx, ny), make)
    send, recv, _, y_boxes = o_rep.plan(shape, P_x, P_y, shared_workers=True)
    y_order = pm.indices(P_y)
    for rank, layer in enumerate(layers):
        def norm(lst):
            return [(tuple((s.start, s.stop) for s in sl), tuple(sh), p) if sl is not None else (None, None, None)
                    for sl, sh, p in lst]
        if rank < nx:
            assert _as_tuples(layer.P_x_to_y_overlaps) == norm(send[rank])
            assert [b is not None for b in layer.P_x_to_y_buffers] == \
                   [sl is not None and p != "self" for sl, sh, p in send[rank]]
        if rank < ny:
            assert _as_tuples(layer.P_y_to_x_overlaps) == norm(recv[rank])
            lo, hi = y_boxes[y_order[rank]]
            assert [int(v) for v in layer.output_tensor_structure.shape] == [h - l for l, h in zip(lo, hi)]


def test_identity_repartition_has_only_self_overlaps():
    def make(P_world):
        P = P_world.create_partition_inclusive(range(4)).create_cartesian_topology_partition([2, 2])
        return Repartition(P, P), torch.zeros(3, 4)

    for layer in _setup_world(4, make):
        for lst in (layer.P_x_to_y_overlaps, layer.P_y_to_x_overlaps):
            assert [p for sl, sh, p in lst if sl is not None] == ["self"]
        assert all(b is None for b in layer.P_x_to_y_buffers + layer.P_y_to_x_buffers)


def test_transpose_network_buffer_counts(golden):
    """Buffer counts per rank after each of the four chained repartitions of
    tests/utilities/test_buffer.py:128-193 (setup only; the GPU test runs it)."""
    g = golden("buffer_network.json")["transpose_network"]
    world = SimWorld(4, device=torch.device("cpu"))
    in_shapes = {"P_1": {0: (1, 10)}, "P_4": {r: (1, n) for r, n in enumerate([3, 3, 2, 2])},
                 "P_3": {r + 1: (1, n) for r, n in enumerate([4, 3, 3])}}

    def body(P_world):
        manager = BufferManager(device=torch.device("cpu"))
        parts = {name: P_world.create_partition_inclusive(spec["workers"]).create_cartesian_topology_partition(
            spec["shape"]) for name, spec in g["partitions"].items()}
        counts = []
        for src, dst in g["layers"]:
            layer = Repartition(parts[src], parts[dst], buffer_manager=manager)
            shape = in_shapes[src].get(P_world.rank)
            x = torch.zeros(shape) if shape is not None else zero_volume_tensor(1)
            layer._distdl_forward_pre_hook(layer, (x,))
            counts.append(len(manager.buffers_map.get(torch.float32, [])))
        return counts

    for rank, counts in enumerate(world.run(body)):
        assert counts == [c[rank] for c in g["n_buffers_by_rank_after_layer"]]


def test_repartition_errors():
    world = SimWorld(4, device=torch.device("cpu"))
    P = world.partition(0)
    P2 = P.create_partition_inclusive(range(4)).create_cartesian_topology_partition([2, 2])
    P3 = P.create_partition_inclusive(range(4)).create_cartesian_topology_partition([1, 2, 2])
    with pytest.raises(ValueError, match="same dimension"):
        Repartition(P2, P3)
    with pytest.raises(ValueError, match="Buffer manager"):
        Repartition(P2, P2, buffer_manager=object())
    layer = Repartition(P2, P2)
    with pytest.raises(ValueError, match="same dimension"):
        layer._distdl_forward_pre_hook(layer, (torch.zeros(2, 3, 4),))
    # the HIP path refuses CPU tensors instead of computing something else
    P14 = P.create_partition_inclusive(range(4)).create_cartesian_topology_partition([1, 4])
    P41 = P.create_partition_inclusive(range(4)).create_cartesian_topology_partition([4, 1])
    layer = Repartition(P14, P41)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        layer(torch.zeros(8, 2))


def test_setup_reruns_when_input_structure_changes():
    world = SimWorld(4, device=torch.device("cpu"))
    P = world.partition(0)
    P14 = P.create_partition_inclusive(range(4)).create_cartesian_topology_partition([1, 4])
    P41 = P.create_partition_inclusive(range(4)).create_cartesian_topology_partition([4, 1])
    layer = Repartition(P14, P41)
    layer._distdl_forward_pre_hook(layer, (torch.zeros(8, 2),))
    first = layer.P_x_to_y_overlaps
    layer._distdl_forward_pre_hook(layer, (torch.zeros(8, 2),))
    assert layer.P_x_to_y_overlaps is first
    layer._distdl_forward_pre_hook(layer, (torch.zeros(12, 2),))
    assert layer.P_x_to_y_overlaps is not first
    assert [int(v) for v in layer.output_tensor_structure.shape] == [3, 8]


# ------------------------------------------------------------ buffers --------

def test_expandable_buffer_views_and_growth():
    buf = ExpandableBuffer(torch.float32, device=torch.device("cpu"))
    assert buf.capacity == 0
    v = buf.get_view((2, 3))
    assert buf.capacity == 6 and v.shape == (2, 3) and v.is_contiguous()
    assert buf.get_view((2, 3)) is v
    v.copy_(torch.arange(6.0).reshape(2, 3))
    w = buf.get_view((4, 5))                        # grows: old contents and old views survive
    assert buf.capacity == 20 and w.shape == (4, 5)
    assert buf.get_view((2, 3)).flatten().tolist() == [0, 1, 2, 3, 4, 5]
    assert buf.get_view((2, 3)).data_ptr() == w.data_ptr() == buf.raw_buffer.data_ptr()
    buf.expand(10)
    assert buf.capacity == 20


def test_buffer_manager_reuses_buffers():
    m = BufferManager(device=torch.device("cpu"))
    a = m.request_buffers(3, torch.float32)
    b = m.request_buffers(2, torch.float32)
    assert b[0] is a[0] and b[1] is a[1] and len(m.buffers_map[torch.float32]) == 3
    c = m.request_buffers(5, torch.float32)
    assert c[:3] == a and len(m.buffers_map[torch.float32]) == 5
    d = m.request_buffers(1, torch.int32)
    assert len(m.buffers_map[torch.int32]) == 1 and d[0] is not a[0]


def test_halo_layer_uses_exactly_four_buffers(golden):
    g = golden("buffer_network.json")["conv2d_network"]
    world = SimWorld(4, device=torch.device("cpu"))

    def body(P_world):
        manager = BufferManager(device=torch.device("cpu"))
        P = P_world.create_partition_inclusive(range(4)).create_cartesian_topology_partition(g["partition_shape"])
        counts = []
        chans = [1, 5, 10, 20]
        local = pm.subshape(g["partition_shape"], tuple(P.index), g["tensor"])
        for cin, cout in zip(chans[:-1], chans[1:]):
            layer = DistributedConv2d(P, in_channels=cin, out_channels=cout, kernel_size=g["kernel_size"],
                                      padding=g["padding"], bias=False, buffer_manager=manager)
            x = torch.zeros([1, cin] + local[2:])
            layer._distdl_forward_pre_hook(layer, (x,))
            padded = [n + int(a) + int(b) for n, (a, b) in zip(x.shape, layer.local_padding + layer.halo_shape)]
            layer.halo_layer._distdl_forward_pre_hook(layer.halo_layer, (torch.zeros(padded),))
            counts.append(len(manager.buffers_map[torch.float32]))
        return counts

    for rank, counts in enumerate(world.run(body)):
        assert counts == [g["n_buffers_by_rank"][rank]] * 3


def test_conv_selector_and_config5_geometry():
    world = SimWorld(8, device=torch.device("cpu"))
    P = world.partition(0).create_partition_inclusive(range(8)).create_cartesian_topology_partition([1, 1, 2, 2, 2])
    layer = DistributedConv3d(P, in_channels=32, out_channels=4, kernel_size=3, padding=1)
    assert type(layer).__name__ == "DistributedFeatureConv3d"
    with pytest.raises(NotImplementedError):
        DistributedConv3d(P, P, P, in_channels=1, out_channels=1, kernel_size=3)
    with pytest.raises(ValueError):
        DistributedConv3d(P, P, None, in_channels=1, out_channels=1, kernel_size=3)
    # meta tensor: shapes only (the real shard is 268 MB)
    layer._distdl_forward_pre_hook(layer, (torch.empty(1, 32, 128, 128, 128, device="meta"),))
    assert layer.halo_shape.tolist() == [[0, 0], [0, 0], [0, 1], [0, 1], [0, 1]]
    assert layer.send_buffer_shape.tolist() == [[0, 0], [0, 0], [0, 1], [0, 1], [0, 1]]
    assert layer.local_padding.tolist() == [[0, 0], [0, 0], [1, 0], [1, 0], [1, 0]]
    assert [(int(s.start), int(s.stop)) for s in layer.needed_slices] == [(0, 1), (0, 32), (0, 130), (0, 130), (0, 130)]
    plan = layer._staging_plan
    assert plan.padded_shape == (1, 32, 130, 130, 130)
    assert plan.slab_shape(2, 1, "bulk") == (1, 32, 1, 129, 129)
    assert plan.slab_shape(3, 1, "ghost") == (1, 32, 130, 1, 129)
    assert plan.slab_shape(4, 1, "bulk") == (1, 32, 130, 130, 1)
    assert plan.slab_shape(2, 0, "ghost") is None


def test_halo_exchange_layer_setup_and_errors():
    world = SimWorld(4, device=torch.device("cpu"))
    P = world.partition(3).create_partition_inclusive(range(4)).create_cartesian_topology_partition([1, 1, 2, 2])
    halo = np.array([[0, 0], [0, 0], [1, 0], [1, 0]])
    layer = HaloExchange(P, halo, halo, halo)
    assert layer.neighbor_ranks == [(-1, -1), (-1, -1), (1, -1), (2, -1)]
    with pytest.raises(ValueError, match="Buffer manager"):
        HaloExchange(P, halo, halo, halo, buffer_manager="nope")
    layer._distdl_forward_pre_hook(layer, (torch.zeros(1, 1, 4, 4),))
    assert [b is not None for b in layer.buffers[2]] == [True, True, False, False]
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        layer(torch.zeros(1, 1, 4, 4))


# ------------------------------------------------------------- backend -------

def test_backend_registry_and_selection(monkeypatch):
    from distdl_amd import backends
    from distdl_amd import config
    assert backends.backend.__name__ == "stub_hip"
    assert "stub_hip" in backends.supported_backends
    for name in ("Partition", "CartesianPartition", "assemble_global_tensor_structure",
                 "assemble_global_tensor_structure_along_axis", "broadcast_tensor_structure", "buffer_allocator",
                 "tensor_comm", "tensor_decomposition", "functional", "ExpandableBuffer", "BufferManager",
                 "get_device", "set_device"):
        assert hasattr(backends.backend, name), name
    for sub in ("all_gather", "all_sum_reduce", "broadcast", "halo_exchange", "reduce_scatter", "repartition",
                "sum_reduce"):
        assert hasattr(backends.backend.functional, sub)
    assert config.set_backend("stub", "hip", check_input_changed=False).__name__ == "stub_hip"
    assert config.check_input_changed is False
    config.set_backend(check_input_changed=True)
    with pytest.raises(ValueError, match="not available"):
        config.set_backend("mpi", "numpy")
    monkeypatch.setenv("DISTDL_CHECK_INPUT_CHANGED", "0")
    assert config.get_default_pre_hook_setting() is False


# --------------------------------------------------------------- C ABI -------

def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "distdl_hip.h")).read()
    declared = set(re.findall(r"\b(ddl_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libdistdl_hip.so not built")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert _lib.load().ddl_version().decode().startswith("distdl_hip")
    assert ctypes.sizeof(_lib.ddl_box_t) == 8 + 8 + 4 + 4 + 3 * 8 * 8


def test_c_abi_rejects_bad_arguments_without_a_gpu():
    """Argument checks run on the host before anything is launched."""
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libdistdl_hip.so not built")
    lib = _lib.load()
    shape = _lib.i64_array([4, 4])
    rc = lib.ddl_pack_boxes(1, shape, shape, 9, 4, 1, shape, shape, _lib.ptr_array([16]), None)
    assert rc == -2 and b"ndim" in lib.ddl_last_error()
    rc = lib.ddl_linear_bf16(16, 16, None, 16, 8, 8, 7, 7, 7, 8, None)
    assert rc == -3
    rc = lib.ddl_ln_normalize_affine_f32(16, 4, 4, 4, 16, 0, shape, None, None, 1e-5, 16, 4, None, None, None)
    assert rc == -5
    rc = lib.ddl_embedding_gather(16, 8, 8, 3, 16, 1, 4, 0, 4, 16, None)
    assert rc == -1
    rc = lib.ddl_embedding_renorm(16, _lib.DDL_DT_F32, 8, 8, 16, 1, 4, 0, 4, -1.0, 2.0, 16, None)     # negative max_norm
    assert rc == -1 and b"max_norm" in lib.ddl_last_error()
    rc = lib.ddl_embedding_renorm(16, _lib.DDL_DT_F64, 8, 8, 16, 1, 4, 0, 4, 1.0, 2.0, 16, None)      # no float64 tables
    assert rc == -5
    assert lib.ddl_embedding_renorm(16, _lib.DDL_DT_F32, 8, 8, 16, 1, 0, 0, 4, 1.0, 2.0, 16, None) == 0   # no ids: nothing to do
    assert lib.ddl_pack_boxes(1, shape, shape, 2, 4, 0, shape, shape, _lib.ptr_array([]), None) == 0


def test_broadcast_partner_follows_the_reference_rule():
    """backends/common/partition.py:552-604, :745-794: shapes compared after an
    optional reversal and left-padding of the smaller one with ones; a worker of
    the larger team belongs to the smaller team's worker with the same index in
    the dimensions whose extents agree."""
    import itertools

    from distdl_amd.backends.stub_hip.transport import TransportError, broadcast_partner

    def owners(small_shape, big_shape, big_index, transpose_small=False, transpose_big=False):
        return [s for s in itertools.product(*[range(n) for n in small_shape])
                if broadcast_partner(small_shape, s, big_shape, big_index, transpose_small, transpose_big)]

    for i in itertools.product(range(2), range(2), range(3)):
        assert owners([2, 2, 1], [2, 2, 3], i) == [(i[0], i[1], 0)]
    for i in itertools.product(range(3), range(2), range(2)):
        assert owners([2, 2, 1], [3, 2, 2], i, transpose_big=True) == [(i[2], i[1], 0)]     # [2, 2, 3] against [2, 2, 1]
        assert owners([2, 2, 1], [3, 2, 2], i, transpose_small=True) == [(i[2], i[1], 0)]   # [3, 2, 2] against [1, 2, 2]
    for c in range(3):
        assert owners([1], [1, 1, 3], (0, 0, c)) == [(0,)]
    # The affine layer: x on 1 x P_fi goes down the columns of P_fo x P_fi,
    # partial outputs are summed along its rows onto 1 x P_fo.
    for o, i in itertools.product(range(3), range(4)):
        assert owners([1, 4], [3, 4], (o, i)) == [(0, i)]
        assert owners([1, 3], [3, 4], (o, i), transpose_big=True) == [(0, o)]
    with pytest.raises(TransportError):
        broadcast_partner([2, 3], [0, 0], [2, 2], [0, 0])
    with pytest.raises(TransportError):
        broadcast_partner([1, 1, 2], [0, 0, 0], [2, 2], [0, 0])


def test_conv_selector_picks_the_feature_class_and_rejects_what_the_reference_rejects():
    """tests/layers/test_conv.py:10-60, :88-100 (a selector given P_x alone
    builds the feature-partitioned layer) and :200-236 (only one of P_y, P_w:
    ValueError).  The channel-partitioned and general layers the reference
    builds when both are given do not exist here: that request says so."""
    from distdl_amd import nn as dnn
    from distdl_amd.backends.stub_hip import SimWorld
    world = SimWorld(8, device="cpu")
    P_world = world.partition(0)
    cases = [(dnn.DistributedConv1d, dnn.DistributedFeatureConv1d, [1, 1, 4], [3]),
             (dnn.DistributedConv2d, dnn.DistributedFeatureConv2d, [1, 1, 2, 2], [3, 3]),
             (dnn.DistributedConv3d, dnn.DistributedFeatureConv3d, [1, 1, 2, 2, 1], [3, 3, 3])]
    for Selector, Feature, shape, ks in cases:
        P_x = P_world.create_partition_inclusive(list(range(4))).create_cartesian_topology_partition(shape)
        layer = Selector(P_x, in_channels=3, out_channels=3, kernel_size=ks)
        assert isinstance(layer, Feature)
    P2 = P_world.create_partition_inclusive([0, 1])
    P4 = P_world.create_partition_inclusive([0, 1, 2, 3])
    P_x = P2.create_cartesian_topology_partition([1, 2, 1, 1])
    P_y = P2.create_cartesian_topology_partition([1, 2, 1, 1])
    P_w = P4.create_cartesian_topology_partition([2, 2, 1, 1])
    with pytest.raises(ValueError):
        dnn.DistributedConv2d(P_x, P_y=P_y, in_channels=3, out_channels=3, kernel_size=[3, 3])
    with pytest.raises(ValueError):
        dnn.DistributedConv2d(P_x, P_w=P_w, in_channels=3, out_channels=3, kernel_size=[3, 3])
    with pytest.raises(NotImplementedError):
        dnn.DistributedConv2d(P_x, P_y=P_y, P_w=P_w, in_channels=3, out_channels=3, kernel_size=[3, 3])


def test_sum_reduce_and_broadcast_layers_with_one_live_worker():
    """Solo transport: the peers are absent, so a reduction hands the live
    worker its own contribution if it receives (and the reference's zero-volume
    tensor if it only sends), and a broadcast is the identity on the owner."""
    from distdl_amd.nn import Broadcast, SumReduce
    for rank, receives in ((0, True), (3, False)):
        world = SimWorld(4, device=torch.device("cpu"))
        P_world = world.partition(rank)
        P_w = P_world.create_partition_inclusive([0, 1, 2, 3]).create_cartesian_topology_partition([2, 2])
        P_y = P_world.create_partition_inclusive([0, 1]).create_cartesian_topology_partition([1, 2])
        layer = SumReduce(P_w, P_y, transpose_src=True, preserve_batch=True)
        x = torch.arange(12.0).reshape(3, 4).requires_grad_(True)
        y = layer(x)
        if receives:
            assert torch.equal(y.detach(), x.detach())
            y.backward(torch.ones_like(y))
            assert torch.equal(x.grad, torch.ones(3, 4))
        else:
            assert tuple(y.shape) == (3, 0)
    world = SimWorld(4, device=torch.device("cpu"))
    P_world = world.partition(0)
    P_x = P_world.create_partition_inclusive([0, 1]).create_cartesian_topology_partition([1, 2])
    P_w = P_world.create_partition_inclusive([0, 1, 2, 3]).create_cartesian_topology_partition([2, 2])
    x = torch.arange(6.0).reshape(2, 3).requires_grad_(True)
    y = Broadcast(P_x, P_w, preserve_batch=True)(x)
    assert torch.equal(y.detach(), x.detach())
    y.backward(2 * torch.ones_like(y))
    assert torch.equal(x.grad, 2 * torch.ones(2, 3))


def test_primitive_functions_take_the_reference_arguments():
    """Every autograd Function of the backend is called by the reference's
    layers with a fixed list of positional arguments
    (backends/mpi_numpy/functional/all_gather.py:36-37, all_sum_reduce.py:32-33,
    broadcast.py:32-34, reduce_scatter.py:35-37, sum_reduce.py:32-34,
    repartition.py:33-36, halo_exchange.py:14); forward takes exactly those and
    backward returns one gradient slot for each."""
    import inspect
    from distdl_amd import backends
    fn = backends.backend.functional
    expected = {
        fn.all_gather.AllGatherFunction:
            ["input", "P_allgather", "input_tensor_structure", "output_tensor_structure", "axes", "scale_backward"],
        fn.all_sum_reduce.AllSumReduceFunction:
            ["input", "P_allreduce", "input_tensor_structure", "output_tensor_structure", "scale_backward"],
        fn.broadcast.BroadcastFunction:
            ["input", "P_send", "P_recv", "preserve_batch", "input_tensor_structure", "output_tensor_structure",
             "scale_backward"],
        fn.reduce_scatter.ReduceScatterFunction:
            ["input", "P_reducescatter", "input_tensor_structure", "output_tensor_structure", "axes"],
        fn.sum_reduce.SumReduceFunction:
            ["input", "P_send", "P_recv", "preserve_batch", "input_tensor_structure", "output_tensor_structure"],
        fn.repartition.RepartitionFunction:
            ["input", "P_union", "x_global_structure", "x_local_structure", "y_local_structure", "P_x",
             "P_x_to_y_overlaps", "P_x_to_y_buffers", "P_y", "P_y_to_x_overlaps", "P_y_to_x_buffers", "preserve_batch"],
        fn.halo_exchange.HaloExchangeFunction: ["input", "P_x", "slices", "buffers", "neighbor_ranks"],
    }
    for Function, names in expected.items():
        params = list(inspect.signature(Function.forward).parameters.values())
        assert [p.name for p in params] == ["ctx"] + names, Function.__name__
        assert all(p.default is inspect.Parameter.empty for p in params), Function.__name__
    # one live worker: identity paths hand back one gradient slot per argument
    world = SimWorld(1, device=torch.device("cpu"))
    P = world.partition(0).create_partition_inclusive([0]).create_cartesian_topology_partition([1, 1])
    x = torch.arange(6.0).reshape(2, 3).requires_grad_(True)
    s = TensorStructure(x)
    y = fn.all_gather.AllGatherFunction.apply(x, P.create_allreduction_partition((1,)), s, s, (1,), None)
    y = fn.reduce_scatter.ReduceScatterFunction.apply(y, P.create_allreduction_partition((1,)), s, s, (1,))
    y = fn.all_sum_reduce.AllSumReduceFunction.apply(y, P.create_allreduction_partition((0,)), s, s, None)
    y.backward(torch.ones_like(y))
    assert torch.equal(x.grad, torch.ones(2, 3))


def test_route_partitions_of_broadcast_and_reduction():
    """create_broadcast_partition_to / create_reduction_partition_to hand back
    (P_send, P_recv), active on the workers of the source resp. destination
    (backends/common/partition.py:490-632, :683-823), and
    create_allreduction_partition the workers that differ along the axes only."""
    world = SimWorld(4, device=torch.device("cpu"))
    for rank in range(4):
        P_world = world.partition(rank)
        P_x = P_world.create_partition_inclusive([0, 1]).create_cartesian_topology_partition([1, 2])
        P_w = P_world.create_partition_inclusive([0, 1, 2, 3]).create_cartesian_topology_partition([2, 2])
        P_send, P_recv = P_x.create_broadcast_partition_to(P_w)
        assert P_send.active == (rank < 2) and P_recv.active
        P_send, P_recv = P_w.create_reduction_partition_to(P_x, transpose_src=True)
        assert P_send.active and P_recv.active == (rank < 2)
        P_r = P_w.create_allreduction_partition((0,))
        assert list(P_r.shape) == [2, 1] and P_r.size == 2
        assert P_r._ranks == ((0, 2) if rank % 2 == 0 else (1, 3)) and P_r.rank == rank // 2
    with pytest.raises(ValueError):
        P_w.create_allreduction_partition((2,))


def test_bench_refuses_more_than_one_gpu():
    """One GPU's share is what is measured; a request for more says so and
    exits before anything touches a device."""
    import subprocess
    import sys
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                          timeout=300)
    assert done.returncode != 0
    assert "ONE GPU" in (done.stderr + done.stdout)
