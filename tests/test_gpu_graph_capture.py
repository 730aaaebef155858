"""The layers of the path under HIP graph capture: every kernel goes to the
stream the caller has made current, nothing on the forward path synchronises or
allocates outside torch's caching allocator, so a forward can be captured with
``torch.cuda.graph`` and replayed.  Each graph is replayed several times with
new input contents and eager work in between, and every replay is checked
against the eager result."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _replay_checks(make_input, run, n_replays=3):
    """Captures run(static_input) once, then compares replays with eager calls."""
    static = make_input(0)
    for _ in range(3):            # warm-up outside capture: set-up hooks, plans, buffers, LDS attributes
        run(static)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            out = run(static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for i in range(1, n_replays + 1):
        fresh = make_input(i)
        want = run(fresh).clone()                     # eager, on the current stream
        scratch = torch.randn(1 << 20, device="cuda").sum()   # unrelated eager work between replays
        static.copy_(fresh)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i} differs from the eager result"
        assert torch.isfinite(scratch)


def test_layernorm_layer_forward_replays_from_a_graph():
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import DistributedLayerNorm
    from distdl_amd.nn.layernorm import STATS_TAG
    from oracle import layernorm as o_ln
    world = SimWorld(4)
    P_x = world.partition(0).create_partition_inclusive(list(range(4))).create_cartesian_topology_partition([1, 1, 4])
    layer = DistributedLayerNorm(P_x, [512])
    gen = torch.Generator().manual_seed(21)
    whole = torch.randn(4, 64, 512, generator=gen)
    peers = [None] + [torch.from_numpy(o_ln.partial_stats(whole[..., 128 * p:128 * (p + 1)].numpy()).astype(np.float32)).cuda()
                      for p in range(1, 4)]
    world.transport.set_gather_provider(STATS_TAG, lambda P, t: list(peers), constant=True)

    def make_input(i):
        g = torch.Generator().manual_seed(100 + i)
        return (whole[..., :128] + 0.1 * torch.randn(4, 64, 128, generator=g)).contiguous().cuda()

    with torch.no_grad():
        _replay_checks(make_input, lambda x: layer(x))


def test_linear_and_embedding_shards_replay_from_a_graph():
    from distdl_amd import hip_ops
    gen = torch.Generator().manual_seed(5)
    w = (0.05 * torch.randn(320, 256, generator=gen)).to(torch.bfloat16).cuda()
    b = (0.05 * torch.randn(320, generator=gen)).to(torch.bfloat16).cuda()

    def make_x(i):
        g = torch.Generator().manual_seed(200 + i)
        return torch.randn(300, 256, generator=g).to(torch.bfloat16).cuda()

    _replay_checks(make_x, lambda x: hip_ops.linear(x, w, b))

    table = torch.randn(1000, 64, generator=gen).to(torch.bfloat16).cuda()

    def make_ids(i):
        g = torch.Generator().manual_seed(300 + i)
        return torch.randint(0, 2000, (4, 128), generator=g).cuda()

    _replay_checks(make_ids, lambda ids: hip_ops.embedding_gather(table, ids, 500, 1500))


def test_repartition_layer_forward_replays_from_a_graph():
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import Repartition
    world = SimWorld(4)
    P_world = world.partition(0)
    P_x = P_world.create_partition_inclusive(list(range(4))).create_cartesian_topology_partition([1, 4, 1])
    P_y = P_world.create_partition_inclusive(list(range(4))).create_cartesian_topology_partition([1, 1, 4])
    layer = Repartition(P_x, P_y)

    def make_input(i):
        g = torch.Generator().manual_seed(400 + i)
        return torch.randn(2, 32, 256, generator=g).cuda()      # rank 0's shard of [2, 128, 256]

    with torch.no_grad():
        _replay_checks(make_input, lambda x: layer(x))
