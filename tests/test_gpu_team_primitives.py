"""Broadcast, SumReduce, AllSumReduce, AllGather and ReduceScatter between
simulated workers, on the parametrizations of the reference's own tests, and
DistributedLinear with a partitioned input dimension on top of them.  The collectives themselves are
stand-ins (rank threads of one process); the sums run on the box kernel and the
shard products on the GEMM kernels.  Expected values come from a rule written
out per case below, not from the transport's own partner search."""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


def _index_of(rank, shape):
    return tuple(int(i) for i in np.unravel_index(rank, shape))


# (small ranks, small shape, big ranks, big shape, transpose of the big side,
#  world size, small index a big index belongs to).  The reference gives the
# same team layouts to tests/primitives/test_broadcast.py:10-133 (small -> big)
# and tests/primitives/test_sum_reduce.py:10-133 (big -> small).
TEAM_LAYOUTS = [
    pytest.param(range(4, 8), [2, 2, 1], range(0, 12), [2, 2, 3], False, 12, lambda i: (i[0], i[1], 0), id="overlap-3D"),
    pytest.param(range(0, 4), [2, 2, 1], range(4, 16), [2, 2, 3], False, 16, lambda i: (i[0], i[1], 0), id="disjoint-3D"),
    pytest.param(range(0, 4), [2, 2, 1], range(5, 17), [2, 2, 3], False, 17, lambda i: (i[0], i[1], 0), id="disjoint-inactive-3D"),
    pytest.param(range(0, 1), [1], range(0, 1), [1], False, 1, lambda i: (0,), id="sequential-identity"),
    pytest.param(range(2, 3), [1], range(0, 3), [1, 1, 3], False, 3, lambda i: (0,), id="overlap-single"),
    pytest.param(range(3, 4), [1], range(0, 3), [1, 1, 3], False, 4, lambda i: (0,), id="disjoint-single"),
    pytest.param(range(4, 5), [1], range(0, 3), [1, 1, 3], False, 5, lambda i: (0,), id="disjoint-inactive-single"),
    # With the source's shape and index read backwards, index (a, b, c) of the big team [3, 2, 2] belongs to
    # small (c, b, 0): [2, 2, 3] against [2, 2, 1] for a reduction, [3, 2, 2] against [1, 2, 2] for a broadcast.
    pytest.param(range(4, 8), [2, 2, 1], range(0, 12), [3, 2, 2], True, 12, lambda i: (i[2], i[1], 0), id="overlap-3D-transposed"),
    pytest.param(range(0, 4), [2, 2, 1], range(4, 16), [3, 2, 2], True, 16, lambda i: (i[2], i[1], 0), id="disjoint-3D-transposed"),
    pytest.param(range(0, 4), [2, 2, 1], range(5, 17), [3, 2, 2], True, 17, lambda i: (i[2], i[1], 0),
                 id="disjoint-inactive-3D-transposed"),
]


def _teams(P_world, small_ranks, small_shape, big_ranks, big_shape):
    P_small = P_world.create_partition_inclusive(list(small_ranks)).create_cartesian_topology_partition(small_shape)
    P_big = P_world.create_partition_inclusive(list(big_ranks)).create_cartesian_topology_partition(big_shape)
    return P_small, P_big


def _values(world, shape, seed, dtype):
    gen = torch.Generator().manual_seed(seed)
    return [(8 * torch.randn(*shape, generator=gen)).to(dtype) for _ in range(world)]


def _run_sum_reduce(small_ranks, small_shape, big_ranks, big_shape, transposed, world, dtype, backward):
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import SumReduce
    from distdl_amd.utilities.torch import zero_volume_tensor
    xs = _values(world, [1, 7, 5], 3, dtype)
    dys = _values(world, [1, 7, 5], 4, dtype)

    def body(P_world):
        P_y, P_x = _teams(P_world, small_ranks, small_shape, big_ranks, big_shape)
        layer = SumReduce(P_x, P_y, transpose_src=transposed, preserve_batch=False)
        me = P_world.rank
        x = xs[me].cuda() if P_x.active else zero_volume_tensor(dtype=dtype, device="cuda")
        x.requires_grad = backward
        y = layer(x)
        dx = None
        if backward:
            y.backward(dys[me].cuda() if P_y.active else zero_volume_tensor(dtype=dtype, device="cuda"))
            dx = x.grad.cpu()
        torch.cuda.synchronize()
        return y.detach().cpu(), dx

    return xs, dys, SimWorld(world).run(body)


@pytest.mark.parametrize("small_ranks,small_shape,big_ranks,big_shape,transposed,world,owner", TEAM_LAYOUTS)
def test_sum_reduce_reference_layouts(small_ranks, small_shape, big_ranks, big_shape, transposed, world, owner):
    """tests/primitives/test_sum_reduce.py:136-211 checks <F x, dy> = <x, F* dy>;
    here every output is compared with the sum of the tensors of the workers
    that reduce onto it (added in rank order, so the bits are fixed), every
    gradient with the gradient of the worker it reduced onto."""
    small_ranks, big_ranks = list(small_ranks), list(big_ranks)
    xs, dys, outs = _run_sum_reduce(small_ranks, small_shape, big_ranks, big_shape, transposed, world, torch.float32, True)
    owner_rank = {}
    for j, r in enumerate(big_ranks):
        small_index = owner(_index_of(j, big_shape))
        owner_rank[r] = small_ranks[int(np.ravel_multi_index(small_index, small_shape))]
    for r in range(world):
        y, dx = outs[r]
        if r in small_ranks:
            want = None
            for s in big_ranks:                        # rank order
                if owner_rank[s] == r:
                    want = xs[s].clone() if want is None else want + xs[s]
            assert want is not None and torch.equal(y, want), f"worker {r}"
        elif r in big_ranks:
            assert y.numel() == 0
        if r in big_ranks:
            assert torch.equal(dx, dys[owner_rank[r]]), f"worker {r}"
        elif r in small_ranks:
            assert dx.numel() == 0
    # The reference's own criterion, on top.
    lhs = sum(float((outs[r][0].double() * dys[r].double()).sum()) for r in small_ranks)
    rhs = sum(float((xs[r].double() * outs[r][1].double()).sum()) for r in big_ranks)
    assert abs(lhs - rhs) <= 1e-6 * max(abs(lhs), abs(rhs), 1.0)      # the outputs are float32 sums


@pytest.mark.parametrize("dtype,backward", [(torch.float32, True), (torch.int32, False), (torch.float64, True)])
def test_sum_reduce_reference_dtype_cases(dtype, backward):
    """tests/primitives/test_sum_reduce.py:214-330: the [2, 2, 3] onto [2, 2, 1]
    layout in float32, int32 (no gradient) and float64; output and gradient keep
    the dtype, and the integer sum is exact."""
    small_ranks, big_ranks = list(range(4, 8)), list(range(12))
    xs, dys, outs = _run_sum_reduce(small_ranks, [2, 2, 1], big_ranks, [2, 2, 3], False, 12, dtype, backward)
    for j, r in enumerate(small_ranks):
        members = [s for s in big_ranks if s // 3 == j]          # [2, 2, 3] row-major: the last index varies fastest
        want = xs[members[0]].clone()
        for s in members[1:]:
            want = want + xs[s]
        y, _ = outs[r]
        assert y.dtype == dtype and torch.equal(y, want)
    if backward:
        for s in big_ranks:
            dx = outs[s][1]
            assert dx.dtype == dtype and torch.equal(dx, dys[small_ranks[s // 3]])


@pytest.mark.parametrize("small_ranks,small_shape,big_ranks,big_shape,transposed,world,owner", TEAM_LAYOUTS)
def test_broadcast_reference_layouts(small_ranks, small_shape, big_ranks, big_shape, transposed, world, owner):
    """tests/primitives/test_broadcast.py:136-211 on the same layouts, read the
    other way round: every worker of the big team receives its owner's tensor,
    every owner the sum of its receivers' gradients."""
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import Broadcast
    from distdl_amd.utilities.torch import zero_volume_tensor
    small_ranks, big_ranks = list(small_ranks), list(big_ranks)
    xs = _values(world, [1, 7, 5], 5, torch.float32)
    dys = _values(world, [1, 7, 5], 6, torch.float32)

    def body(P_world):
        P_x, P_y = _teams(P_world, small_ranks, small_shape, big_ranks, big_shape)
        layer = Broadcast(P_x, P_y, transpose_src=transposed, preserve_batch=False)
        me = P_world.rank
        x = xs[me].cuda() if P_x.active else zero_volume_tensor(device="cuda")
        x.requires_grad = True
        y = layer(x)
        y.backward(dys[me].cuda() if P_y.active else torch.zeros_like(y))
        torch.cuda.synchronize()
        return y.detach().cpu(), x.grad.cpu()

    outs = SimWorld(world).run(body)
    owner_rank = {}
    for j, r in enumerate(big_ranks):
        owner_rank[r] = small_ranks[int(np.ravel_multi_index(owner(_index_of(j, big_shape)), small_shape))]
    for r in big_ranks:
        assert torch.equal(outs[r][0], xs[owner_rank[r]]), f"worker {r}"
    for r in small_ranks:
        want = None
        for s in big_ranks:
            if owner_rank[s] == r:
                want = dys[s].clone() if want is None else want + dys[s]
        assert torch.equal(outs[r][1], want), f"worker {r}"


def test_all_sum_reduce_is_its_own_adjoint():
    """reference: backends/mpi_numpy/functional/all_sum_reduce.py:95-161 -- the
    gradient is all-sum-reduced over the same workers as the input."""
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import AllSumReduce
    xs = _values(6, [3, 4], 7, torch.float32)
    dys = _values(6, [3, 4], 8, torch.float32)

    def body(P_world):
        P_x = P_world.create_partition_inclusive(list(range(6))).create_cartesian_topology_partition([2, 3])
        layer = AllSumReduce(P_x, axes_reduce=(1,))
        x = xs[P_world.rank].cuda().requires_grad_(True)
        y = layer(x)
        y.backward(dys[P_world.rank].cuda())
        torch.cuda.synchronize()
        return y.detach().cpu(), x.grad.cpu()

    outs = SimWorld(6).run(body)
    for r in range(6):
        row = [3 * (r // 3) + c for c in range(3)]
        assert torch.allclose(outs[r][0], sum(xs[s] for s in row), rtol=0, atol=1e-5)
        assert torch.allclose(outs[r][1], sum(dys[s] for s in row), rtol=0, atol=1e-5)


@pytest.mark.parametrize("x_ranks,P_x_shape,y_ranks,P_y_shape,P_w_shape,batch,c_in,c_out,use_bias", [
    pytest.param(range(4, 8), [1, 4], range(0, 3), [1, 3], [3, 4], 1, 12, 6, False, id="distributed"),
    pytest.param(range(0, 1), [1, 1], range(0, 1), [1, 1], [1, 1], 1, 12, 6, False, id="sequential"),
    pytest.param(range(4, 8), [1, 4], range(0, 3), [1, 3], [3, 4], 9, 26, 20, True, id="distributed-uneven-bias"),
    pytest.param(range(1, 3), [1, 2], range(2, 4), [1, 2], [2, 2], 5, 16, 8, True, id="2x2-shifted-teams"),
])
def test_linear_layer_reference_cases(x_ranks, P_x_shape, y_ranks, P_y_shape, P_w_shape, batch, c_in, c_out, use_bias):
    """DistributedLinear on the team layouts of tests/layers/test_linear.py:10-35
    (x on workers 4-7 as 1 x 4, y on workers 0-2 as 1 x 3, weights on all twelve
    as 3 x 4; [1, 12] -> [1, 6]) and on larger, uneven sizes with a bias: the
    input is broadcast down the columns of the weight partition, every worker
    applies its shard, the partial outputs are summed along the rows.  Forward
    and gradients against torch.nn.functional.linear on the whole tensors."""
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import DistributedLinear
    from distdl_amd.utilities.torch import zero_volume_tensor
    from oracle import repartition as o_rep
    x_ranks, y_ranks = list(x_ranks), list(y_ranks)
    P_fo, P_fi = P_w_shape
    world = max(P_fo * P_fi, x_ranks[-1] + 1, y_ranks[-1] + 1)
    gen = torch.Generator().manual_seed(batch * 100 + c_in)
    x = torch.randn(batch, c_in, generator=gen)
    w = 0.3 * torch.randn(c_out, c_in, generator=gen)
    b = 0.3 * torch.randn(c_out, generator=gen) if use_bias else None
    dy = torch.randn(batch, c_out, generator=gen)
    xs = o_rep.scatter(x.numpy(), P_x_shape)
    dys = o_rep.scatter(dy.numpy(), P_y_shape)
    ws = o_rep.scatter(w.numpy(), P_w_shape)
    bs = o_rep.scatter(b.numpy(), [P_fo]) if use_bias else None

    def body(P_world):
        P_x = P_world.create_partition_inclusive(x_ranks).create_cartesian_topology_partition(P_x_shape)
        P_y = P_world.create_partition_inclusive(y_ranks).create_cartesian_topology_partition(P_y_shape)
        P_w = P_world.create_partition_inclusive(list(range(P_fo * P_fi))).create_cartesian_topology_partition(P_w_shape)
        layer = DistributedLinear(P_x, P_y, P_w, c_in, c_out, bias=use_bias)
        dw = db = None
        if P_w.active:
            with torch.no_grad():
                layer.sublinear.weight.copy_(torch.from_numpy(ws[P_w.rank]))
                if layer.sublinear.bias is not None:
                    assert int(P_w.index[1]) == 0
                    layer.sublinear.bias.copy_(torch.from_numpy(bs[int(P_w.index[0])]))
        xin = torch.from_numpy(xs[P_x.rank]).cuda() if P_x.active else zero_volume_tensor(batch, device="cuda")
        xin.requires_grad = True
        y = layer(xin)
        y.backward(torch.from_numpy(dys[P_y.rank]).cuda() if P_y.active else torch.zeros_like(y))
        torch.cuda.synchronize()
        if P_w.active:
            dw = layer.sublinear.weight.grad.cpu()
            db = layer.sublinear.bias.grad.cpu() if layer.sublinear.bias is not None else None
        return (P_x.rank if P_x.active else None, P_y.rank if P_y.active else None, P_w.rank if P_w.active else None,
                y.detach().cpu(), xin.grad.cpu(), dw, db)

    outs = SimWorld(world).run(body)
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    br = b.clone().requires_grad_(True) if use_bias else None
    yr = F.linear(xr, wr, br)
    yr.backward(dy)
    want_y = o_rep.scatter(yr.detach().numpy(), P_y_shape)
    want_dx = o_rep.scatter(xr.grad.numpy(), P_x_shape)
    want_dw = o_rep.scatter(wr.grad.numpy(), P_w_shape)
    want_db = o_rep.scatter(br.grad.numpy(), [P_fo]) if use_bias else None
    seen = [0, 0, 0, 0]
    for rx, ry, rw, y, dx, dw, db in outs:
        if ry is not None:
            seen[0] += 1
            assert np.allclose(y.numpy(), want_y[ry], rtol=1e-5, atol=1e-5)
        else:
            assert y.numel() == 0
        if rx is not None:
            seen[1] += 1
            assert np.allclose(dx.numpy(), want_dx[rx], rtol=1e-5, atol=1e-5)
        if rw is not None:
            seen[2] += 1
            assert np.allclose(dw.numpy(), want_dw[rw], rtol=1e-5, atol=1e-5)
            if db is not None:
                seen[3] += 1
                assert rw % P_fi == 0 and np.allclose(db.numpy(), want_db[rw // P_fi], rtol=1e-5, atol=1e-5)
    assert seen == [len(y_ranks), len(x_ranks), P_fo * P_fi, P_fo if use_bias else 0]


def _integers(n, shape, seed):
    rng = np.random.default_rng(seed)
    return [rng.integers(-4, 5, size=shape).astype(np.float32) for _ in range(n)]


# (P_x shape, shape of the scattered tensor, shape of the gathered tensor, axis).
# The shapes are "global" in the reference's sense: every worker holds the
# balanced piece of each at its own index.
GATHER_LAYOUTS = [
    pytest.param([2, 3], [2, 3], [4, 3], 0, id="2x3-axis0"),
    pytest.param([2, 3], [2, 3], [2, 9], 1, id="2x3-axis1"),
    pytest.param([4], [4], [16], 0, id="4-axis0"),
    pytest.param([2, 3], [3, 3], [6, 3], 0, id="2x3-axis0-uneven"),
    pytest.param([2, 3], [2, 4], [2, 12], 1, id="2x3-axis1-uneven"),
    pytest.param([4], [6], [24], 0, id="4-axis0-uneven"),
]


def _piece_shapes(P_shape, global_shape):
    from oracle import partition_math as pm
    boxes = pm.boxes_balanced(P_shape, global_shape)
    return [tuple(int(b) - int(a) for a, b in zip(*boxes[idx])) for idx in pm.indices(P_shape)]


def _line_of(rank, P_shape, axis):
    """World ranks of the workers that differ from `rank` along `axis` only, in order."""
    index = list(_index_of(rank, P_shape))
    line = []
    for k in range(P_shape[axis]):
        index[axis] = k
        line.append(int(np.ravel_multi_index(index, P_shape)))
    return line


@pytest.mark.parametrize("P_shape,small_global,big_global,axis", GATHER_LAYOUTS)
def test_all_gather_and_reduce_scatter_reference_layouts(P_shape, small_global, big_global, axis):
    """tests/primitives/test_all_gather.py:10-81 and test_reduce_scatter.py:10-81:
    partitions with a second, untouched dimension and one-dimensional ones, even
    and uneven pieces.  AllGather: every worker ends with the pieces of its line
    along the axis, concatenated in order; ReduceScatter: with its piece of the
    line's sum; each is the other's adjoint.  Small integers, so sums are exact."""
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import AllGather, ReduceScatter
    n = int(np.prod(P_shape))
    small_shapes = _piece_shapes(P_shape, small_global)
    xs = [_integers(1, small_shapes[r], 10 + r)[0] for r in range(n)]
    lines = [_line_of(r, P_shape, axis) for r in range(n)]
    gathered_shapes = []
    for r in range(n):
        shape = list(small_shapes[r])
        shape[axis] = sum(small_shapes[s][axis] for s in lines[r])
        gathered_shapes.append(tuple(shape))
    dys = [_integers(1, gathered_shapes[r], 40 + r)[0] for r in range(n)]
    fulls = [_integers(1, gathered_shapes[r], 70 + r)[0] for r in range(n)]
    dzs = [_integers(1, small_shapes[r], 100 + r)[0] for r in range(n)]

    def body(P_world):
        P_x = P_world.create_partition_inclusive(list(range(n))).create_cartesian_topology_partition(P_shape)
        r = P_x.rank
        xin = torch.from_numpy(xs[r]).cuda().requires_grad_(True)
        y = AllGather(P_x, axes_all_gather=(axis,))(xin)
        y.backward(torch.from_numpy(dys[r]).cuda())
        fin = torch.from_numpy(fulls[r]).cuda().requires_grad_(True)
        z = ReduceScatter(P_x, axes_reduce_scatter=(axis,))(fin)
        z.backward(torch.from_numpy(dzs[r]).cuda())
        torch.cuda.synchronize()
        return y.detach().cpu().numpy(), xin.grad.cpu().numpy(), z.detach().cpu().numpy(), fin.grad.cpu().numpy()

    outs = SimWorld(n).run(body)
    for r, (y, dx, z, dfull) in enumerate(outs):
        line = lines[r]
        me = line.index(r)
        starts = np.cumsum([0] + [small_shapes[s][axis] for s in line])
        mine = [slice(None)] * len(P_shape)
        mine[axis] = slice(int(starts[me]), int(starts[me + 1]))
        assert np.array_equal(y, np.concatenate([xs[s] for s in line], axis=axis)), f"worker {r}"
        assert np.array_equal(dx, sum(dys[s] for s in line)[tuple(mine)]), f"worker {r}"
        assert np.array_equal(z, sum(fulls[s] for s in line)[tuple(mine)]), f"worker {r}"
        assert np.array_equal(dfull, np.concatenate([dzs[s] for s in line], axis=axis)), f"worker {r}"


@pytest.mark.parametrize("P_shape,shape,axes", [
    ([2, 2, 3], [3, 4], ()), ([2, 2, 3], [3, 4], (0,)), ([2, 2, 3], [3, 4], (1,)), ([2, 2, 3], [3, 4], (2,)),
    ([2, 2, 3], [3, 4], (0, 1)), ([2, 2, 3], [3, 4], (0, 2)), ([2, 2, 3], [3, 4], (1, 2)), ([2, 2, 3], [3, 4], (0, 1, 2)),
    ([12], [30, 344], (0,)),
])
def test_all_sum_reduce_reference_layouts(P_shape, shape, axes):
    """tests/primitives/test_all_sum_reduce.py:10-107: twelve workers as
    2 x 2 x 3, reduced along every subset of the axes, and the twelve-way sum
    of a [30, 344] weight; output and gradient are the sums over the workers
    that share the index outside the reduced axes."""
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import AllSumReduce
    n = int(np.prod(P_shape))
    xs = _integers(n, shape, 5)
    dys = _integers(n, shape, 6)

    def body(P_world):
        P_x = P_world.create_partition_inclusive(list(range(n))).create_cartesian_topology_partition(P_shape)
        layer = AllSumReduce(P_x, axes_reduce=axes)
        x = torch.from_numpy(xs[P_x.rank]).cuda().requires_grad_(True)
        y = layer(x)
        y.backward(torch.from_numpy(dys[P_x.rank]).cuda())
        torch.cuda.synchronize()
        return y.detach().cpu().numpy(), x.grad.cpu().numpy()

    outs = SimWorld(n).run(body)
    for r in range(n):
        mine = _index_of(r, P_shape)
        group = [s for s in range(n)
                 if all(a == b for d, (a, b) in enumerate(zip(_index_of(s, P_shape), mine)) if d not in axes)]
        assert len(group) == int(np.prod([P_shape[d] for d in axes])) if axes else group == [r]
        assert np.array_equal(outs[r][0], sum(xs[s] for s in group)), f"worker {r}"
        assert np.array_equal(outs[r][1], sum(dys[s] for s in group)), f"worker {r}"


def test_scale_backward_divides_the_gradients_before_they_are_summed():
    """Broadcast, AllGather and AllSumReduce with ``scale_backward`` (reference:
    backends/mpi_numpy/functional/broadcast.py:208-209, all_gather.py:188-190,
    all_sum_reduce.py:127-128): forward unchanged, every worker's gradient
    divided by the scalar before the adjoint's sum.  Integers and a power of two,
    so the quotients are exact."""
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import AllGather, AllSumReduce, Broadcast
    xs = _integers(4, [2, 6], 21)
    dys = _integers(4, [2, 6], 22)
    dgs = _integers(4, [2, 24], 23)

    def body(P_world):
        r = P_world.rank
        P_one = P_world.create_partition_inclusive([0]).create_cartesian_topology_partition([1, 1])
        P_all = P_world.create_partition_inclusive([0, 1, 2, 3]).create_cartesian_topology_partition([1, 4])
        x = torch.from_numpy(xs[r]).cuda().requires_grad_(True)
        y = Broadcast(P_one, P_all, scale_backward=4)(x)
        y.backward(torch.from_numpy(dys[r]).cuda())
        xa = torch.from_numpy(xs[r]).cuda().requires_grad_(True)
        ya = AllGather(P_all, axes_all_gather=(1,), scale_backward=2)(xa)
        ya.backward(torch.from_numpy(dgs[r]).cuda())
        xr = torch.from_numpy(xs[r]).cuda().requires_grad_(True)
        yr = AllSumReduce(P_all, axes_reduce=(1,), scale_backward=8)(xr)
        yr.backward(torch.from_numpy(dys[r]).cuda())
        torch.cuda.synchronize()
        return (y.detach().cpu().numpy(), x.grad.cpu().numpy(), ya.detach().cpu().numpy(), xa.grad.cpu().numpy(),
                yr.detach().cpu().numpy(), xr.grad.cpu().numpy())

    outs = SimWorld(4).run(body)
    for r, (y, dx, ya, dxa, yr, dxr) in enumerate(outs):
        assert np.array_equal(y, xs[0])
        if r == 0:
            assert np.array_equal(dx, sum(dys) / 4)
        assert np.array_equal(ya, np.concatenate(xs, axis=1))
        assert np.array_equal(dxa, (sum(dgs) / 2)[:, 6 * r:6 * (r + 1)])
        assert np.array_equal(yr, sum(xs))
        assert np.array_equal(dxr, sum(dys) / 8)
