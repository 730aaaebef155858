"""GPU parity of the box-copy kernels (pack / unpack / self copy / zero /
accumulate) and of the Repartition layer built on them, through the C ABI.
Bit-exact against the oracle and the committed golden vectors."""

import numpy as np
import pytest
import torch

from oracle import repartition as o_rep

pytestmark = pytest.mark.gpu

INT_VIEW = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}


def bits(t):
    return t.contiguous().view(INT_VIEW[t.element_size()])


def random_bits(shape, dtype, gen):
    """Tensor of the given dtype filled with random BIT patterns (NaN payloads,
    subnormals, signed zeros included)."""
    es = torch.empty((), dtype=dtype).element_size()
    raw = torch.randint(0, 256, tuple(shape) + (es,), dtype=torch.uint8, generator=gen)
    return raw.view(dtype).reshape(shape)


def to_np_bits(t):
    return bits(t.cpu()).numpy()


@pytest.fixture(scope="module")
def ops():
    import distdl_amd  # noqa: F401
    from distdl_amd import hip_ops
    return hip_ops


def random_boxes(shape, nbox, rng):
    """Disjoint boxes: slabs of a random split of dimension 0, each cropped in
    the other dimensions."""
    cuts = sorted(set(rng.integers(0, shape[0] + 1, size=nbox + 1).tolist()))
    boxes = []
    for a, b in zip(cuts[:-1], cuts[1:]):
        lo, hi = [a], [b]
        for n in shape[1:]:
            x0 = int(rng.integers(0, n))
            x1 = int(rng.integers(x0 + 1, n + 1))
            lo.append(x0)
            hi.append(x1)
        boxes.append(tuple(slice(l, h) for l, h in zip(lo, hi)))
    return boxes


@pytest.mark.parametrize("dtype", [torch.uint8, torch.bfloat16, torch.float32, torch.float64])
@pytest.mark.parametrize("shape", [(37,), (5, 130), (6, 7, 64), (3, 4, 5, 6, 7), (2, 3, 2, 3, 2, 3, 2, 5)])
def test_pack_unpack_random_boxes(ops, dtype, shape):
    gen = torch.Generator().manual_seed(sum(shape) * 64 + torch.empty((), dtype=dtype).element_size())
    rng = np.random.default_rng(len(shape) * 131 + 7)
    x_cpu = random_bits(shape, dtype, gen)
    x = x_cpu.cuda()
    boxes = random_boxes(shape, 5, rng) + [None]
    plan = ops.BoxPlan.from_slices(x, boxes)
    bufs = [None if sl is None else torch.zeros([s.stop - s.start for s in sl], dtype=dtype, device="cuda")
            for sl in boxes]
    plan.pack(x, bufs)
    torch.cuda.synchronize()
    for sl, buf in zip(boxes, bufs):
        if sl is not None:
            assert np.array_equal(to_np_bits(buf), to_np_bits(x_cpu[sl]))
    # unpack into a differently filled tensor: boxes replaced, rest untouched
    y_cpu = random_bits(shape, dtype, gen)
    y = y_cpu.cuda()
    plan.unpack(y, bufs)
    want = bits(y_cpu).clone()
    for sl in boxes:
        if sl is not None:
            want[sl] = bits(x_cpu)[sl]
    assert torch.equal(bits(y.cpu()), want)
    # zero
    plan.zero(y)
    for sl in boxes:
        if sl is not None:
            want[sl] = 0
    assert torch.equal(bits(y.cpu()), want)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.uint8])
@pytest.mark.parametrize("rows,strip,nbox,axis", [
    (64, 1024, 8, 1),      # equal column strips of 2 KiB (bf16): whole tiles of 8 rows, box after box
    (64, 1024, 16, 1),     # a full batch of sixteen boxes
    (16, 1024, 17, 1),     # one more than a launch holds: a batch of sixteen equal boxes and one of one
    (60, 1024, 4, 1),      # rows that are no whole number of tiles: the general kernel
    (64, 1000, 4, 1),      # strips that are no whole number of 16-byte vectors per tile row
    (8, 64, 3, 1),         # tiny
    (4, 40960, 1, 1),      # one box of long contiguous rows
    (6, 32768, 8, 0),      # equal slabs of long runs (64 KiB and more): boxes take turns, 4 KiB per wavefront
    (6, 16384, 2, 0),      # runs of 16 KiB to 64 KiB: box after box, 4 KiB per wavefront
    (3, 8200, 5, 0),       # long runs that are no whole number of tiles
])
def test_equal_boxes_pack_and_unpack_bit_exact(ops, dtype, rows, strip, nbox, axis):
    """Batches of boxes that differ only in their base addresses take a kernel
    of their own when their extents are whole tiles, the general kernel
    otherwise; either way every bit arrives.  Column strips of a matrix
    (axis 1: the pack of a Repartition along the last dimension) and slabs of
    rows (axis 0: its unpack), random bit patterns."""
    gen = torch.Generator().manual_seed(rows * 7 + strip + nbox)
    shape = (rows, strip * nbox) if axis == 1 else (nbox, rows, strip)
    x_cpu = random_bits(shape, dtype, gen)
    x = x_cpu.cuda()
    if axis == 1:
        boxes = [(slice(0, rows), slice(strip * j, strip * (j + 1))) for j in range(nbox)]
    else:
        boxes = [(slice(j, j + 1), slice(0, rows), slice(0, strip)) for j in range(nbox)]
    plan = ops.BoxPlan.from_slices(x, boxes)
    bufs = [torch.zeros([s.stop - s.start for s in sl], dtype=dtype, device="cuda") for sl in boxes]
    plan.pack(x, bufs)
    for sl, buf in zip(boxes, bufs):
        assert np.array_equal(to_np_bits(buf), to_np_bits(x_cpu[sl]))
    y = torch.zeros_like(x)
    plan.unpack(y, bufs[::-1])                         # buffers in reverse: every box lands where its slot says
    want = torch.zeros_like(bits(x_cpu))
    for sl, src in zip(boxes, boxes[::-1]):
        want[sl] = bits(x_cpu)[src]
    assert torch.equal(bits(y.cpu()), want)


def test_pack_from_non_contiguous_tensor(ops):
    gen = torch.Generator().manual_seed(11)
    base = random_bits((9, 12, 10), torch.float32, gen).cuda()
    x = base.permute(2, 0, 1)[:, 1:8, ::2]          # shape (10, 7, 6), awkward strides
    boxes = [(slice(0, 4), slice(1, 6), slice(0, 6)), (slice(4, 10), slice(0, 7), slice(2, 5))]
    plan = ops.BoxPlan.from_slices(x, boxes)
    bufs = [torch.empty([s.stop - s.start for s in sl], dtype=x.dtype, device="cuda") for sl in boxes]
    plan.pack(x, bufs)
    for sl, buf in zip(boxes, bufs):
        assert torch.equal(bits(buf.cpu()), bits(x[sl].cpu()))
    y = torch.zeros_like(base).permute(2, 0, 1)[:, 1:8, ::2]
    ops.BoxPlan.from_slices(y, boxes).unpack(y, bufs)
    for sl in boxes:
        assert torch.equal(bits(y[sl].cpu()), bits(x[sl].cpu()))


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 0), (torch.float64, 0), (torch.bfloat16, 0), (torch.float16, 0)])
def test_accumulating_unpack_matches_torch_add(ops, dtype, tol):
    torch.manual_seed(5)
    y_cpu = torch.randn(6, 33, 10).to(dtype)
    sl = (slice(1, 5), slice(2, 31), slice(0, 10))
    buf_cpu = torch.randn(4, 29, 10).to(dtype)
    y = y_cpu.cuda()
    ops.BoxPlan.from_slices(y, [sl]).unpack(y, [buf_cpu.cuda()], accumulate=True)
    want = y_cpu.clone()
    want[sl] += buf_cpu
    assert torch.equal(bits(y.cpu()), bits(want))


def test_copy_box_strided_to_strided(ops):
    gen = torch.Generator().manual_seed(21)
    src = random_bits((7, 40, 9), torch.bfloat16, gen).cuda()
    dst = random_bits((12, 50, 9), torch.bfloat16, gen).cuda()
    want = bits(dst.cpu()).clone()
    s_sl = (slice(2, 6), slice(5, 37), slice(0, 9))
    d_sl = (slice(8, 12), slice(10, 42), slice(0, 9))
    ops.copy_box(src, s_sl, dst, d_sl)
    want[d_sl] = bits(src.cpu())[s_sl]
    assert torch.equal(bits(dst.cpu()), want)


def test_box_outside_tensor_is_rejected(ops):
    x = torch.zeros(4, 4, device="cuda")
    plan = ops.BoxPlan(x.shape, x.stride(), [([0, 2], [4, 3])])
    with pytest.raises(RuntimeError, match="outside extent"):
        plan.pack(x, [torch.zeros(4, 3, device="cuda")])


def test_cpu_tensor_is_rejected(ops):
    x = torch.zeros(4, 4)
    plan = ops.BoxPlan(x.shape, x.stride(), [([0, 0], [4, 4])])
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        plan.pack(x, [torch.zeros(4, 4)])


# ------------------------------------------------ Repartition, full config --

def test_repartition_config2_rank0_bit_exact(ops):
    """[8,4096,8192] bf16 from P_x=[1,8,1] to P_y=[1,1,8]: rank 0 packs its
    [8,512,8192] shard into 8 boxes of [8,512,1024] and unpacks 8 seeded boxes
    into its [8,4096,1024] output."""
    g = [8, 4096, 8192]
    send, recv, xb, yb = o_rep.plan(g, [1, 8, 1], [1, 1, 8])
    gen = torch.Generator().manual_seed(1002)
    x_cpu = (2 * torch.rand(8, 512, 8192, generator=gen) - 1).to(torch.bfloat16)
    x = x_cpu.cuda()
    send0 = [(sl, sh, 99 if p == "self" else p) for sl, sh, p in send[0]]   # pack all 8, self included
    plan = ops.BoxPlan.from_slices(x, [sl for sl, sh, p in send0])
    bufs = [torch.empty(sh, dtype=torch.bfloat16, device="cuda") for sl, sh, p in send0]
    plan.pack(x, bufs)
    want = o_rep.pack(to_np_bits(x_cpu), send0)
    for b, w in zip(bufs, want):
        assert np.array_equal(to_np_bits(b), w)

    gen2 = torch.Generator().manual_seed(1102)
    recv0 = [(sl, sh, 99 if p == "self" else p) for sl, sh, p in recv[0]]
    rbufs_cpu = [(2 * torch.rand(*sh, generator=gen2) - 1).to(torch.bfloat16) for sl, sh, p in recv0]
    y = torch.empty(8, 4096, 1024, dtype=torch.bfloat16, device="cuda")
    ops.BoxPlan.from_slices(y, [sl for sl, sh, p in recv0]).unpack(y, [b.cuda() for b in rbufs_cpu])
    want_y = o_rep.unpack(recv0, [to_np_bits(b) for b in rbufs_cpu], (8, 4096, 1024), np.int16)
    assert np.array_equal(to_np_bits(y), want_y)
    # size-independent property: unpack(pack(x)) over a matching pair of plans is the identity
    y2 = torch.empty_like(x)
    plan.unpack(y2, bufs)
    assert torch.equal(bits(y2.cpu()), bits(x_cpu))


@pytest.mark.parametrize("nbox,rows,run", [(2, 3, 32768), (3, 5, 40960), (7, 4, 262144), (8, 2, 32768), (5, 3, 32772)])
def test_boxes_with_long_rows_are_walked_round_robin(ops, nbox, rows, run):
    """Boxes of equal size whose rows are long contiguous runs (64 KiB and more)
    share a launch tile by tile in turn instead of box after box: a split of
    dimension 1 of [rows, nbox * run] bf16, packed, unpacked and accumulated.
    7 x 4 x 512 KiB is more tiles than the launch has workgroups; a run of
    32772 elements leaves a ragged last tile in every row."""
    gen = torch.Generator().manual_seed(nbox * 1000 + rows)
    x_cpu = random_bits((rows, nbox * run), torch.bfloat16, gen)
    x = x_cpu.cuda()
    slices = [(slice(0, rows), slice(b * run, (b + 1) * run)) for b in range(nbox)]
    plan = ops.BoxPlan.from_slices(x, slices)
    bufs = [torch.empty(rows, run, dtype=torch.bfloat16, device="cuda") for _ in range(nbox)]
    plan.pack(x, bufs)
    for b, sl in zip(bufs, slices):
        assert torch.equal(bits(b.cpu()), bits(x_cpu[sl]))
    y = torch.empty_like(x)
    plan.unpack(y, bufs)
    assert torch.equal(bits(y.cpu()), bits(x_cpu))
    # accumulate: every element exactly once
    acc_cpu = torch.randint(-8, 9, (rows, nbox * run), generator=gen).to(torch.float32)
    add_cpu = [torch.randint(-8, 9, (rows, run), generator=gen).to(torch.float32) for _ in range(nbox)]
    acc = acc_cpu.cuda()
    ops.BoxPlan.from_slices(acc, slices).unpack(acc, [a.cuda() for a in add_cpu], accumulate=True)
    assert torch.equal(acc.cpu(), acc_cpu + torch.cat(add_cpu, dim=1))


# ---------------------------------------------- Repartition layer, loopback --

def _run_repartition_world(world_size, P_x_workers, P_x_shape, P_y_workers, P_y_shape, x_by_rank, dy_by_rank, dtype,
                           preserve_batch=False):
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import Repartition
    from distdl_amd.utilities.torch import zero_volume_tensor

    def body(P_world):
        P_x = P_world.create_partition_inclusive(P_x_workers).create_cartesian_topology_partition(P_x_shape)
        P_y = P_world.create_partition_inclusive(P_y_workers).create_cartesian_topology_partition(P_y_shape)
        layer = Repartition(P_x, P_y, preserve_batch=preserve_batch)
        x = zero_volume_tensor(device="cuda", dtype=dtype)
        if P_x.active:
            x = x_by_rank[P_x.rank].to(dtype).cuda()
        x.requires_grad = True
        y = layer(x)
        dy = zero_volume_tensor(device="cuda", dtype=dtype)
        if P_y.active:
            dy = dy_by_rank[P_y.rank].to(dtype).cuda()
        y.backward(dy)
        torch.cuda.synchronize()
        return (P_x.rank if P_x.active else None, P_y.rank if P_y.active else None,
                y.detach().cpu(), x.grad.cpu() if x.grad is not None else None, layer)

    return SimWorld(world_size).run(body)


# The rank layouts of the reference's own adjoint test (tests/primitives/test_repartition.py:11-127):
# (P_x ranks, P_x shape, P_y ranks, P_y shape, world size), global tensor [77, 55].
REFERENCE_LAYOUTS = {
    "distributed-overlap": (range(4, 8), [4, 1], range(0, 12), [3, 4], 12),
    "distributed-disjoint": (range(0, 4), [4, 1], range(4, 16), [3, 4], 16),
    "distributed-disjoint-inactive": (range(0, 4), [4, 1], range(5, 17), [3, 4], 17),
    "sequential-identity": (range(0, 1), [1, 1], range(0, 1), [1, 1], 1),
    "as_scatter-overlap": (range(4, 5), [1, 1], range(0, 12), [3, 4], 12),
    "as_scatter-disjoint": (range(0, 1), [1, 1], range(1, 13), [3, 4], 13),
    "as_scatter-disjoint-inactive": (range(0, 1), [1, 1], range(2, 14), [3, 4], 14),
    "as_gather-overlap": (range(0, 12), [3, 4], range(4, 5), [1, 1], 12),
    "as_gather-disjoint": (range(1, 13), [3, 4], range(0, 1), [1, 1], 13),
    "as_gather-disjoint-inactive": (range(2, 14), [3, 4], range(0, 1), [1, 1], 14),
}


def _shard_bounds(extent, parts, balanced):
    """[start, stop) of every part of one dimension: the balanced split, or the
    reference test's unbalanced one (part 0 takes the whole remainder,
    test_repartition.py:176-181)."""
    q, r = divmod(extent, parts)
    sizes = [q + (1 if i < r else 0) for i in range(parts)] if balanced else [q + (r if i == 0 else 0) for i in range(parts)]
    starts = np.concatenate([[0], np.cumsum(sizes)])
    return [(int(starts[i]), int(starts[i + 1])) for i in range(parts)]


@pytest.mark.parametrize("balanced", [True, False])
@pytest.mark.parametrize("layout", list(REFERENCE_LAYOUTS))
def test_repartition_reference_adjoint_layouts(layout, balanced):
    """The reference's test_repartition_adjoint on its own parametrisation:
    overlapping, disjoint and partly idle teams; scatter and gather shapes;
    balanced input shards and the unbalanced ones the reference feeds it.
    Checked three ways: y is the balanced split of the global tensor the x
    shards form, dx the x-shaped split of the global dy (both exact), and the
    reference's own criterion <F x, dy> = <x, F* dy>."""
    P_x_ranks, P_x_shape, P_y_ranks, P_y_shape, world = REFERENCE_LAYOUTS[layout]
    shape = [77, 55]
    gen = torch.Generator().manual_seed(len(layout) * 2 + balanced)
    gx, gdy = torch.randn(*shape, generator=gen), torch.randn(*shape, generator=gen)
    xb = [_shard_bounds(shape[d], P_x_shape[d], balanced) for d in range(2)]
    yb = [_shard_bounds(shape[d], P_y_shape[d], True) for d in range(2)]

    def split(t, bounds, pshape):
        return [t[bounds[0][i][0]:bounds[0][i][1], bounds[1][j][0]:bounds[1][j][1]].contiguous()
                for i in range(pshape[0]) for j in range(pshape[1])]       # row-major rank order
    xs, dys = split(gx, xb, P_x_shape), split(gdy, yb, P_y_shape)
    want_y, want_dx = split(gx, yb, P_y_shape), split(gdy, xb, P_x_shape)
    res = _run_repartition_world(world, list(P_x_ranks), P_x_shape, list(P_y_ranks), P_y_shape, xs, dys, torch.float32)
    ipx = ipy = 0.0
    seen_x, seen_y = set(), set()
    for xr, yr, y, dx, layer in res:
        if yr is not None:
            assert torch.equal(y, want_y[yr])
            ipy += float((y.double() * dys[yr].double()).sum())
            seen_y.add(yr)
        else:
            assert y.numel() == 0
        if xr is not None:
            assert torch.equal(dx, want_dx[xr])
            ipx += float((xs[xr].double() * dx.double()).sum())
            seen_x.add(xr)
    assert len(seen_x) == len(xs) and len(seen_y) == len(dys)
    d = max(float(gx.norm() * gdy.norm()), 1e-30)
    assert np.isclose(ipx / d, ipy / d)


@pytest.mark.parametrize("dtype,test_backward", [(torch.float32, True), (torch.int32, False), (torch.float64, True)])
def test_repartition_reference_dtype_cases(dtype, test_backward):
    """The reference's test_repartition_dtype (tests/primitives/test_repartition.py:428-546):
    [77, 55] from a 4 x 1 to a 2 x 2 partition of the same four workers in
    float32, int32 (no gradient) and float64; the output, and the gradient where
    there is one, keep the dtype -- and here also the values."""
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import Repartition
    shape, P_x_shape, P_y_shape = [77, 55], [4, 1], [2, 2]
    gen = torch.Generator().manual_seed(17)
    gx = (10 * torch.randn(*shape, generator=gen)).to(dtype)
    gdy = (10 * torch.randn(*shape, generator=gen)).to(dtype)
    xb = [_shard_bounds(shape[d], P_x_shape[d], True) for d in range(2)]
    yb = [_shard_bounds(shape[d], P_y_shape[d], True) for d in range(2)]

    def split(t, bounds, pshape):
        return [t[bounds[0][i][0]:bounds[0][i][1], bounds[1][j][0]:bounds[1][j][1]].contiguous()
                for i in range(pshape[0]) for j in range(pshape[1])]
    xs, dys = split(gx, xb, P_x_shape), split(gdy, yb, P_y_shape)
    want_y, want_dx = split(gx, yb, P_y_shape), split(gdy, xb, P_x_shape)

    def body(P_world):
        P_x = P_world.create_partition_inclusive([0, 1, 2, 3]).create_cartesian_topology_partition(P_x_shape)
        P_y = P_world.create_partition_inclusive([0, 1, 2, 3]).create_cartesian_topology_partition(P_y_shape)
        layer = Repartition(P_x, P_y, preserve_batch=False)
        x = xs[P_x.rank].cuda()
        x.requires_grad = test_backward
        y = layer(x)
        dx = None
        if test_backward:
            y.backward(dys[P_y.rank].cuda())
            dx = x.grad.cpu()
        torch.cuda.synchronize()
        return P_x.rank, P_y.rank, y.detach().cpu(), dx

    for xr, yr, y, dx in SimWorld(4).run(body):
        assert y.dtype == dtype and torch.equal(y, want_y[yr])
        if test_backward:
            assert dx.dtype == dtype and torch.equal(dx, want_dx[xr])


def test_repartition_layer_golden_example(golden):
    g = golden("repartition_7x5.json")
    xs = [torch.tensor(a) for a in g["input_by_x_rank"]]
    dys = [torch.tensor(a) for a in g["adjoint_input_by_y_rank"]]
    for world, y_workers in ((4, [0, 1, 2, 3]), (8, [4, 5, 6, 7])):       # shared team / disjoint teams
        res = _run_repartition_world(world, [0, 1, 2, 3], g["P_x_shape"], y_workers, g["P_y_shape"], xs, dys,
                                     torch.float16)
        for xr, yr, y, dx, layer in res:
            if yr is not None:
                assert torch.equal(y, torch.tensor(g["forward_by_y_rank"][yr], dtype=torch.float16))
            if xr is not None:
                assert torch.equal(dx, torch.tensor(g["adjoint_by_x_rank"][xr], dtype=torch.float16))


@pytest.mark.parametrize("shape,P_x,P_y", [([3, 10, 11], [1, 4, 1], [1, 1, 4]), ([5, 6, 7], [2, 3, 1], [1, 2, 2]),
                                          ([4, 9], [1, 1], [2, 3]), ([2, 16, 24], [1, 4, 2], [1, 2, 4])])
def test_repartition_layer_matches_oracle(shape, P_x, P_y):
    gen = torch.Generator().manual_seed(31)
    x = random_bits(shape, torch.bfloat16, gen)
    dy = random_bits(shape, torch.bfloat16, gen)
    nx, ny = int(np.prod(P_x)), int(np.prod(P_y))
    xs = [torch.from_numpy(a.copy()).view(torch.bfloat16) for a in o_rep.scatter(bits(x).numpy(), P_x)]
    dys = [torch.from_numpy(a.copy()).view(torch.bfloat16) for a in o_rep.scatter(bits(dy).numpy(), P_y)]
    world = max(nx, ny)
    res = _run_repartition_world(world, list(range(nx)), P_x, list(range(ny)), P_y, xs, dys, torch.bfloat16)
    want_y = o_rep.forward_all([bits(a).numpy() for a in xs], shape, P_x, P_y, shared_workers=True)
    want_dx = o_rep.adjoint_all([bits(a).numpy() for a in dys], shape, P_x, P_y, shared_workers=True)
    for xr, yr, y, dx, layer in res:
        if yr is not None:
            assert np.array_equal(bits(y).numpy(), want_y[yr])
        if xr is not None:
            assert np.array_equal(bits(dx).numpy(), want_dx[xr])


def test_identity_repartition_only_self_overlaps():
    xs = [torch.randn(3, 4) for _ in range(4)]
    res = _run_repartition_world(4, [0, 1, 2, 3], [2, 2], [0, 1, 2, 3], [2, 2], xs, xs, torch.float32)
    for xr, yr, y, dx, layer in res:
        assert torch.equal(y, xs[xr]) and torch.equal(dx, xs[xr])
        for lst in (layer.P_x_to_y_overlaps, layer.P_y_to_x_overlaps):
            assert [p for sl, sh, p in lst if sl is not None] == ["self"]


def test_transpose_network_buffers_and_adjoint(golden):
    """The four chained repartitions of the reference's buffer test
    (tests/utilities/test_buffer.py:128-222): buffer counts per rank after each
    layer, and <Fx, dy> == <x, F*dy> through the whole chain."""
    from distdl_amd.backends.stub_hip import BufferManager
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import Repartition
    from distdl_amd.utilities.torch import zero_volume_tensor
    g = golden("buffer_network.json")["transpose_network"]
    torch.manual_seed(9)
    x0, dy0 = torch.randn(1, 10), torch.randn(1, 10)

    def body(P_world):
        manager = BufferManager()
        parts = {}
        for name, spec in g["partitions"].items():
            parts[name] = P_world.create_partition_inclusive(spec["workers"]).create_cartesian_topology_partition(
                spec["shape"])
        layers = [Repartition(parts[a], parts[b], buffer_manager=manager) for a, b in g["layers"]]
        x = zero_volume_tensor(1, device="cuda")
        if parts["P_1"].active:
            x = x0.cuda()
        x.requires_grad = True
        counts = []
        h = x
        for layer in layers:
            h = layer(h)
            counts.append(len(manager.buffers_map[torch.float32]))
        dy = zero_volume_tensor(1, device="cuda")
        if parts["P_1"].active:
            dy = dy0.cuda()
        h.backward(dy)
        counts.append(len(manager.buffers_map[torch.float32]))
        return counts, h.detach().cpu(), x.grad.cpu()

    res = SimWorld(4).run(body)
    for rank, (counts, y, dx) in enumerate(res):
        assert counts[:4] == [c[rank] for c in g["n_buffers_by_rank_after_layer"]]
        assert counts[4] == counts[3]
    y, dx = res[0][1], res[0][2]
    assert torch.equal(y, x0)                      # scatter ... gather is the identity
    assert torch.equal(dx, dy0)


# ------------------------------------------------- all-gather / reduce-scatter --

@pytest.mark.parametrize("P,shape,axis", [([1, 4], [3, 10], 1), ([3, 1, 1], [7, 2, 5], 0), ([1, 2, 1], [2, 9, 4], 1),
                                          ([1, 1, 4], [2, 3, 8], 2)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_all_gather_and_reduce_scatter_layers(P, shape, axis, dtype):
    """Loopback over all workers.  AllGather: every worker ends with the
    concatenation of the (possibly uneven) shards, bit for bit; its backward is
    the reduce-scatter of the gradients.  ReduceScatter: the slab of the sum;
    its backward is the all-gather.  Values are small integers, so the sums are
    exact in either dtype."""
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import AllGather
    from distdl_amd.nn import ReduceScatter
    from oracle import relayout as o_rl
    from oracle import repartition as o_rep
    n = int(np.prod(P))
    rng = np.random.default_rng(sum(shape) + axis)
    x = rng.integers(-3, 4, size=shape).astype(np.float32)
    shards = o_rep.scatter(x, P)                                   # balanced split, first workers larger
    dys = [rng.integers(-3, 4, size=shape).astype(np.float32) for _ in range(n)]
    fulls = [rng.integers(-3, 4, size=shape).astype(np.float32) for _ in range(n)]
    dzs = o_rep.scatter(rng.integers(-3, 4, size=shape).astype(np.float32), P)

    def body(P_world):
        P_x = P_world.create_partition_inclusive(list(range(n))).create_cartesian_topology_partition(P)
        r = P_x.rank
        xin = torch.from_numpy(shards[r]).to(dtype).cuda().requires_grad_(True)
        y = AllGather(P_x, axes_all_gather=(axis,))(xin)
        y.backward(torch.from_numpy(dys[r]).to(dtype).cuda())
        fin = torch.from_numpy(fulls[r]).to(dtype).cuda().requires_grad_(True)
        z = ReduceScatter(P_x, axes_reduce_scatter=(axis,))(fin)
        z.backward(torch.from_numpy(dzs[r]).to(dtype).cuda())
        xs = torch.from_numpy(shards[r]).to(dtype).cuda().requires_grad_(True)
        AllGather(P_x, axes_all_gather=(axis,), scale_backward=4)(xs).backward(torch.from_numpy(dys[r]).to(dtype).cuda())
        torch.cuda.synchronize()
        return (y.detach().float().cpu().numpy(), xin.grad.float().cpu().numpy(),
                z.detach().float().cpu().numpy(), fin.grad.float().cpu().numpy(), xs.grad.float().cpu().numpy())

    outs = SimWorld(n).run(body)
    want_dx = o_rep.scatter(sum(dys), P)
    want_z = o_rep.scatter(sum(fulls), P)
    dz_full = np.concatenate([dzs[r] for r in range(n)], axis=axis)
    # the oracle's restatement of the reference's pad / gather / rearrange / strip sequence, all workers at once
    o_y = o_rl.all_gather(shards, axis)
    o_dx = o_rl.all_gather_adjoint(dys, axis)
    o_z = o_rl.reduce_scatter(fulls, axis)
    o_dfull = o_rl.reduce_scatter_adjoint(dzs, axis)
    o_dx_scaled = o_rl.all_gather_adjoint(dys, axis, scale_backward=4)      # quarters of small integers: exact in bf16 too
    for r, (y, dx, z, dfull, dx_scaled) in enumerate(outs):
        assert np.array_equal(dx_scaled, o_dx_scaled[r])
        assert np.array_equal(y, x) and np.array_equal(y, o_y)
        assert np.array_equal(dx, want_dx[r]) and np.array_equal(dx, o_dx[r])
        assert np.array_equal(z, want_z[r]) and np.array_equal(z, o_z[r])
        assert np.array_equal(dfull, dz_full) and np.array_equal(dfull, o_dfull[r])


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
def test_box_accumulate_integers_wrap_around(dtype):
    """dst += src on integer boxes (the forward-only integer cases of the
    reference's reduction tests): exact, and two's-complement wrap-around at
    the ends of the range, as NumPy and ATen add."""
    from distdl_amd import hip_ops
    info = torch.iinfo(dtype)
    gen = torch.Generator().manual_seed(3)
    src = torch.randint(-1000, 1000, (5, 37, 19), generator=gen).to(dtype)
    dst = torch.randint(-1000, 1000, (7, 40, 23), generator=gen).to(dtype)
    src[0, 0, 0], dst[1, 2, 3] = info.max, 5            # wraps to min + 4
    src[4, 36, 18], dst[5, 38, 21] = info.min, -1       # wraps to max
    want = dst.clone()
    want[1:6, 2:39, 3:22] += src
    assert int(want[1, 2, 3]) == info.min + 4 and int(want[5, 38, 21]) == info.max
    d = dst.cuda()
    hip_ops.copy_box(src.cuda(), [slice(0, 5), slice(0, 37), slice(0, 19)], d, [slice(1, 6), slice(2, 39), slice(3, 22)],
                     accumulate=True)
    assert torch.equal(d.cpu(), want)


# ------------------------------------------------------------- sum of boxes --

def _sequential_sum(srcs, divisor):
    """What ddl_sum_boxes promises: every source divided (true division, in
    fp32 for the 16-bit types, rounded to the element type), then added in
    order with a rounding after every addition -- torch on the CPU, step by step."""
    acc = None
    for s in srcs:
        t = s if divisor == 1 else (s / divisor).to(s.dtype)
        acc = t.clone() if acc is None else (acc + t).to(s.dtype)
    return acc


@pytest.mark.parametrize("dtype,nsrc,divisor", [
    (dtype, nsrc, divisor)
    for dtype in (torch.float32, torch.float64, torch.bfloat16, torch.float16, torch.int32, torch.int64)
    for nsrc, divisor in ((1, 1), (1, 3), (3, 1), (8, 7), (64, 2))
    if dtype.is_floating_point or divisor == 1])          # integers are summed, not divided
def test_sum_boxes_matches_step_by_step_arithmetic(ops, dtype, nsrc, divisor):
    """One launch = the chain of divisions and additions, bit for bit, on a
    strided box of every source into a strided box of the destination."""
    gen = torch.Generator().manual_seed(nsrc * 100 + divisor)
    shape, box = (5, 9, 44), (slice(1, 5), slice(2, 9), slice(4, 41))
    if dtype.is_floating_point:
        srcs = [(torch.randn(shape, generator=gen) * 3).to(dtype) for _ in range(nsrc)]
    else:
        srcs = [torch.randint(-2 ** 30, 2 ** 30, shape, generator=gen).to(dtype) for _ in range(nsrc)]
        srcs[0][1, 2, 4] = torch.iinfo(dtype).max          # wraps around with the next addend
        if nsrc > 1:
            srcs[1][1, 2, 4] = 9
    dst = torch.full((6, 8, 50), 5, dtype=dtype)
    dbox = (slice(2, 6), slice(0, 7), slice(10, 47))
    want = dst.clone()
    want[dbox] = _sequential_sum([s[box] for s in srcs], divisor)
    d = dst.cuda()
    ops.sum_boxes([s.cuda() for s in srcs], box, d, dbox, divisor)
    assert torch.equal(bits(d.cpu()), bits(want))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16, torch.float16, torch.int32, torch.int64])
@pytest.mark.parametrize("nsrc", [5, 8, 13])
@pytest.mark.parametrize("rows,row_elems,pitch_elems", [
    (64, 128, 128 * 3),        # rows of 256 / 512 B: eight or four rows per quarter tile
    (24, 1024, 8192),          # the re-layout's rows (2 KiB in bf16), 8 rows per tile
    (6, 4096, 4096 * 2),       # rows longer than a quarter tile
    (1, 16384 * 3, 16384 * 3), # one contiguous run
])
def test_sum_boxes_of_many_sources_over_whole_tiles(ops, dtype, nsrc, rows, row_elems, pitch_elems):
    """Five and more sources over boxes made of whole tiles take the kernel
    that has eight sources in flight per quarter tile: the same step-by-step
    arithmetic, also divided, also into one of the sources, on row lengths on
    either side of a quarter tile."""
    gen = torch.Generator().manual_seed(nsrc * 7 + rows)
    es = torch.empty((), dtype=dtype).element_size()
    row_elems, pitch_elems = max(row_elems * 4 // es, 16 // es), pitch_elems * 4 // es
    if dtype.is_floating_point:
        srcs = [(torch.randn(rows, pitch_elems, generator=gen) * 3).to(dtype) for _ in range(nsrc)]
    else:
        srcs = [torch.randint(-2 ** 30, 2 ** 30, (rows, pitch_elems), generator=gen).to(dtype) for _ in range(nsrc)]
    first = pitch_elems - row_elems if pitch_elems > row_elems else 0
    box = (slice(0, rows), slice(first, first + row_elems))
    full = (slice(0, rows), slice(0, row_elems))
    for divisor in ((1, 4, 3) if dtype.is_floating_point else (1,)):
        want = _sequential_sum([t[box] for t in srcs], divisor)
        out = torch.zeros(rows, row_elems, dtype=dtype, device="cuda")
        dev = [t.cuda() for t in srcs]
        ops.sum_boxes(dev, box, out, full, divisor)
        assert torch.equal(bits(out.cpu()), bits(want))
        ops.sum_boxes(dev, box, dev[2], box, divisor)                  # into the third source
        assert torch.equal(bits(dev[2].cpu()[box]), bits(want))
        untouched = torch.ones(rows, pitch_elems, dtype=torch.bool)
        untouched[box] = False
        assert torch.equal(bits(dev[2].cpu())[untouched], bits(srcs[2])[untouched])


def test_sum_boxes_in_place_and_fallbacks(ops):
    """The destination may be one of the sources (scaling a gradient in place);
    sources that are not 16 bytes apart, or more than 64 of them, go through
    the same arithmetic one source at a time; bad arguments are refused."""
    gen = torch.Generator().manual_seed(5)
    x = torch.randn(7, 33, generator=gen)
    full = (slice(0, 7), slice(0, 33))
    d = x.cuda()
    ops.sum_boxes([d], full, d, full, 3)
    assert torch.equal(d.cpu(), x / 3)
    assert torch.equal(ops.scaled(x.cuda().t(), 5).cpu(), (x / 5).t())
    pool = torch.randn(3 * 7 * 33 + 8, generator=gen).cuda()
    odd = [pool[1 + q * 231: 1 + (q + 1) * 231].view(7, 33) for q in range(3)]       # 4 bytes past a 16-byte boundary, 924 apart
    odd[1] = pool[2 + 231: 2 + 2 * 231].view(7, 33)
    out = torch.empty(7, 33, device="cuda")
    ops.sum_boxes(odd, full, out, full)
    assert torch.equal(out.cpu(), _sequential_sum([t.cpu() for t in odd], 1))
    ops.sum_boxes(odd, full, out, full, 3)
    assert torch.equal(out.cpu(), _sequential_sum([t.cpu() for t in odd], 3))
    many = [torch.full((4, 8), float(q), device="cuda") for q in range(70)]
    out = torch.empty(4, 8, device="cuda")
    ops.sum_boxes(many, (slice(0, 4), slice(0, 8)), out, (slice(0, 4), slice(0, 8)))
    assert torch.equal(out.cpu(), torch.full((4, 8), float(sum(range(70)))))
    with pytest.raises(ValueError):
        ops.sum_boxes([x.cuda(), x.cuda().double()], full, out, full)
    from distdl_amd import _lib
    lib = _lib.load()
    box = _lib.ddl_box_t()
    box.ndim = 1
    box.shape[0], box.src_stride[0], box.dst_stride[0] = 8, 1, 1
    box.dst = out.data_ptr()
    ptrs = _lib.ptr_array([x.cuda().data_ptr()])
    assert lib.ddl_sum_boxes(box, ptrs, 0, 4, _lib.DDL_DT_F32, 1.0, None) == -5
    assert lib.ddl_sum_boxes(box, ptrs, 1, 4, _lib.DDL_DT_F32, 0.0, None) == -1
    assert lib.ddl_sum_boxes(box, ptrs, 1, 4, _lib.DDL_DT_I32, 2.0, None) == -5
    assert lib.ddl_sum_boxes(box, ptrs, 1, 2, _lib.DDL_DT_F32, 1.0, None) == -1


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("divisor", [2, 8, 0.25, -4, 2.0 ** 40, 2.0 ** -40, 3, 7, 10, -6, 1e-3])
def test_sum_boxes_divides_every_16_bit_pattern_like_true_division(ops, dtype, divisor):
    """All 65 536 bit patterns of a 16-bit type, zeros, subnormals, infinities
    and NaNs included, divided by powers of two (which the kernel multiplies by
    the exact reciprocal) and by other numbers (which it divides by): the bits
    of the quotient computed in fp32 and rounded once to the element type.  NaNs
    are compared as NaNs: the CPU's own conversions do not agree on their bits."""
    x = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16).view(dtype)
    want = (x.float() / divisor).to(dtype)
    got = ops.scaled(x.cuda(), divisor).cpu()
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan)
    assert torch.equal(bits(got)[~nan], bits(want)[~nan])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_box_add_of_every_16_bit_pattern(ops, dtype):
    """All 65 536 bit patterns of a 16-bit type plus a handful of partners
    (zeros, the smallest subnormal, numbers that cancel or tie, the largest
    finite one, infinity): the sum computed in fp32 and rounded once to nearest
    even, through the accumulating copy and through the sum of two sources."""
    x = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16).view(dtype)
    info = torch.finfo(dtype)
    partners = torch.tensor([0.0, -0.0, 1.0, -1.0, 1.0 + info.eps, 3 * info.eps / 2, info.tiny, -info.tiny * 0.5, info.max, -info.max,
                             float("inf"), 0.3, -255.0], dtype=torch.float32).to(dtype)
    smallest = torch.tensor([1], dtype=torch.int16).view(dtype)
    full = (slice(0, 65536),)
    for p in list(partners) + [smallest[0]]:
        y = p.expand(65536).contiguous()
        want = (x.float() + y.float()).to(dtype)
        nan = torch.isnan(want)
        d = y.cuda()
        ops.copy_box(x.cuda(), full, d, full, accumulate=True)
        got = d.cpu()
        assert torch.equal(torch.isnan(got), nan)
        assert torch.equal(bits(got)[~nan], bits(want)[~nan])
        out = torch.empty(65536, dtype=dtype, device="cuda")
        ops.sum_boxes([x.cuda(), y.cuda()], full, out, full)
        assert torch.equal(bits(out.cpu())[~nan], bits(want)[~nan])


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("divisor", [2, 0.125, -16, 2.0 ** 60, 2.0 ** -60, 3, 1e-3])
def test_sum_boxes_divides_special_values_like_true_division(ops, dtype, divisor):
    """Subnormal, tiny, huge and non-finite inputs and quotients in fp32 and
    fp64: the product with the reciprocal of a power of two is the quotient
    itself, also where it underflows or overflows."""
    info = torch.finfo(dtype)
    gen = torch.Generator().manual_seed(17)
    special = torch.tensor([0.0, -0.0, info.tiny, -info.tiny, info.tiny / 8, info.tiny * 0.75, info.tiny * 1.5, info.max, -info.max,
                            info.max / 3, info.eps, 1.0, -1.0, float("inf"), float("-inf"), float("nan"),
                            info.smallest_normal * (1 + info.eps), 5e-324 if dtype == torch.float64 else 1.4e-45], dtype=dtype)
    spread = (torch.randn(4096, generator=gen, dtype=torch.float64)
              * torch.exp2(torch.randint(-140, 128, (4096,), generator=gen).double())).to(dtype)
    x = torch.cat([special, spread])
    want = x / divisor
    got = ops.scaled(x.cuda(), divisor).cpu()
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan)
    assert torch.equal(bits(got)[~nan], bits(want)[~nan])


def test_reduce_scatter_relayout_at_config4_activation_size(ops):
    """The local half of a reduce-scatter over 8 workers at the activation
    shape of configuration 4 ([4,2048,8192] bf16, split along the features):
    the own slab of the sum of eight full tensors in one launch, against the
    step-by-step sum on sampled rows and against linearity (the sum of A and of
    B, scaled by powers of two, is exact)."""
    gen = torch.Generator(device="cuda").manual_seed(77)
    fulls = [torch.randn(4, 2048, 8192, generator=gen, device="cuda").to(torch.bfloat16) for _ in range(8)]
    src = (slice(0, 4), slice(0, 2048), slice(3072, 4096))           # worker 3's slab
    dst = (slice(0, 4), slice(0, 2048), slice(0, 1024))
    out = torch.empty(4, 2048, 1024, dtype=torch.bfloat16, device="cuda")
    ops.sum_boxes(fulls, src, out, dst)
    rows = [0, 1, 777, 2047]
    want = _sequential_sum([f[:, rows, 3072:4096].cpu() for f in fulls], 1)
    assert torch.equal(bits(out[:, rows].cpu()), bits(want))
    doubled = torch.empty_like(out)
    ops.sum_boxes([ops.scaled(f, 0.5) for f in fulls], src, doubled, dst)        # every addend times two
    quartered = torch.empty_like(out)
    ops.sum_boxes(fulls, src, quartered, dst, 4)
    assert torch.equal(bits(doubled.cpu()), bits((out.float() * 2).to(torch.bfloat16).cpu()))
    assert torch.equal(bits(quartered.cpu()), bits((out.float() / 4).to(torch.bfloat16).cpu()))
