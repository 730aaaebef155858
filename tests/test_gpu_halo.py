"""GPU parity of the halo path: HaloExchange layer (forward and adjoint), the
fused pad + ghost fill + bulk pack kernel, and the staging of the feature
convolution.  Bit-exact against the oracle and the committed golden vectors;
the convolution end-to-end check uses the reference's own tolerance."""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import halo as o_halo
from oracle import partition_math as pm
from oracle import repartition as o_rep

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import distdl_amd  # noqa: F401
    from distdl_amd import hip_ops
    return hip_ops


def _world_geometry(P, gshape, kernel, stride, dilation):
    recv, send, halo = {}, {}, {}
    for idx in pm.indices(P):
        h, rc, sd, _ = o_halo.exchange_info(gshape, kernel, stride, [0] * len(kernel), dilation, P, idx)
        halo[idx], recv[idx], send[idx] = h, rc, sd
    return halo, recv, send


def _run_halo_world(P, padded_by_rank, dy_by_rank, halo, recv, send):
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import HaloExchange
    order = pm.indices(P)

    def body(P_world):
        P_x = P_world.create_partition_inclusive(list(range(len(order)))).create_cartesian_topology_partition(list(P))
        idx = order[P_x.rank]
        layer = HaloExchange(P_x, np.array(halo[idx]), np.array(recv[idx]), np.array(send[idx]))
        x = padded_by_rank[P_x.rank].cuda()
        x.requires_grad = True
        y = layer(x)
        y.backward(dy_by_rank[P_x.rank].cuda())
        torch.cuda.synchronize()
        return y.detach().cpu(), x.grad.cpu(), layer

    return SimWorld(len(order)).run(body)


def test_halo_exchange_golden_example(golden):
    g = golden("halo_exchange_2x2.json")
    P = tuple(g["partition_shape"])
    halo, recv, send = _world_geometry(P, g["x_global_shape"], g["kernel_size"], g["stride"], g["dilation"])
    padded = [torch.tensor(m, dtype=torch.float32)[None, None] for m in g["padded_input"]]
    dys = [torch.full_like(p, float(c)) for p, c in zip(padded, g["adjoint_input_constant_per_rank"])]
    res = _run_halo_world(P, padded, dys, halo, recv, send)
    for r, (y, dx, layer) in enumerate(res):
        assert torch.equal(y[0, 0], torch.tensor(g["forward"][r], dtype=torch.float32))
        assert torch.equal(dx[0, 0], torch.tensor(g["adjoint"][r], dtype=torch.float32))
        assert len(layer.buffer_manager.buffers_map[torch.float32]) == 4


@pytest.mark.parametrize("P,gshape,kernel", [((1, 1, 3, 3), [1, 2, 12, 13], [3, 5]), ((1, 2, 2), [2, 3, 17], [5]),
                                             ((1, 1, 2, 1, 2), [1, 2, 9, 5, 10], [3, 3, 5]),
                                             ((1, 1, 2, 2, 2), [1, 3, 8, 8, 8], [3, 3, 3])])
def test_halo_exchange_layer_matches_oracle(P, gshape, kernel):
    nf = len(kernel)
    halo, recv, send = _world_geometry(P, gshape, kernel, [1] * nf, [1] * nf)
    gen = torch.Generator().manual_seed(41)
    order = pm.indices(P)
    padded, dys = {}, {}
    for idx in order:
        shape = [n + a + b for n, (a, b) in zip(pm.subshape(P, idx, gshape), halo[idx])]
        padded[idx] = torch.randn(shape, generator=gen)
        dys[idx] = torch.randn(shape, generator=gen)
    res = _run_halo_world(P, [padded[i] for i in order], [dys[i] for i in order], halo, recv, send)
    want_y = o_halo.forward_all({i: padded[i].numpy() for i in order}, P, recv, send)
    want_dx = o_halo.adjoint_all({i: dys[i].numpy() for i in order}, P, recv, send)
    for idx, (y, dx, layer) in zip(order, res):
        assert np.array_equal(y.numpy(), want_y[idx])          # pure moves: bit-exact
        assert np.array_equal(dx.numpy(), want_dx[idx])        # one add per element: bit-exact in fp32


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("P,gshape,kernel,stride", [((1, 1, 3, 3), [1, 1, 10, 7], [3, 3], [1, 1]),
                                                    ((1, 1, 3), [1, 1, 10], [2], [2])])
def test_halo_exchange_reference_adjoint_cases(P, gshape, kernel, stride, dtype):
    """The reference's test_halo_exchange_adjoint on its own parametrisation
    (tests/primitives/test_halo_exchange.py:24-88: 3 x 3 workers on [1,1,10,7]
    with a 3 x 3 kernel, 3 workers on [1,1,10] with kernel 2 / stride 2, each
    in float32 and float64): shards zero-padded by their halos, forward and
    adjoint against the oracle, and the reference's criterion
    <F x, dy> = <x, F* dy> over all workers."""
    nf = len(kernel)
    halo, recv, send = _world_geometry(P, gshape, kernel, stride, [1] * nf)
    gen = torch.Generator().manual_seed(43 + nf)
    order = pm.indices(P)
    padded, dys = {}, {}
    for idx in order:
        local = torch.randn(pm.subshape(P, idx, gshape), generator=gen, dtype=dtype)
        pad = [w for a, b in reversed(halo[idx]) for w in (a, b)]
        padded[idx] = torch.nn.functional.pad(local, pad)
        dys[idx] = torch.randn(padded[idx].shape, generator=gen, dtype=dtype)
    res = _run_halo_world(P, [padded[i] for i in order], [dys[i] for i in order], halo, recv, send)
    want_y = o_halo.forward_all({i: padded[i].numpy() for i in order}, P, recv, send)
    want_dx = o_halo.adjoint_all({i: dys[i].numpy() for i in order}, P, recv, send)
    ipx = ipy = nx = ny = 0.0
    for idx, (y, dx, layer) in zip(order, res):
        assert y.dtype == dtype and dx.dtype == dtype
        assert np.array_equal(y.numpy(), want_y[idx])
        assert np.array_equal(dx.numpy(), want_dx[idx])
        ipx += float((padded[idx].double() * dx.double()).sum())
        ipy += float((y.double() * dys[idx].double()).sum())
        nx += float(padded[idx].double().pow(2).sum())
        ny += float(dys[idx].double().pow(2).sum())
    d = max(np.sqrt(nx) * np.sqrt(ny), 1e-30)
    assert np.isclose(ipx / d, ipy / d)


# ------------------------------------------------------------ fused kernel --

@pytest.fixture(params=["rows", "lines", "default"])
def halo_path(request, ops):
    """The fused kernel has two ways of writing fp32 tensors (row by row, or in
    whole 128-byte lines through LDS); every fused case runs on both and on the
    library's own choice."""
    from distdl_amd import _lib
    return {"rows": _lib.DDL_HALO_ROWS, "lines": _lib.DDL_HALO_LINES, "default": _lib.DDL_HALO_AUTO}[request.param]


_INT_VIEW = {2: torch.int16, 4: torch.int32, 8: torch.int64}
_NP_INT = {2: np.int16, 4: np.int32, 8: np.int64}


def _random_bits(shape, dtype, gen):
    """Random BIT patterns of the dtype: NaN payloads, subnormals, signed zeros."""
    es = torch.empty((), dtype=dtype).element_size()
    raw = torch.randint(0, 256, tuple(shape) + (es,), dtype=torch.uint8, generator=gen)
    return raw.view(dtype).reshape(tuple(shape))


def _np_bits(t):
    """The tensor's elements as NumPy integers of the same width (NaN == NaN under this view)."""
    return t.contiguous().view(_INT_VIEW[t.element_size()]).cpu().numpy()


def _fused_case_bits(ops, x_shape, pad, recv, send, dtype, seed, kernel):
    """The same comparison as ``_fused_case`` on raw bit patterns: shard, ghost
    slabs and results are compared as integers, so NaN payloads, negative
    zeros and subnormals must come through both kernels unchanged (the oracle
    only moves elements, so it runs on the integer view)."""
    gen = torch.Generator().manual_seed(seed)
    x = _random_bits(x_shape, dtype, gen)
    plan = ops.HaloPadPlan(x_shape, pad, recv, send)
    nd = len(x_shape)
    ghosts_np, ghosts, bulks = [], [], []
    for d in range(nd):
        grow_n, grow, brow = [], [], []
        for s in range(2):
            gs, bs = plan.slab_shape(d, s, "ghost"), plan.slab_shape(d, s, "bulk")
            gc = None if gs is None else _random_bits(gs, dtype, gen)
            grow_n.append(None if gc is None else _np_bits(gc))
            grow.append(None if gc is None else gc.cuda())
            brow.append(None if bs is None else torch.full(bs, 7, dtype=dtype, device="cuda"))
        ghosts_np.append(grow_n)
        ghosts.append(grow)
        bulks.append(brow)
    out = plan.run(x.cuda(), ghosts, bulks, kernel=kernel)
    torch.cuda.synchronize()
    want, want_bulks = o_halo.pad_exchange_single(_np_bits(x), pad, recv, send, ghosts_np)
    assert np.array_equal(_np_bits(out), want)
    for d in range(nd):
        for s in range(2):
            if bulks[d][s] is not None:
                assert np.array_equal(_np_bits(bulks[d][s]), want_bulks[d][s]), (d, s)


def _fused_case(ops, x_shape, pad, recv, send, dtype, seed, kernel=0):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(x_shape, generator=gen).to(dtype)
    plan = ops.HaloPadPlan(x_shape, pad, recv, send)
    nd = len(x_shape)
    ghosts_cpu, ghosts, bulks = [], [], []
    for d in range(nd):
        grow_c, grow, brow = [], [], []
        for s in range(2):
            gs, bs = plan.slab_shape(d, s, "ghost"), plan.slab_shape(d, s, "bulk")
            gc = None if gs is None else torch.randn(gs, generator=gen).to(dtype)
            grow_c.append(gc)
            grow.append(None if gc is None else gc.cuda())
            brow.append(None if bs is None else torch.full(bs, 7, dtype=dtype, device="cuda"))
        ghosts_cpu.append(grow_c)
        ghosts.append(grow)
        bulks.append(brow)
    out = plan.run(x.cuda(), ghosts, bulks, kernel=kernel)
    torch.cuda.synchronize()
    np_dtype = {torch.float32: np.float32, torch.float64: np.float64, torch.float16: np.float16}[dtype]
    want, want_bulks = o_halo.pad_exchange_single(
        x.numpy().astype(np_dtype), pad, recv, send,
        [[None if g is None else g.numpy() for g in row] for row in ghosts_cpu])
    assert np.array_equal(out.cpu().numpy(), want)
    for d in range(nd):
        for s in range(2):
            if bulks[d][s] is not None:
                assert np.array_equal(bulks[d][s].cpu().numpy(), want_bulks[d][s]), (d, s)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16])
def test_fused_halo_interior_rank_3d(ops, dtype, halo_path):
    # every side has a ghost and a bulk strip, widths differ per side
    _fused_case(ops, (2, 3, 9, 10, 70), [[0, 0], [0, 0], [1, 2], [2, 1], [1, 3]],
                [[0, 0], [0, 0], [1, 2], [2, 1], [1, 3]], [[0, 0], [0, 0], [2, 1], [1, 2], [3, 1]], dtype, 51, halo_path)


def test_fused_halo_corner_rank_with_explicit_padding(ops, halo_path):
    # rank 0 of a 2x2x2 split, kernel 3 / padding 1: left sides are zero padding, right sides ghosts
    _fused_case(ops, (1, 4, 16, 16, 16), [[0, 0], [0, 0], [1, 1], [1, 1], [1, 1]],
                [[0, 0], [0, 0], [0, 1], [0, 1], [0, 1]], [[0, 0], [0, 0], [0, 1], [0, 1], [0, 1]], torch.float32, 52, halo_path)


def test_fused_halo_long_rows_and_other_ranks(ops, halo_path):
    _fused_case(ops, (3, 5, 300), [[0, 0], [2, 2], [4, 4]], [[0, 0], [2, 2], [4, 0]], [[0, 0], [1, 2], [0, 3]],
                torch.float32, 53, halo_path)
    _fused_case(ops, (40,), [[3, 2]], [[3, 2]], [[2, 3]], torch.float32, 54, halo_path)
    _fused_case(ops, (6, 20), [[0, 0], [0, 0]], [[0, 0], [0, 0]], [[0, 0], [0, 0]], torch.float32, 55, halo_path)   # plain copy
    _fused_case(ops, (4, 6, 20), [[1, 0], [0, 2], [3, 3]], [[0, 0], [0, 0], [0, 0]], [[0, 0], [0, 0], [0, 0]],
                torch.float32, 56, halo_path)                                                                        # F.pad only


def test_fused_halo_wide_rows_geometries(ops, halo_path):
    # rows longer than a 1024-element piece; pieces that begin and end inside a row
    _fused_case(ops, (2, 3, 2500), [[0, 0], [1, 1], [2, 3]], [[0, 0], [1, 1], [2, 3]], [[0, 0], [1, 1], [3, 2]],
                torch.float32, 57, halo_path)
    # padding wider than the ghosts on every side, missing neighbours on some sides
    _fused_case(ops, (2, 7, 9, 100), [[0, 0], [3, 2], [2, 3], [4, 5]], [[0, 0], [1, 0], [0, 2], [2, 0]],
                [[0, 0], [2, 0], [0, 1], [1, 0]], torch.float32, 58, halo_path)
    # four exchanged dimensions, output volume not a multiple of four elements
    _fused_case(ops, (3, 5, 6, 33), [[1, 1], [1, 1], [1, 1], [1, 1]], [[1, 1], [1, 1], [1, 1], [1, 1]],
                [[1, 1], [1, 1], [1, 1], [1, 1]], torch.float32, 59, halo_path)
    # 2-D and 1-D tensors with long rows, int32 payload of the same element size
    _fused_case(ops, (5, 1030), [[2, 2], [1, 1]], [[2, 2], [1, 1]], [[2, 2], [1, 1]], torch.float32, 60, halo_path)
    _fused_case(ops, (4099,), [[3, 2]], [[3, 2]], [[2, 3]], torch.float32, 61, halo_path)
    # ghost strips without bulk strips and the reverse
    _fused_case(ops, (2, 6, 40, 64), [[0, 0], [2, 2], [1, 1], [2, 2]], [[0, 0], [2, 2], [1, 1], [2, 2]],
                [[0, 0], [0, 0], [0, 0], [0, 0]], torch.float32, 62, halo_path)
    _fused_case(ops, (2, 6, 40, 64), [[0, 0], [2, 2], [1, 1], [2, 2]], [[0, 0], [0, 0], [0, 0], [0, 0]],
                [[0, 0], [2, 1], [1, 1], [1, 2]], torch.float32, 63, halo_path)
    # 2-byte elements: odd widths, pieces of 1024 elements that end inside a row, a volume that is not a multiple of 8
    _fused_case(ops, (3, 9, 131), [[0, 0], [1, 1], [1, 1]], [[0, 0], [1, 1], [1, 1]], [[0, 0], [1, 1], [1, 1]],
                torch.float16, 64, halo_path)
    _fused_case(ops, (2, 3, 2500), [[0, 0], [1, 1], [2, 3]], [[0, 0], [1, 1], [2, 3]], [[0, 0], [1, 1], [3, 2]],
                torch.float16, 65, halo_path)


def test_fused_halo_random_geometries(ops, halo_path):
    """Seeded sweep over ranks, widths, missing neighbours and row lengths either
    side of the whole-line kernel's limits; every case bit-exact against the oracle."""
    rng = np.random.default_rng(20240611)
    for case in range(36):
        nd = int(rng.integers(1, 6))
        x_shape, pad, recv, send = [], [], [], []
        for d in range(nd):
            last = d == nd - 1
            n = int(rng.integers(20, 140)) if last else int(rng.integers(1, 7))
            exchanged = last or rng.random() < 0.6
            r = [int(rng.integers(0, 3)) if exchanged else 0 for _ in range(2)]
            p = [r[k] + (int(rng.integers(0, 3)) if exchanged and rng.random() < 0.3 else 0) for k in range(2)]
            s_ = [int(rng.integers(0, min(3, n) + 1)) if exchanged else 0 for _ in range(2)]
            x_shape.append(n)
            pad.append(p)
            recv.append(r)
            send.append(s_)
        dtype = (torch.float32, torch.float16, torch.float64)[case % 3]
        _fused_case(ops, tuple(x_shape), pad, recv, send, dtype, 1000 + case, halo_path)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.float64])
def test_fused_halo_moves_bit_patterns_unchanged(ops, dtype, halo_path):
    """Random bit patterns (NaN payloads, -0, subnormals) through both kernels:
    the 2-byte whole-line path widens elements on the way into LDS and packs them
    on the way out, the 8-byte path moves pairs of words; neither may alter a bit."""
    # interior rank, rows longer than a wavefront's piece and rows that end inside one
    _fused_case_bits(ops, (2, 3, 9, 10, 70), [[0, 0], [0, 0], [1, 2], [2, 1], [1, 3]],
                     [[0, 0], [0, 0], [1, 2], [2, 1], [1, 3]], [[0, 0], [0, 0], [2, 1], [1, 2], [3, 1]], dtype, 71, halo_path)
    _fused_case_bits(ops, (2, 3, 2500), [[0, 0], [1, 1], [2, 3]], [[0, 0], [1, 1], [2, 3]], [[0, 0], [1, 1], [3, 2]],
                     dtype, 72, halo_path)
    # corner rank with explicit zero padding on the left sides, odd row length
    _fused_case_bits(ops, (1, 4, 16, 16, 131), [[0, 0], [0, 0], [1, 1], [1, 1], [1, 1]],
                     [[0, 0], [0, 0], [0, 1], [0, 1], [0, 1]], [[0, 0], [0, 0], [0, 1], [0, 1], [0, 1]], dtype, 73, halo_path)
    # short rows (row kernel under every choice) and a 1-D tensor
    _fused_case_bits(ops, (3, 5, 6, 12), [[1, 1], [1, 1], [1, 1], [1, 1]], [[1, 1], [1, 1], [1, 1], [1, 1]],
                     [[1, 1], [1, 1], [1, 1], [1, 1]], dtype, 74, halo_path)
    _fused_case_bits(ops, (4099,), [[3, 2]], [[3, 2]], [[2, 3]], dtype, 75, halo_path)


def test_fused_halo_config5_interior_rank_full_size(ops):
    """The shard of configuration 5 as an interior rank of a partition at least
    three wide in every spatial dimension: six ghost and six bulk slabs
    ([1,32,1,128,128], [1,32,130,1,128], [1,32,130,130,1] per side), bit-exact
    against the oracle at full size."""
    w = [[0, 0], [0, 0], [1, 1], [1, 1], [1, 1]]
    plan = ops.HaloPadPlan((1, 32, 128, 128, 128), w, w, w)
    assert plan.slab_shape(2, 0, "ghost") == (1, 32, 1, 128, 128) and plan.slab_shape(3, 1, "bulk") == (1, 32, 130, 1, 128)
    assert plan.slab_shape(4, 0, "bulk") == (1, 32, 130, 130, 1)
    _fused_case(ops, (1, 32, 128, 128, 128), w, w, w, torch.float32, 1105)


def test_fused_halo_config5_rank0_bit_exact(ops, halo_path):
    """[1,32,128,128,128] fp32 shard of a 2x2x2 split, kernel 3, padding 1."""
    g = [1, 32, 256, 256, 256]
    P = (1, 1, 2, 2, 2)
    idx = (0, 0, 0, 0, 0)
    gpad = [0, 0, 1, 1, 1]
    lpad = o_halo.local_padding(P, idx, gpad)
    padded_global = [n + 2 * q for n, q in zip(g, gpad)]
    shapes = {i: tuple(n + a + b for n, (a, b) in zip(pm.subshape(P, i, g), o_halo.local_padding(P, i, gpad)))
              for i in pm.indices(P)}
    halo, recv, send, needed = o_halo.exchange_info(padded_global, [3, 3, 3], [1, 1, 1], [0, 0, 0], [1, 1, 1], P, idx,
                                                    shapes=shapes)
    assert halo == [[0, 0], [0, 0], [0, 1], [0, 1], [0, 1]] and send == halo
    total = [[a + c, b + e] for (a, b), (c, e) in zip(lpad, halo)]
    assert total == [[0, 0], [0, 0], [1, 1], [1, 1], [1, 1]]
    _fused_case(ops, (1, 32, 128, 128, 128), total, recv, send, torch.float32, 1005, halo_path)


# ------------------------------------------------------- conv, end to end --

def _run_conv_world(geom, x, weight, bias):
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import DistributedConv1d
    from distdl_amd.nn import DistributedConv2d
    from distdl_amd.nn import DistributedConv3d
    P = geom["P_x_shape"]
    nf = len(geom["kernel_size"])
    Conv = {1: DistributedConv1d, 2: DistributedConv2d, 3: DistributedConv3d}[nf]
    shards = o_rep.scatter(x, P)
    n = int(np.prod(P))

    def body(P_world):
        P_x = P_world.create_partition_inclusive(list(range(n))).create_cartesian_topology_partition(P)
        layer = Conv(P_x, in_channels=x.shape[1], out_channels=weight.shape[0], kernel_size=geom["kernel_size"],
                     stride=geom["stride"], padding=geom["padding"], dilation=geom["dilation"], bias=geom["bias"])
        if P_x.rank == 0:
            with torch.no_grad():
                layer.weight.copy_(weight.cuda())
                if geom["bias"]:
                    layer.bias.copy_(bias.cuda())
        with torch.no_grad():
            y = layer(torch.from_numpy(shards[P_x.rank]).cuda())
        torch.cuda.synchronize()
        return y.cpu().numpy()

    return SimWorld(n).run(body)


def test_feature_conv_matches_sequential_conv(golden):
    rng = np.random.default_rng(61)
    for geom in golden("layer_geometries.json")["conv_feature"]:
        if int(np.prod(geom["P_x_shape"])) > 16:
            continue          # 18-rank case: covered by the oracle test on the CPU
        gshape, k = geom["x_global_shape"], geom["kernel_size"]
        x = rng.standard_normal(gshape).astype(np.float32)
        w = torch.from_numpy(rng.standard_normal([4, gshape[1]] + k).astype(np.float32))
        b = torch.from_numpy(rng.standard_normal(4).astype(np.float32)) if geom["bias"] else None
        conv = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}[len(k)]
        want = conv(torch.from_numpy(x), w, b, stride=geom["stride"], padding=geom["padding"],
                    dilation=geom["dilation"]).numpy()
        outs = _run_conv_world(geom, x, w, b)
        for got, part in zip(outs, o_rep.scatter(want, geom["P_x_shape"])):
            assert got.shape == part.shape, geom["id"]
            # reference tolerance: tests/layers/test_conv_feature.py:392-393 (atol 1e-5 on its sizes);
            # the sums here run over up to 5*5*5*5 terms on two different conv implementations
            assert np.allclose(got, part, atol=1e-4, rtol=1e-4), geom["id"]


@pytest.mark.parametrize("P,gshape,out_channels,padding,y_local", [
    pytest.param([1, 1, 2, 2], [2, 3, 11, 13], 4, 1, None, id="2d-uneven-padded"),
    # tests/layers/test_conv_1d.py:10-19, test_conv_2d.py:10-19, test_conv_3d.py:10-19 (kernel 3, ten output channels)
    pytest.param([1, 1, 3], [1, 5, 10], 10, 0, None, id="reference-1d"),
    pytest.param([1, 1, 2, 2], [1, 5, 10, 10], 10, 0, [1, 10, 4, 4], id="reference-2d"),
    pytest.param([1, 1, 3, 2, 2], [1, 5, 10, 10, 10], 10, 0, None, id="reference-3d"),
    # tests/layers/test_conv_2d.py:233-256: the local output shapes it states
    pytest.param([1, 1, 2, 2], [1, 5, 10, 10], 10, 1, [1, 10, 5, 5], id="reference-2d-padded"),
])
def test_feature_conv_backward_matches_sequential_conv(P, gshape, out_channels, padding, y_local):
    """Input and parameter gradients of the distributed convolution (staging
    crop, halo-exchange adjoint, broadcast adjoint) against torch autograd on
    the whole tensor: the reference's adjoint tests of the input, the weight and
    the bias on its own partitions and sizes, with values instead of the inner
    products, and the local output shapes its shape test states."""
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd import nn as dnn
    nd = len(gshape) - 2
    n = int(np.prod(P))
    Conv = {1: dnn.DistributedConv1d, 2: dnn.DistributedConv2d, 3: dnn.DistributedConv3d}[nd]
    conv = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}[nd]
    rng = np.random.default_rng(62 + nd)
    k = [3] * nd
    x = rng.standard_normal(gshape).astype(np.float32)
    w = torch.from_numpy(rng.standard_normal([out_channels, gshape[1]] + k).astype(np.float32))
    b = torch.from_numpy(rng.standard_normal(out_channels).astype(np.float32))
    xr, wr, br = torch.from_numpy(x).requires_grad_(True), w.clone().requires_grad_(True), b.clone().requires_grad_(True)
    yr = conv(xr, wr, br, padding=padding)
    dy = rng.standard_normal(tuple(yr.shape)).astype(np.float32)
    yr.backward(torch.from_numpy(dy))
    shards, dys = o_rep.scatter(x, P), o_rep.scatter(dy, P)

    def body(P_world):
        P_x = P_world.create_partition_inclusive(list(range(n))).create_cartesian_topology_partition(P)
        layer = Conv(P_x, in_channels=gshape[1], out_channels=out_channels, kernel_size=k, padding=padding, bias=True)
        if P_x.rank == 0:
            with torch.no_grad():
                layer.weight.copy_(w.cuda())
                layer.bias.copy_(b.cuda())
        xin = torch.from_numpy(shards[P_x.rank]).cuda().requires_grad_(True)
        y = layer(xin)
        assert tuple(y.shape) == dys[P_x.rank].shape
        if y_local is not None:
            assert list(y.shape) == y_local
        y.backward(torch.from_numpy(dys[P_x.rank]).cuda())
        torch.cuda.synchronize()
        wg = layer.weight.grad.cpu().numpy() if P_x.rank == 0 else None
        bg = layer.bias.grad.cpu().numpy() if P_x.rank == 0 else None
        return y.detach().cpu().numpy(), xin.grad.cpu().numpy(), wg, bg

    outs = SimWorld(n).run(body)
    for (y, _, _, _), part in zip(outs, o_rep.scatter(yr.detach().numpy(), P)):
        assert np.allclose(y, part, atol=1e-4, rtol=1e-4)
    for (_, dx, _, _), part in zip(outs, o_rep.scatter(xr.grad.numpy(), P)):
        assert np.allclose(dx, part, atol=1e-4, rtol=1e-4)
    assert np.allclose(outs[0][2], wr.grad.numpy(), atol=1e-3, rtol=1e-4)
    assert np.allclose(outs[0][3], br.grad.numpy(), atol=1e-3, rtol=1e-4)


def test_solo_conv_staging_uses_fused_kernel_and_matches_oracle(ops):
    """One live rank (the benchmark configuration, small): staging through the
    layer equals the oracle's pad + exchange with the seeded ghost slabs."""
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import DistributedConv3d
    world = SimWorld(8)
    P_x = world.partition(0).create_partition_inclusive(list(range(8))).create_cartesian_topology_partition(
        [1, 1, 2, 2, 2])
    layer = DistributedConv3d(P_x, in_channels=3, out_channels=2, kernel_size=3, padding=1, bias=False)
    gen = torch.Generator().manual_seed(62)
    x = torch.randn(1, 3, 10, 12, 14, generator=gen)
    xg = x.cuda()
    layer._distdl_forward_pre_hook(layer, (xg,))
    ghost, bulk = layer._fused_slabs(xg)
    ghosts_np = []
    for row in ghost:
        out_row = []
        for gbuf in row:
            if gbuf is None:
                out_row.append(None)
            else:
                vals = torch.randn(gbuf.shape, generator=gen)
                gbuf.copy_(vals)
                out_row.append(vals.numpy())
        ghosts_np.append(out_row)
    staged = layer.stage_input(xg)
    total = (layer.local_padding + layer.halo_shape).tolist()
    want, want_bulks = o_halo.pad_exchange_single(x.numpy(), total, layer.recv_buffer_shape.tolist(),
                                                  layer.send_buffer_shape.tolist(), ghosts_np)
    crop = tuple(slice(int(s.start), int(s.stop)) for s in layer.needed_slices)
    assert np.array_equal(staged.cpu().numpy(), want[crop])
    for d in range(5):
        for s in range(2):
            if bulk[d][s] is not None:
                assert np.array_equal(bulk[d][s].cpu().numpy(), want_bulks[d][s])


# ------------------------------------- layers sharing one buffer manager --

def _adjoint_tight(results):
    """The reference's criterion (tests/adjoint_test.py:11-56) over the per-rank
    tensors (x, dx, y, dy): <F x, dy> and <x, F* dy>, each divided by the larger
    product of norms, agree to np.isclose."""
    sums = np.zeros(6)
    for x, dx, y, dy in results:
        x, dx, y, dy = (t.double() for t in (x, dx, y, dy))
        sums += [float((x * x).sum()), float((dx * dx).sum()), float((y * y).sum()), float((dy * dy).sum()),
                 float((x * dx).sum()), float((y * dy).sum())]
    nx1, nx2, ny1, ny2 = np.sqrt(sums[:4])
    d = max(ny1 * ny2, nx1 * nx2)
    assert d > 0 and np.isclose(sums[4] / d, sums[5] / d), (sums[4] / d, sums[5] / d)


@pytest.mark.parametrize("repartitions_share_the_manager,counts_by_rank", [
    # tests/utilities/test_buffer.py:226-343: only the convolutions use the manager
    (False, {"c1": (4, 4, 4, 4), "c2": (4, 4, 4, 4), "c3": (4, 4, 4, 4), "backward": (4, 4, 4, 4)}),
    # tests/utilities/test_buffer.py:346-466: the two repartitions use it too
    (True, {"tr1": (3, 1, 1, 1), "c1": (4, 4, 4, 4), "c2": (4, 4, 4, 4), "c3": (4, 4, 4, 4), "tr2": (4, 4, 4, 4),
            "backward": (4, 4, 4, 4)}),
])
def test_buffer_manager_shared_by_a_network_of_layers(repartitions_share_the_manager, counts_by_rank):
    """The reference's networks of a scatter, three 3x3 convolutions over a 2x2
    partition and a gather with ONE buffer manager, four workers moving real
    data: the number of pooled float32 buffers after every layer's forward and
    after the backward pass is the reference's, the output equals the three
    stock convolutions on the whole tensor, and the chain passes the tight
    adjoint test."""
    from distdl_amd.backends.stub_hip import BufferManager
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import DistributedConv2d
    from distdl_amd.nn import Repartition
    from distdl_amd.utilities.torch import zero_volume_tensor
    gen = torch.Generator().manual_seed(226)
    x0 = torch.randn(1, 1, 5, 5, generator=gen)
    dy0 = torch.randn(1, 20, 5, 5, generator=gen)
    weights = [torch.randn(o, i, 3, 3, generator=gen) * 0.3 for i, o in ((1, 5), (5, 10), (10, 20))]

    def body(P_world):
        manager = BufferManager()
        P_1 = P_world.create_partition_inclusive([0]).create_cartesian_topology_partition([1, 1, 1, 1])
        P_22 = P_world.create_partition_inclusive([0, 1, 2, 3]).create_cartesian_topology_partition([1, 1, 2, 2])
        shared = {"buffer_manager": manager} if repartitions_share_the_manager else {}
        tr1 = Repartition(P_1, P_22, **shared)
        convs = [DistributedConv2d(P_22, in_channels=i, out_channels=o, kernel_size=[3, 3], padding=[1, 1], bias=False,
                                   buffer_manager=manager) for i, o in ((1, 5), (5, 10), (10, 20))]
        tr2 = Repartition(P_22, P_1, **shared)
        if P_22.rank == 0:
            with torch.no_grad():
                for conv, w in zip(convs, weights):
                    conv.weight.copy_(w.cuda())
        x = zero_volume_tensor(1, device="cuda")
        if P_1.active:
            x = x0.cuda()
        x.requires_grad = True
        counts = {}

        def count():
            return len(manager.buffers_map.get(torch.float32, []))
        h = tr1(x)
        counts["tr1"] = count()
        for name, conv in zip(("c1", "c2", "c3"), convs):
            h = conv(h)
            counts[name] = count()
        y = tr2(h)
        counts["tr2"] = count()
        dy = zero_volume_tensor(1, device="cuda")
        if P_1.active:
            dy = dy0.cuda()
        y.backward(dy)
        counts["backward"] = count()
        torch.cuda.synchronize()
        return counts, x.detach().cpu(), x.grad.cpu(), y.detach().cpu(), dy.cpu()

    res = SimWorld(4).run(body)
    for rank, (counts, *_) in enumerate(res):
        for name, by_rank in counts_by_rank.items():
            assert counts[name] == by_rank[rank], (name, rank, counts)
    want = x0
    for w in weights:
        want = F.conv2d(want, w, padding=1)
    assert torch.allclose(res[0][3], want, atol=1e-4, rtol=1e-4)
    _adjoint_tight([r[1:] for r in res])


K2S2_1D = {"id": "kernel-2-stride-2-1d", "P_x_shape": [1, 1, 4], "x_global_shape": [1, 1, 10], "kernel_size": [2],
           "stride": [2], "padding": [0], "dilation": [1]}


@pytest.mark.parametrize("geom_id", ["kernel-needs-offset", "kernel-2-stride-2-1d"])
def test_feature_conv_with_cropped_staging_forward_and_backward(golden, geom_id):
    """Strided geometries in which the needed range of some worker is smaller
    than its padded shard (reference nn/conv_feature.py:410) -- one of the
    reference's feature-conv test (tests/layers/test_conv_feature.py:9-247) and
    the kernel 2 / stride 2 case of tests/utilities/test_halo_mixin.py:46-87:
    the crop hands the convolution a contiguous window, and the output and the
    input gradient equal those of the stock convolution on the whole tensor."""
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd import nn as dnn
    geom = next(g for g in golden("layer_geometries.json")["conv_feature"] + [K2S2_1D] if g["id"] == geom_id)
    P, gshape, k = geom["P_x_shape"], geom["x_global_shape"], geom["kernel_size"]
    nd, n = len(k), int(np.prod(P))
    Conv = {1: dnn.DistributedConv1d, 2: dnn.DistributedConv2d, 3: dnn.DistributedConv3d}[nd]
    conv = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}[nd]
    rng = np.random.default_rng(410)
    x = rng.standard_normal(gshape).astype(np.float32)
    w = torch.from_numpy(rng.standard_normal([4, gshape[1]] + k).astype(np.float32))
    xr = torch.from_numpy(x).requires_grad_(True)
    yr = conv(xr, w, None, stride=geom["stride"], padding=geom["padding"], dilation=geom["dilation"])
    dy = rng.standard_normal(tuple(yr.shape)).astype(np.float32)
    yr.backward(torch.from_numpy(dy))
    shards, dys = o_rep.scatter(x, P), o_rep.scatter(dy, P)

    def body(P_world):
        P_x = P_world.create_partition_inclusive(list(range(n))).create_cartesian_topology_partition(P)
        layer = Conv(P_x, in_channels=gshape[1], out_channels=4, kernel_size=k, stride=geom["stride"],
                     padding=geom["padding"], dilation=geom["dilation"], bias=False)
        if P_x.rank == 0:
            with torch.no_grad():
                layer.weight.copy_(w.cuda())
        xin = torch.from_numpy(shards[P_x.rank]).cuda().requires_grad_(True)
        layer._distdl_forward_pre_hook(layer, (xin,))
        staged = layer.stage_input(xin)
        padded_shape = [int(v) for v in np.asarray(xin.shape) + (layer.local_padding + layer.halo_shape).sum(axis=1)]
        cropped = list(staged.shape) != padded_shape
        assert staged.is_contiguous()
        y = layer(xin)
        y.backward(torch.from_numpy(dys[P_x.rank]).cuda())
        torch.cuda.synchronize()
        return y.detach().cpu().numpy(), xin.grad.cpu().numpy(), cropped

    outs = SimWorld(n).run(body)
    assert any(cropped for _, _, cropped in outs), "no worker of this geometry crops: the test would prove nothing"
    for (y, _, _), part in zip(outs, o_rep.scatter(yr.detach().numpy(), P)):
        assert np.allclose(y, part, atol=1e-4, rtol=1e-4)
    for (_, dx, _), part in zip(outs, o_rep.scatter(xr.grad.numpy(), P)):
        assert np.allclose(dx, part, atol=1e-4, rtol=1e-4)
