"""Pins the oracle (oracle/*.py) before anything is compared with it: the
reference's own known answers (tests/golden), library routines the reference
itself calls (torch CPU), closed forms and brute force."""

import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import embedding as o_emb
from oracle import halo as o_halo
from oracle import layernorm as o_ln
from oracle import linear as o_lin
from oracle import partition_math as pm
from oracle import relayout as o_rl
from oracle import repartition as o_rep


# ---------------------------------------------------------------- partition --

def test_balanced_split_known_answers(golden):
    g = golden("buffer_network.json")
    tn = g["transpose_network"]
    for key, P in (("split_10_over_4", 4), ("split_10_over_3", 3)):
        blocks = tn[key]
        for i, block in enumerate(blocks):
            assert pm.subshape_1d(P, i, 10) == len(block)
            assert pm.start_1d(P, i, 10) == block[0]
    for i, block in enumerate(g["conv2d_network"]["split_5_over_2"]):
        assert pm.subshape_1d(2, i, 5) == len(block)
        assert pm.start_1d(2, i, 5) == block[0]


@pytest.mark.parametrize("P_shape,shape", [([3], [10]), ([2, 2], [7, 5]), ([1, 4, 3], [2, 9, 11]), ([5], [3])])
def test_boxes_tile_the_tensor(P_shape, shape):
    owner = np.full(shape, -1)
    for r, idx in enumerate(pm.indices(P_shape)):
        lo, hi = pm.boxes_balanced(P_shape, shape)[idx]
        region = owner[pm.as_slices(lo, hi)]
        assert (region == -1).all()          # disjoint
        region[...] = r
        assert list(region.shape) == pm.subshape(P_shape, idx, shape)
    assert (owner >= 0).all()                # cover


def test_intersection_brute_force():
    rng = np.random.default_rng(0)
    for _ in range(200):
        lo0, lo1 = rng.integers(0, 6, 2), rng.integers(0, 6, 2)
        hi0, hi1 = lo0 + rng.integers(1, 5, 2), lo1 + rng.integers(1, 5, 2)
        hit = pm.intersect(list(lo0), list(hi0), list(lo1), list(hi1))
        cells0 = set(itertools.product(range(lo0[0], hi0[0]), range(lo0[1], hi0[1])))
        cells1 = set(itertools.product(range(lo1[0], hi1[0]), range(lo1[1], hi1[1])))
        both = cells0 & cells1
        if hit is None:
            assert not both
        else:
            rel = set(itertools.product(range(hit[0][0], hit[1][0]), range(hit[0][1], hit[1][1])))
            assert {(a + lo0[0], b + lo0[1]) for a, b in rel} == both


# -------------------------------------------------------------- repartition --

def test_repartition_example_forward_and_adjoint(golden):
    g = golden("repartition_7x5.json")
    xs = [np.array(a, dtype=np.float16) for a in g["input_by_x_rank"]]
    ys = o_rep.forward_all(xs, g["x_global_shape"], g["P_x_shape"], g["P_y_shape"])
    for got, want in zip(ys, g["forward_by_y_rank"]):
        assert np.array_equal(got, np.array(want, dtype=np.float16))
    dys = [np.array(a, dtype=np.float16) for a in g["adjoint_input_by_y_rank"]]
    dxs = o_rep.adjoint_all(dys, g["x_global_shape"], g["P_x_shape"], g["P_y_shape"])
    for got, want in zip(dxs, g["adjoint_by_x_rank"]):
        assert np.array_equal(got, np.array(want, dtype=np.float16))
    # The same example with disjoint worker teams (8 ranks, no self copies).
    ys2 = o_rep.forward_all(xs, g["x_global_shape"], g["P_x_shape"], g["P_y_shape"], shared_workers=False)
    for got, want in zip(ys2, g["forward_by_y_rank"]):
        assert np.array_equal(got, np.array(want, dtype=np.float16))


def test_identity_repartition_has_only_self_overlaps():
    send, recv, _, _ = o_rep.plan([6, 9], [2, 3], [2, 3])
    for lists in (send, recv):
        for r, lst in enumerate(lists):
            partners = [p for sl, sh, p in lst if sl is not None]
            assert partners == ["self"]


@pytest.mark.parametrize("shape,P_x,P_y", [([7, 5], [4, 1], [2, 2]), ([3, 10, 11], [1, 4, 1], [1, 1, 4]),
                                          ([5, 6, 7], [2, 3, 1], [1, 2, 2]), ([4, 9], [1, 1], [2, 3])])
def test_repartition_is_a_permutation_of_the_global_tensor(shape, P_x, P_y):
    rng = np.random.default_rng(1)
    x = rng.integers(0, 2 ** 16, size=shape).astype(np.uint16)
    shared = int(np.prod(P_x)) == int(np.prod(P_y))
    ys = o_rep.forward_all(o_rep.scatter(x, P_x), shape, P_x, P_y, shared_workers=shared)
    for got, want in zip(ys, o_rep.scatter(x, P_y)):
        assert np.array_equal(got, want)
    back = o_rep.adjoint_all(ys, shape, P_x, P_y, shared_workers=shared)
    for got, want in zip(back, o_rep.scatter(x, P_x)):
        assert np.array_equal(got, want)


def test_repartition_unbalanced_input_shapes():
    # 10 columns held as 3|3|2|2 repartitioned to three workers (4|3|3): the
    # transpose-network diagram of the reference's buffer test.
    x = np.arange(10, dtype=np.int32).reshape(1, 10)
    shards = [x[:, 0:3], x[:, 3:6], x[:, 6:8], x[:, 8:10]]
    shapes = {(0, i): s.shape for i, s in enumerate(shards)}
    ys = o_rep.forward_all(shards, [1, 10], [1, 4], [1, 3], x_shapes=shapes, shared_workers=False)
    assert [y.tolist() for y in ys] == [[[0, 1, 2, 3]], [[4, 5, 6]], [[7, 8, 9]]]


# --------------------------------------------------------------------- halo --

def test_halo_widths_known_answers(golden):
    g = golden("halo_mixin_k2s2.json")
    for entry in g["ranks"]:
        halo, recv, send, needed = o_halo.exchange_info(g["x_global_shape"], g["kernel_size"], g["stride"],
                                                        g["padding"], g["dilation"], g["partition_shape"],
                                                        entry["index"])
        assert halo == entry["halo"] and recv == entry["recv"] and send == entry["send"] and needed == entry["needed"]


@pytest.mark.parametrize("n,P,k,s,p,d", [(10, 4, 2, 2, 0, 1), (20, 3, 5, 1, 0, 1), (17, 4, 3, 2, 0, 2), (12, 2, 7, 2, 0, 1),
                                          (15, 4, 3, 1, 0, 1)])
def test_halo_widths_brute_force(n, P, k, s, p, d):
    ny = o_halo.out_extent(n, k, s, p, d)
    for i in range(P):
        y0, yl = pm.start_1d(P, i, ny), pm.subshape_1d(P, i, ny)
        touched = [s * o + d * t - p for o in range(y0, y0 + yl) for t in range(k)]
        touched = [t for t in touched if 0 <= t < n]
        x0, xl = pm.start_1d(P, i, n), pm.subshape_1d(P, i, n)
        left, right = o_halo.halo_1d(P, i, n, k, s, p, d, nonneg=False)
        if touched:
            assert left == x0 - min(touched)
            assert right == max(touched) - (x0 + xl - 1)


def _example_world(g):
    P = tuple(g["partition_shape"])
    padded, recv, send = {}, {}, {}
    for r, idx in enumerate(pm.indices(P)):
        h, rc, sd, _ = o_halo.exchange_info(g["x_global_shape"], g["kernel_size"], g["stride"], g["padding"],
                                            g["dilation"], P, idx)
        x = np.zeros(pm.subshape(P, idx, g["x_global_shape"]), dtype=np.float32) + (r + 1)
        padded[idx] = np.pad(x, [tuple(a) for a in h])
        recv[idx], send[idx] = rc, sd
    return P, padded, recv, send


def test_halo_exchange_example_forward_and_adjoint(golden):
    g = golden("halo_exchange_2x2.json")
    P, padded, recv, send = _example_world(g)
    for r, idx in enumerate(pm.indices(P)):
        assert np.array_equal(padded[idx][0, 0], np.array(g["padded_input"][r], dtype=np.float32))
    out = o_halo.forward_all(padded, P, recv, send)
    for r, idx in enumerate(pm.indices(P)):
        assert np.array_equal(out[idx][0, 0], np.array(g["forward"][r], dtype=np.float32))
    dy = {idx: np.zeros_like(out[idx]) + g["adjoint_input_constant_per_rank"][r] for r, idx in enumerate(pm.indices(P))}
    dx = o_halo.adjoint_all(dy, P, recv, send)
    for r, idx in enumerate(pm.indices(P)):
        assert np.array_equal(dx[idx][0, 0], np.array(g["adjoint"][r], dtype=np.float32))


def test_halo_adjoint_identity():
    # <F x, y> == <x, F* y> over all workers (the reference's adjoint test, tests/adjoint_test.py:11-56)
    rng = np.random.default_rng(3)
    P, g = (1, 1, 2, 3), [1, 2, 9, 11]
    padded, recv, send = {}, {}, {}
    for idx in pm.indices(P):
        h, rc, sd, _ = o_halo.exchange_info(g, [5, 3], [1, 1], [0, 0], [1, 1], P, idx)
        shape = [a + b[0] + b[1] for a, b in zip(pm.subshape(P, idx, g), h)]
        padded[idx] = rng.standard_normal(shape)
        recv[idx], send[idx] = rc, sd
    y = {idx: rng.standard_normal(a.shape) for idx, a in padded.items()}
    Fx = o_halo.forward_all(padded, P, recv, send)
    Fty = o_halo.adjoint_all(y, P, recv, send)
    lhs = sum(float((Fx[i] * y[i]).sum()) for i in padded)
    rhs = sum(float((padded[i] * Fty[i]).sum()) for i in padded)
    assert np.isclose(lhs, rhs, rtol=1e-12)


def _staged_conv_all_ranks(geom, x, weight, bias):
    """pad -> exchange -> crop -> torch conv on every worker; returns the
    outputs reassembled into the global output."""
    P = tuple(geom["P_x_shape"])
    gshape = geom["x_global_shape"]
    nd = len(gshape)
    k, s, d, pad = geom["kernel_size"], geom["stride"], geom["dilation"], geom["padding"]
    gpad = [0] * (nd - len(pad)) + list(pad)
    padded_global = [n + 2 * q for n, q in zip(gshape, gpad)]
    shards = dict(zip(pm.indices(P), o_rep.scatter(x, P)))
    shapes, lpad = {}, {}
    for idx in shards:
        lpad[idx] = o_halo.local_padding(P, idx, gpad)
        shapes[idx] = tuple(n + a + b for n, (a, b) in zip(shards[idx].shape, lpad[idx]))
    padded, recv, send, needed = {}, {}, {}, {}
    for idx in shards:
        h, rc, sd, nr = o_halo.exchange_info(padded_global, k, s, [0] * len(k), d, P, idx, shapes=shapes)
        total = [(a + c, b + e) for (a, b), (c, e) in zip(lpad[idx], h)]
        padded[idx] = np.pad(shards[idx], total)
        recv[idx], send[idx], needed[idx] = rc, sd, nr
    ex = o_halo.forward_all(padded, P, recv, send)
    conv = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}[len(k)]
    outs = {}
    for idx in ex:
        crop = ex[idx][tuple(slice(a, b) for a, b in needed[idx])]
        outs[idx] = conv(torch.from_numpy(np.ascontiguousarray(crop)), weight, bias, stride=s, dilation=d).numpy()
    return outs


def test_staged_conv_matches_sequential_conv(golden):
    rng = np.random.default_rng(5)
    for geom in golden("layer_geometries.json")["conv_feature"]:
        gshape = geom["x_global_shape"]
        k = geom["kernel_size"]
        x = rng.standard_normal(gshape).astype(np.float32)
        w = torch.from_numpy(rng.standard_normal([4, gshape[1]] + k).astype(np.float32))
        b = torch.from_numpy(rng.standard_normal(4).astype(np.float32)) if geom["bias"] else None
        conv = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}[len(k)]
        want = conv(torch.from_numpy(x), w, b, stride=geom["stride"], padding=geom["padding"],
                    dilation=geom["dilation"]).numpy()
        outs = _staged_conv_all_ranks(geom, x, w, b)
        P = tuple(geom["P_x_shape"])
        for idx, part in zip(pm.indices(P), o_rep.scatter(want, P)):
            assert outs[idx].shape == part.shape, geom["id"]
            assert np.allclose(outs[idx], part, atol=1e-4, rtol=1e-4), geom["id"]


def test_pad_exchange_single_equals_all_rank_exchange():
    # One worker fed with the slabs its neighbours pack must reproduce its
    # tensor in the all-worker exchange -- corners included.
    rng = np.random.default_rng(7)
    P, g = (1, 1, 3, 3), [1, 2, 12, 13]
    shards = dict(zip(pm.indices(P), o_rep.scatter(rng.standard_normal(g).astype(np.float32), P)))
    padded, recv, send, halo = {}, {}, {}, {}
    for idx in shards:
        h, rc, sd, _ = o_halo.exchange_info(g, [3, 5], [1, 1], [0, 0], [1, 1], P, idx)
        padded[idx] = np.pad(shards[idx], [tuple(a) for a in h])
        halo[idx], recv[idx], send[idx] = h, rc, sd
    ex = o_halo.forward_all(padded, P, recv, send)
    me = (0, 0, 1, 1)
    sl = o_halo.slab_slices(ex[me].shape, recv[me], send[me])
    ghosts = [[np.ascontiguousarray(ex[me][sl[i][1]]) if recv[me][i][0] else None,
               np.ascontiguousarray(ex[me][sl[i][3]]) if recv[me][i][1] else None] for i in range(4)]
    got, bulks = o_halo.pad_exchange_single(shards[me], halo[me], recv[me], send[me], ghosts)
    assert np.array_equal(got, ex[me])
    for i in range(4):
        for side, q in ((0, 0), (1, 2)):
            if send[me][i][side]:
                assert np.array_equal(bulks[i][side], ex[me][sl[i][q]])


# ---------------------------------------------------------------- layernorm --

def test_layernorm_oracle_matches_torch_layer_norm(golden):
    torch.manual_seed(0)
    for geom in golden("layer_geometries.json")["layernorm"] + [
            {"P_x_shape": [1, 1, 4], "input_shape": [4, 8, 64], "normalized_shape": [64]}]:
        P, shape, norm = geom["P_x_shape"], geom["input_shape"], geom["normalized_shape"]
        nn_ = len(norm)
        if any(n % p for n, p in zip(shape[-nn_:], P[-nn_:])):
            continue  # unequal widths: the reference is not a layer norm there
        x = torch.rand(shape, dtype=torch.float32)
        gamma = 1 + 0.1 * torch.randn(norm)
        beta = 0.1 * torch.randn(norm)
        want = F.layer_norm(x, tuple(norm), gamma, beta, 1e-5).numpy()
        Pn = [1] * (len(shape) - nn_) + list(P[-nn_:])
        full = [1] * (len(shape) - nn_) + list(norm)
        xs = o_rep.scatter(x.numpy(), Pn)
        gs = o_rep.scatter(gamma.numpy().reshape(full), Pn)
        bs = o_rep.scatter(beta.numpy().reshape(full), Pn)
        ys = o_ln.forward_shards(xs, gs, bs, 1e-5, num_norm_dims=nn_)
        for got, part in zip(ys, o_rep.scatter(want, Pn)):
            assert np.allclose(got, part, rtol=1e-4, atol=1e-5)
        ys64 = o_ln.forward_shards(xs, gs, bs, 1e-5, num_norm_dims=nn_, dtype=np.float64)
        want64 = F.layer_norm(x.double(), tuple(norm), gamma.double(), beta.double(), 1e-5).numpy()
        for got, part in zip(ys64, o_rep.scatter(want64, Pn)):
            assert np.allclose(got, part, rtol=1e-9, atol=1e-9)


def test_layernorm_oracle_unequal_widths_closed_form():
    # mean of local means and mean of local variances, by hand on one row
    a, b = np.array([[1.0, 2.0, 3.0]]), np.array([[10.0]])
    mean = (2.0 + 10.0) / 2
    var = (((a - mean) ** 2).mean() + ((b - mean) ** 2).mean()) / 2
    ya, yb = o_ln.forward_shards([a, b], [None, None], [None, None], 0.0, dtype=np.float64)
    assert np.allclose(ya, (a - mean) / np.sqrt(var)) and np.allclose(yb, (b - mean) / np.sqrt(var))


def test_partial_stats_closed_form():
    x = np.array([[1.0, 2.0, 3.0, 6.0], [0.0, 0.0, 0.0, 0.0]])
    st = o_ln.partial_stats(x)
    assert np.allclose(st, [[3.0, 14.0], [0.0, 0.0]])


# ---------------------------------------------------------------- embedding --

def test_embedding_oracle_matches_torch_and_loop():
    torch.manual_seed(1)
    table = torch.randn(50, 12).to(torch.bfloat16)
    ids = torch.randint(0, 50, (3, 7))
    bits = table.view(torch.int16).numpy().view(np.uint16)
    want = F.embedding(ids, table).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(o_emb.gather(bits, ids.numpy()), want)
    lo, hi = 10, 25
    got = o_emb.gather(bits[lo:hi], ids.numpy(), lo, hi)
    for i in range(3):
        for j in range(7):
            t = int(ids[i, j])
            row = bits[t] if lo <= t < hi else np.zeros(12, dtype=np.uint16)
            assert np.array_equal(got[i, j], row)


# ------------------------------------------------------------------- linear --

def test_bf16_conversions_match_torch():
    torch.manual_seed(2)
    x = torch.randn(1000) * 100
    x[::50] = float("nan")
    x[1::50] = float("inf")
    want = x.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = o_lin.f32_to_bf16_bits(x.numpy())
    nan = np.isnan(x.numpy())
    assert np.array_equal(got[~nan], want[~nan])        # NaN payloads are not pinned
    assert np.isnan(o_lin.bf16_bits_to_f32(got[nan])).all()
    back = o_lin.bf16_bits_to_f32(got)
    ref = x.to(torch.bfloat16).float().numpy()
    assert np.array_equal(np.nan_to_num(back, nan=7.0), np.nan_to_num(ref, nan=7.0))


def test_linear_oracle_matches_torch_and_exact_cases():
    torch.manual_seed(3)
    x = torch.randn(5, 6, 32).to(torch.bfloat16)
    w = (0.02 * torch.randn(24, 32)).to(torch.bfloat16)
    b = (0.02 * torch.randn(24)).to(torch.bfloat16)

    def bits(t):
        return t.contiguous().view(torch.int16).numpy().view(np.uint16)
    want = F.linear(x.float(), w.float(), b.float()).numpy()
    got = o_lin.linear(bits(x), bits(w), bits(b))
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    # exact: small integers are representable in bf16 and their products sum exactly in fp32
    xi = torch.randint(-4, 5, (7, 16)).float()
    wi = torch.randint(-4, 5, (9, 16)).float()
    exact = (xi.double() @ wi.double().T).numpy()
    assert np.array_equal(o_lin.linear(bits(xi.to(torch.bfloat16)), bits(wi.to(torch.bfloat16))), exact)


def test_linear_backward_oracle_matches_torch_autograd():
    """The adjoint restatement against what autograd derives for F.linear, on
    float64 copies of the same bf16 values (sums exact enough to compare at 1e-12)."""
    torch.manual_seed(4)
    x = torch.randn(11, 24).to(torch.bfloat16)
    w = (0.1 * torch.randn(7, 24)).to(torch.bfloat16)
    b = torch.randn(7).to(torch.bfloat16)
    dy = torch.randn(11, 7).to(torch.bfloat16)

    def bits(t):
        return t.contiguous().view(torch.int16).numpy().view(np.uint16)
    xd, wd, bd = (t.double().requires_grad_(True) for t in (x, w, b))
    F.linear(xd, wd, bd).backward(dy.double())
    dx, dw, db = o_lin.linear_backward(bits(x), bits(w), bits(dy))
    assert np.allclose(dx, xd.grad.numpy(), rtol=1e-12, atol=1e-12)
    assert np.allclose(dw, wd.grad.numpy(), rtol=1e-12, atol=1e-12)
    assert np.allclose(db, bd.grad.numpy(), rtol=1e-12, atol=1e-12)
    # a transposed operand or a swapped product would break these shapes / values
    assert dx.shape == (11, 24) and dw.shape == (7, 24) and db.shape == (7,)


@pytest.mark.parametrize("widths", [[8, 8], [5, 11, 3], [16]])
def test_layernorm_backward_oracle_matches_autograd_of_the_reference_sequence(widths):
    """The reference's forward, restated op by op in torch (nn/layernorm.py:230-247,
    295-309; an all-reduce is a sum over the shards), differentiated by autograd,
    against the closed form of oracle.backward_shards -- for unequal widths too,
    where the result is NOT the gradient of a plain layer norm."""
    torch.manual_seed(sum(widths))
    rows, P, eps = 6, len(widths), 1e-5
    xs = [torch.randn(rows, w, dtype=torch.float64, requires_grad=True) for w in widths]
    gs = [(1 + 0.1 * torch.randn(w, dtype=torch.float64)).requires_grad_(True) for w in widths]
    bs = [(0.1 * torch.randn(w, dtype=torch.float64)).requires_grad_(True) for w in widths]
    dys = [torch.randn(rows, w, dtype=torch.float64) for w in widths]
    mean = sum(x.mean(dim=-1, keepdim=True) for x in xs) / P                      # :230-233
    var = sum(((x - mean) ** 2).mean(dim=-1, keepdim=True) for x in xs) / P       # :246-247
    ys = [g * ((x - mean) / torch.sqrt(var + eps)) + b for x, g, b in zip(xs, gs, bs)]   # :302, :309
    sum((y * d).sum() for y, d in zip(ys, dys)).backward()
    dxs, dgs, dbs = o_ln.backward_shards([x.detach().numpy() for x in xs], [g.detach().numpy() for g in gs],
                                         [d.numpy() for d in dys], eps)
    for p in range(P):
        assert np.allclose(dxs[p], xs[p].grad.numpy(), rtol=1e-10, atol=1e-12)
        assert np.allclose(dgs[p], gs[p].grad.numpy(), rtol=1e-10, atol=1e-12)
        assert np.allclose(dbs[p], bs[p].grad.numpy(), rtol=1e-10, atol=1e-12)
    if len(set(widths)) == 1:
        # equal widths: the gradient of torch's layer norm on the concatenated row
        x = torch.cat([t.detach() for t in xs], dim=1).requires_grad_(True)
        g = torch.cat([t.detach() for t in gs]).requires_grad_(True)
        b = torch.cat([t.detach() for t in bs]).requires_grad_(True)
        (F.layer_norm(x, (sum(widths),), g, b, eps) * torch.cat(dys, dim=1)).sum().backward()
        assert np.allclose(np.concatenate(dxs, axis=1), x.grad.numpy(), rtol=1e-9, atol=1e-11)
        assert np.allclose(np.concatenate(dgs), g.grad.numpy(), rtol=1e-9, atol=1e-11)


def test_layernorm_forward_rank_equals_forward_shards():
    """The one-worker form used for the CPU baseline is the all-worker form seen from worker 0."""
    rng = np.random.default_rng(8)
    widths = [5, 7, 4]
    shards = [rng.standard_normal((3, 6, w)) for w in widths]
    gammas = [rng.standard_normal(w) for w in widths]
    betas = [rng.standard_normal(w) for w in widths]
    want = o_ln.forward_shards(shards, gammas, betas, 1e-5, dtype=np.float64)
    P = len(widths)
    mean = sum(s.mean(axis=-1, keepdims=True) for s in shards) / P
    for live in range(P):
        peer_mean = sum(s.mean(axis=-1, keepdims=True) for p, s in enumerate(shards) if p != live)
        peer_var = sum(((s - mean) ** 2).mean(axis=-1, keepdims=True) for p, s in enumerate(shards) if p != live)
        got = o_ln.forward_rank(shards[live], peer_mean, peer_var, P, gammas[live], betas[live], 1e-5, dtype=np.float64)
        assert np.allclose(got, want[live], rtol=1e-12, atol=1e-12)


def test_embedding_backward_oracle_matches_torch_autograd():
    torch.manual_seed(6)
    table = torch.randn(20, 5, dtype=torch.float64, requires_grad=True)
    ids = torch.randint(0, 20, (4, 9))
    dy = torch.randn(4, 9, 5, dtype=torch.float64)
    F.embedding(ids, table, padding_idx=3).backward(dy)
    got = o_emb.backward(dy.numpy(), ids.numpy(), 0, 20, padding_idx=3)
    assert np.allclose(got, table.grad.numpy(), rtol=1e-13, atol=1e-13)
    # a window: exactly the rows [lo, hi) of the full gradient (padding row excluded as above)
    full = o_emb.backward(dy.numpy(), ids.numpy(), 0, 20)
    assert np.array_equal(o_emb.backward(dy.numpy(), ids.numpy(), 5, 12), full[5:12])
    # scale_grad_by_freq: torch divides each row's gradient by the row's number of occurrences in the batch
    table2 = table.detach().clone().requires_grad_(True)
    F.embedding(ids, table2, padding_idx=3, scale_grad_by_freq=True).backward(dy)
    got = o_emb.backward(dy.numpy(), ids.numpy(), 0, 20, padding_idx=3, scale_grad_by_freq=True)
    assert np.allclose(got, table2.grad.numpy(), rtol=1e-13, atol=1e-13)
    assert not np.allclose(got, table.grad.numpy())      # the option changes the answer on this input


@pytest.mark.parametrize("norm_type", [1.0, 2.0, 3.5, float("inf")])
def test_embedding_renorm_oracle_matches_torch(norm_type):
    """max_norm: torch.nn.functional.embedding renormalises the looked-up rows
    in place (repeated ids once), leaves the others alone, and the lookup then
    returns the renormalised rows; a window renormalises its own rows only."""
    torch.manual_seed(8)
    table = 2 * torch.randn(30, 7, dtype=torch.float64)
    ids = torch.tensor([[3, 3, 9, 27], [0, 9, 9, 15]])
    want_table = table.clone()
    want_out = F.embedding(ids, want_table, max_norm=1.5, norm_type=norm_type)
    got = o_emb.renorm(table.numpy(), ids.numpy(), 0, 30, 1.5, norm_type)
    assert np.allclose(got, want_table.numpy(), rtol=1e-12, atol=1e-12)
    untouched = [r for r in range(30) if r not in (0, 3, 9, 15, 27)]
    assert np.array_equal(got[untouched], table.numpy()[untouched])
    assert not np.allclose(got[[3, 9]], table.numpy()[[3, 9]])            # something was scaled on this input
    assert np.allclose(o_emb.gather(got, ids.numpy(), 0, 30), want_out.numpy(), rtol=1e-12, atol=1e-12)
    part = o_emb.renorm(table.numpy()[5:20], ids.numpy(), 5, 20, 1.5, norm_type)
    assert np.allclose(part[[4, 10]], want_table.numpy()[[9, 15]], rtol=1e-12, atol=1e-12)
    rest = [r for r in range(15) if r not in (4, 10)]
    assert np.array_equal(part[rest], table.numpy()[5:20][rest])


# ------------------------------------------- all-gather / reduce-scatter re-layouts --

RELAYOUT_CASES = [((3, 10), 1, 4), ((7, 2, 5), 0, 3), ((2, 9, 4), 1, 2), ((2, 3, 8), 2, 4), ((5,), 0, 5), ((4, 6), 0, 6)]


def test_relayout_shard_extents_known_answers(golden):
    """The split the re-layouts assume is the balanced split of the reference's
    own known answers (10 over 4 -> 3,3,2,2; 10 over 3 -> 4,3,3)."""
    assert o_rl.shard_extents(10, 4) == [3, 3, 2, 2]
    assert o_rl.shard_extents(10, 3) == [4, 3, 3]
    for n, P in ((10, 4), (7, 3), (8, 8), (5, 6)):
        assert o_rl.shard_extents(n, P) == [pm.subshape_1d(P, i, n) for i in range(P)]


@pytest.mark.parametrize("shape,axis,P", RELAYOUT_CASES)
def test_all_gather_oracle_closed_form_and_brute_force(shape, axis, P):
    """A gather of the balanced split of x is x; and element by element: the
    element j of the gathered axis comes from the worker whose range holds j."""
    rng = np.random.default_rng(sum(shape) * 7 + axis + P)
    x = rng.standard_normal(shape).astype(np.float32)
    extents = o_rl.shard_extents(shape[axis], P)
    starts = np.concatenate([[0], np.cumsum(extents)])
    parts = [np.take(x, range(starts[r], starts[r + 1]), axis=axis) for r in range(P)]
    got = o_rl.all_gather(parts, axis)
    assert np.array_equal(got, x)
    marked = [np.full(p.shape, 10 * r, dtype=np.int64) + np.arange(p.shape[axis]).reshape(
        [-1 if d == axis else 1 for d in range(p.ndim)]) for r, p in enumerate(parts)]
    tagged = o_rl.all_gather(marked, axis)
    for j in range(shape[axis]):
        r = int(np.searchsorted(starts, j, side="right") - 1)
        assert np.all(np.take(tagged, j, axis=axis) == 10 * r + (j - starts[r]))
    with pytest.raises(ValueError):
        o_rl.all_gather(parts[::-1] if extents != extents[::-1] else [parts[0][..., :0]] + parts[1:], axis)


@pytest.mark.parametrize("shape,axis,P", RELAYOUT_CASES)
def test_reduce_scatter_oracle_closed_form_and_brute_force(shape, axis, P):
    """Worker r ends with slab r of the element-wise sum; P copies of x give P
    times the split of x; written out element by element on integers."""
    rng = np.random.default_rng(sum(shape) * 11 + axis + P)
    fulls = [rng.integers(-5, 6, size=shape).astype(np.int64) for _ in range(P)]
    extents = o_rl.shard_extents(shape[axis], P)
    starts = np.concatenate([[0], np.cumsum(extents)])
    got = o_rl.reduce_scatter(fulls, axis)
    total = np.zeros(shape, dtype=np.int64)
    for idx in np.ndindex(*shape):
        total[idx] = sum(int(f[idx]) for f in fulls)
    for r in range(P):
        want = np.take(total, range(starts[r], starts[r + 1]), axis=axis)
        assert got[r].shape == want.shape and np.array_equal(got[r], want)
    x = rng.standard_normal(shape).astype(np.float32)
    same = o_rl.reduce_scatter([x] * P, axis)
    if P & (P - 1) == 0:                                   # a power of two: the repeated additions are exact
        for r in range(P):
            assert np.array_equal(same[r], P * np.take(x, range(starts[r], starts[r + 1]), axis=axis))


@pytest.mark.parametrize("shape,axis,P", RELAYOUT_CASES)
def test_relayout_oracle_adjoint_identity(shape, axis, P):
    """<A x, y> = <x, A* y> over all workers, exactly (integers), for the
    gather with its reduce-scatter adjoint and the other way round; with
    scale_backward the adjoint is divided by it."""
    rng = np.random.default_rng(sum(shape) * 13 + axis + P)
    extents = o_rl.shard_extents(shape[axis], P)

    def shard_like(r):
        s = list(shape)
        s[axis] = extents[r]
        return rng.integers(-4, 5, size=s).astype(np.int64)

    xs = [shard_like(r) for r in range(P)]
    ys = [rng.integers(-4, 5, size=shape).astype(np.int64) for _ in range(P)]
    Ax = o_rl.all_gather(xs, axis)                         # every worker holds Ax
    lhs = sum(int(np.sum(Ax * y)) for y in ys)
    Aty = o_rl.all_gather_adjoint(ys, axis)
    assert lhs == sum(int(np.sum(x * g)) for x, g in zip(xs, Aty))
    Bf = o_rl.reduce_scatter(ys, axis)
    gs = [shard_like(r) for r in range(P)]
    lhs = sum(int(np.sum(b * g)) for b, g in zip(Bf, gs))
    Btg = o_rl.reduce_scatter_adjoint(gs, axis)
    assert lhs == sum(int(np.sum(y * t)) for y, t in zip(ys, Btg))
    halves = o_rl.all_gather_adjoint([y.astype(np.float64) for y in ys], axis, scale_backward=2)
    for h, g in zip(halves, Aty):
        assert np.array_equal(h, g / 2)
