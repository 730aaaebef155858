"""Tensors of more than 2^31 elements or 4 GiB: byte offsets, row numbers and
token numbers are 64-bit in every kernel, and what a kernel cannot address it
refuses on the host.  Results are compared on the device with torch (sampled
rows for the arithmetic kernels); nothing of this size visits the host."""
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import distdl_amd  # noqa: F401
    from distdl_amd import hip_ops
    return hip_ops


def test_boxes_beyond_four_gib(ops):
    """Offsets are 64-bit throughout: a box of a 5 GiB tensor whose rows start
    past 2^32 bytes, copied, unpacked, packed and accumulated; compared on the
    device (the tensors never visit the host)."""
    rows, cols = 5, 2 ** 30
    gen = torch.Generator(device="cuda").manual_seed(77)
    src = torch.randint(0, 256, (rows, cols), dtype=torch.uint8, device="cuda", generator=gen)
    dst = torch.zeros(rows, cols, dtype=torch.uint8, device="cuda")
    sbox = (slice(1, 5), slice(100, cols - 50))
    dbox = (slice(0, 4), slice(150, cols))
    ops.copy_box(src, sbox, dst, dbox)
    assert torch.equal(dst[dbox], src[sbox])
    assert int(dst[:, :150].max()) == 0 and int(dst[4].max()) == 0
    del dst
    # the last row alone (it starts at 4 GiB) through pack and unpack
    buf = torch.empty(1, 4096, dtype=torch.uint8, device="cuda")
    plan = ops.BoxPlan.from_slices(src, [(slice(4, 5), slice(cols - 4096, cols))])
    plan.pack(src, [buf])
    assert torch.equal(buf, src[4:5, cols - 4096:])
    buf.fill_(7)
    plan.unpack(src, [buf])
    assert int(src[4, cols - 4096:].min()) == 7 and int(src[4, cols - 4096:].max()) == 7
    del src
    # accumulation in float32 across the 4 GiB line: 1.25 Gi elements
    a = torch.ones(5 * 2 ** 28, dtype=torch.float32, device="cuda")
    b = torch.full((5 * 2 ** 28,), 2.0, dtype=torch.float32, device="cuda")
    span = (slice(2 ** 28 - 3, 5 * 2 ** 28 - 1),)
    ops.copy_box(a, span, b, span, accumulate=True)
    assert float(b[:2 ** 28 - 3].max()) == 2.0 and float(b[-1]) == 2.0
    assert float(b[span].min()) == 3.0 and float(b[span].max()) == 3.0



def test_embedding_gather_beyond_2_31_output_elements(ops):
    """2^19 + 24 tokens of 4096 bf16 columns: the output is just over 4 GiB."""
    gen = torch.Generator(device="cuda").manual_seed(3)
    weight = torch.randn(1000, 4096, device="cuda", generator=gen).to(torch.bfloat16)
    n = 2 ** 19 + 24
    ids = torch.randint(0, 1200, (n,), device="cuda", generator=gen)
    out = ops.embedding_gather(weight, ids, 0, 1000)
    assert out.shape == (n, 4096)
    pick = torch.cat([torch.arange(0, 512, device="cuda"), torch.arange(n - 512, n, device="cuda"),
                      torch.randint(0, n, (4096,), device="cuda", generator=gen)])
    hit = ids[pick] < 1000
    want = torch.where(hit[:, None], weight[ids[pick].clamp(max=999)], torch.zeros((), dtype=torch.bfloat16, device="cuda"))
    assert torch.equal(out[pick].view(torch.int16), want.view(torch.int16))


def test_layer_norm_beyond_2_31_elements(ops):
    """2^21 + 3 rows of 1024 fp32 columns (8 GiB): the single launch and the
    two launches of the distributed case, against torch on sampled rows."""
    rows, cols = 2 ** 21 + 3, 1024
    gen = torch.Generator(device="cuda").manual_seed(4)
    x = torch.randn(rows, cols, device="cuda", generator=gen)
    gamma = 1 + 0.1 * torch.randn(cols, device="cuda", generator=gen)
    beta = 0.1 * torch.randn(cols, device="cuda", generator=gen)
    pick = torch.cat([torch.arange(0, 64, device="cuda"), torch.arange(rows - 64, rows, device="cuda"),
                      torch.randint(0, rows, (256,), device="cuda", generator=gen)])
    want = F.layer_norm(x[pick].double(), (cols,), gamma.double(), beta.double(), 1e-5)
    y = ops.layer_norm(x, gamma, beta, 1e-5)
    assert float((y[pick].double() - want).abs().max()) <= 1e-5 * float(want.abs().max())
    del y
    stats = ops.ln_partial_stats(x)
    y2 = ops.ln_normalize_affine(x, stats.unsqueeze(0), [cols], gamma, beta, 1e-5)
    assert float((y2[pick].double() - want).abs().max()) <= 1e-5 * float(want.abs().max())


def test_linear_rows_beyond_2_31_elements(ops):
    """x of 2^18 + 8 rows and K = 8192 in bf16 (4 GiB): sampled rows of the
    product against torch in fp32 (2e-2 relative, the bf16 bar of the shard GEMM)."""
    m, n, k = 2 ** 18 + 8, 256, 8192
    gen = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(m, k, device="cuda", generator=gen).to(torch.bfloat16)
    w = (0.02 * torch.randn(n, k, device="cuda", generator=gen)).to(torch.bfloat16)
    bias = (0.02 * torch.randn(n, device="cuda", generator=gen)).to(torch.bfloat16)
    y = ops.linear(x, w, bias)
    pick = torch.cat([torch.arange(0, 256, device="cuda"), torch.arange(m - 264, m, device="cuda"),
                      torch.randint(0, m, (512,), device="cuda", generator=gen)])
    want = x[pick].float() @ w.float().t() + bias.float()
    err = (y[pick].float() - want).abs().max()
    assert float(err) <= 2e-2 * float(want.abs().max())


def test_halo_staging_beyond_2_31_elements(ops):
    """A shard of 1300^3 fp32 (2.2e9 elements) padded by one on every side of its
    three feature dimensions, the right-hand ghosts received, the right-hand
    bulk packed: against F.pad plus slab assignments, on the device."""
    n = 1300
    gen = torch.Generator(device="cuda").manual_seed(6)
    x = torch.randn(1, 1, n, n, n, device="cuda", generator=gen)
    pad = [[0, 0], [0, 0], [1, 1], [1, 1], [1, 1]]
    recv = [[0, 0], [0, 0], [0, 1], [0, 1], [0, 1]]
    plan = ops.HaloPadPlan(x.shape, pad, recv, recv)
    ghosts = [[None, None] for _ in range(5)]
    bulks = [[None, None] for _ in range(5)]
    for d in (2, 3, 4):
        shape = plan.slab_shape(d, 1, "ghost")
        ghosts[d][1] = torch.randn(shape, device="cuda", generator=gen)
        bulks[d][1] = torch.empty(plan.slab_shape(d, 1, "bulk"), device="cuda")
    out = plan.run(x, ghosts, bulks)
    want = F.pad(x, (1, 1, 1, 1, 1, 1))
    del x
    # the reference's loop: dimension after dimension, pack the bulk slab, then unpack the ghost slab
    for d in (2, 3, 4):
        sl = [slice(None)] * 5
        for j in range(d + 1, 5):
            sl[j] = slice(0, n + 1)                      # bulk range of the later dimensions (right ghost excluded)
        bulk_sl, ghost_sl = list(sl), list(sl)
        bulk_sl[d] = slice(n, n + 1)
        ghost_sl[d] = slice(n + 1, n + 2)
        assert torch.equal(bulks[d][1], want[tuple(bulk_sl)])
        want[tuple(ghost_sl)] = ghosts[d][1]
    assert torch.equal(out, want)


def test_embedding_backward_beyond_2_31_gradient_elements(ops):
    """2^19 + 24 tokens of 4096 bf16 columns (a 4 GiB gradient) into a shard of
    1000 rows: every row's sum against an fp32 index_add (the kernel adds in
    fp32 in token order and rounds once; 1e-2 relative covers the order)."""
    gen = torch.Generator(device="cuda").manual_seed(7)
    n, dim = 2 ** 19 + 24, 4096
    ids = torch.randint(0, 1200, (n,), device="cuda", generator=gen)
    dy = torch.randn(n, dim, device="cuda", generator=gen).to(torch.bfloat16)
    dw = ops.embedding_backward(dy, ids, 0, 1000)
    hit = ids < 1000
    want = torch.zeros(1000, dim, device="cuda")
    want.index_add_(0, ids[hit], dy[hit].float())
    assert float((dw.float() - want).abs().max()) <= 1e-2 * float(want.abs().max())


def test_layer_norm_backward_beyond_2_31_elements(ops):
    """dy and x of 2^21 + 3 rows by 1024 fp32 columns: dx on sampled rows, the
    parameter gradients (sums over two million rows) against float64."""
    rows, cols = 2 ** 21 + 3, 1024
    gen = torch.Generator(device="cuda").manual_seed(8)
    x = torch.randn(rows, cols, device="cuda", generator=gen)
    dy = torch.randn(rows, cols, device="cuda", generator=gen)
    gamma = 1 + 0.1 * torch.randn(cols, device="cuda", generator=gen)
    beta = torch.zeros(cols, device="cuda")
    _, mean, rstd = ops.layer_norm(x, gamma, beta, 1e-5, want_stats=True)
    dx, dg, db = ops.ln_backward_one_pass(dy, x, mean, rstd, gamma, 1.0 / cols)
    pick = torch.cat([torch.arange(0, 64, device="cuda"), torch.arange(rows - 64, rows, device="cuda"),
                      torch.randint(0, rows, (256,), device="cuda", generator=gen)])
    xs = x[pick].double().requires_grad_(True)
    ys = F.layer_norm(xs, (cols,), gamma.double(), beta.double(), 1e-5)
    ys.backward(dy[pick].double())
    assert float((dx[pick].double() - xs.grad).abs().max()) <= 1e-5 * float(xs.grad.abs().max())
    xhat = (x - mean[:, None]) * rstd[:, None]
    want_g = (dy.double() * xhat.double()).sum(0)
    want_b = dy.double().sum(0)
    assert float((dg.double() - want_g).abs().max()) <= 1e-4 * float(want_g.abs().max())
    assert float((db.double() - want_b).abs().max()) <= 1e-4 * float(want_b.abs().max())


def test_linear_backward_rows_beyond_2_31_elements(ops):
    """The adjoint of the shard GEMM with 2^18 + 8 rows, K = 8192 in bf16: dw
    sums over all rows (x is too large to be read in place along its rows, so it
    goes through the transposed copy), dx on sampled rows, db."""
    m, n, k = 2 ** 18 + 8, 256, 8192
    gen = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randn(m, k, device="cuda", generator=gen).to(torch.bfloat16)
    w = (0.02 * torch.randn(n, k, device="cuda", generator=gen)).to(torch.bfloat16)
    dy = (0.05 * torch.randn(m, n, device="cuda", generator=gen)).to(torch.bfloat16)
    dx, dw, db = ops.linear_backward(x, w, dy)
    pick = torch.cat([torch.arange(0, 256, device="cuda"), torch.arange(m - 264, m, device="cuda"),
                      torch.randint(0, m, (512,), device="cuda", generator=gen)])
    want_dx = dy[pick].float() @ w.float()
    assert float((dx[pick].float() - want_dx).abs().max()) <= 2e-2 * float(want_dx.abs().max())
    want_dw = torch.zeros(n, k, device="cuda")
    for lo in range(0, m, 2 ** 15):                    # in slices: the fp32 copies of x stay small
        want_dw += dy[lo:lo + 2 ** 15].float().t() @ x[lo:lo + 2 ** 15].float()
    assert float((dw.float() - want_dw).abs().max()) <= 2e-2 * float(want_dw.abs().max())
    want_db = dy.float().sum(0)
    assert float((db.float() - want_db).abs().max()) <= 2e-2 * float(want_db.abs().max())
