"""ddl_embedding_backward_static: the embedding-gradient entry point that
allocates nothing.  Its counters and buckets live in a device array built into
the library, so all calls on a GPU share them; the test calls it twice in a
row through the C ABI, the second time with a smaller input (stale contents of
the first call must not leak), and compares each result bit for bit with
ddl_embedding_backward run on a caller-provided workspace.
"""

import ctypes

import numpy as np
import pytest
import torch

from distdl_amd import _lib
from oracle import embedding as o_emb

pytestmark = pytest.mark.gpu


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _both(lib, dy, ids, lo, hi, padding_idx, by_freq=0):
    """(static result, workspace result) of one gradient call; dy [n, dim], ids [n]."""
    n, dim = dy.shape
    rows = hi - lo
    dt = _lib.DDL_DT_BF16 if dy.dtype == torch.bfloat16 else _lib.DDL_DT_F32
    i64 = 1 if ids.dtype == torch.int64 else 0
    # outputs and the reference workspace exist before the allocation-free call
    got = torch.full((rows, dim), 7, dtype=dy.dtype, device="cuda")
    ref = torch.full((rows, dim), 9, dtype=dy.dtype, device="cuda")
    work = torch.full((3 * rows + 1 + n,), -1, dtype=torch.int32, device="cuda")
    # The call is made twice and the second one is watched: the first call on a device looks up the built-in array's
    # address, and the first launch of a kernel may make the runtime grow its own pools -- neither is the entry point's doing.
    rc = lib.ddl_embedding_backward_static(dy.data_ptr(), dt, dim, dim, ids.data_ptr(), i64, n, lo, hi, padding_idx,
                                           by_freq, got.data_ptr(), dim, _stream())
    _lib.check(rc, "ddl_embedding_backward_static")
    got.fill_(7)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before, _ = torch.cuda.mem_get_info()          # the driver's own count: sees allocations torch's allocator does not
    rc = lib.ddl_embedding_backward_static(dy.data_ptr(), dt, dim, dim, ids.data_ptr(), i64, n, lo, hi, padding_idx, by_freq,
                                           got.data_ptr(), dim, _stream())
    _lib.check(rc, "ddl_embedding_backward_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    rc = lib.ddl_embedding_backward(dy.data_ptr(), dt, dim, dim, ids.data_ptr(), i64, n, lo, hi, padding_idx, by_freq,
                                    ref.data_ptr(), dim, work.data_ptr(), work.numel(), _stream())
    _lib.check(rc, "ddl_embedding_backward")
    torch.cuda.synchronize()
    return got, ref


def _bits(t):
    return t.contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32).cpu().numpy()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_entry_matches_workspace_entry_on_two_calls_in_a_row(dtype):
    lib = _lib.load()
    gen = torch.Generator().manual_seed(77)
    # first call: 3000-row window of a 24000-row vocabulary, 20000 tokens (below 64 per row, so sums have one order)
    # second call: smaller in rows and tokens; it finds the first call's counters and buckets in the array
    for rows, tokens, dim, vocab, idt in ((3000, 20000, 256, 24000, torch.int64), (700, 1500, 136, 2100, torch.int32)):
        lo = 11
        ids = torch.randint(0, vocab, (tokens,), generator=gen).to(idt)
        dy = torch.randn(tokens, dim, generator=gen).to(dtype)
        pad = lo + 5
        got, ref = _both(lib, dy.cuda(), ids.cuda(), lo, lo + rows, pad)
        assert np.array_equal(_bits(got), _bits(ref))
        # and against the oracle: fp32 accumulation, one rounding to the output type
        exact = o_emb.backward(dy.double().numpy(), ids.numpy(), lo, lo + rows, padding_idx=pad)
        err = np.abs(got.cpu().double().numpy() - exact)
        assert (err <= 2.0 ** -7 * np.abs(exact) + 1e-5).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_entry_long_buckets_and_frequency_scaling_on_the_shared_array(dtype):
    """Two calls in a row on the built-in array whose buckets take the sorted
    paths -- a row with a few hundred tokens (sorted in LDS) and one with more
    than 8192 (sorted in place) -- the first with scale_grad_by_freq, the second
    smaller and without: bit for bit the workspace entry point's results."""
    lib = _lib.load()
    gen = torch.Generator().manual_seed(78)
    for rows, tokens, dim, hot, by_freq in ((500, 30000, 64, (9000, 300), 1), (120, 12000, 40, (8300, 70), 0)):
        lo = 3
        ids = torch.randint(0, rows + 40, (tokens,), generator=gen)
        order = torch.randperm(tokens, generator=gen)
        ids[order[:hot[0]]] = lo + 7                     # more than 8192 tokens on one row
        ids[order[hot[0]:hot[0] + hot[1]]] = lo + 8      # more than 64 on another
        dy = torch.randn(tokens, dim, generator=gen).to(dtype)
        got, ref = _both(lib, dy.cuda(), ids.cuda(), lo, lo + rows, -1, by_freq)
        assert np.array_equal(_bits(got), _bits(ref))
        exact = o_emb.backward(dy.double().numpy(), ids.numpy(), lo, lo + rows, scale_grad_by_freq=bool(by_freq))
        err = np.abs(got.cpu().double().numpy() - exact)
        tol = 2.0 ** -7 if dtype == torch.bfloat16 else 1e-5
        assert (err <= tol * (np.abs(exact) + np.abs(exact).max())).all()


def test_static_entry_exact_small_integers():
    """Sums of small integers are exact in any order: equal to the oracle bit for bit."""
    lib = _lib.load()
    gen = torch.Generator().manual_seed(5)
    for rows, tokens, dim in ((40, 6000, 520), (3, 100, 8)):
        ids = torch.randint(0, rows + 9, (tokens,), generator=gen)
        dy = torch.randint(-2, 3, (tokens, dim), generator=gen).to(torch.float32)
        got, ref = _both(lib, dy.cuda(), ids.cuda(), 2, 2 + rows, -1)
        want = o_emb.backward(dy.double().numpy(), ids.numpy(), 2, 2 + rows)
        assert np.array_equal(got.cpu().double().numpy(), want)
        assert np.array_equal(ref.cpu().double().numpy(), want)


def test_static_entry_rejects_sizes_beyond_the_built_in_workspace():
    lib = _lib.load()
    cap = _lib.DDL_EMBEDDING_BACKWARD_STATIC_MAX_ELEMS
    dy = torch.zeros(8, 8, device="cuda")
    ids = torch.zeros(8, dtype=torch.int64, device="cuda")
    dw = torch.zeros(8, 8, device="cuda")
    # the size test comes before any pointer is used: n_ids alone exceeds the capacity
    rc = lib.ddl_embedding_backward_static(dy.data_ptr(), _lib.DDL_DT_F32, 8, 8, ids.data_ptr(), 1, cap, 0, 8, -1, 0,
                                           dw.data_ptr(), 8, _stream())
    assert rc == -5
    assert b"exceeds the built-in workspace" in lib.ddl_last_error()
    rc = lib.ddl_embedding_backward_static(dy.data_ptr(), _lib.DDL_DT_F32, 8, 8, ids.data_ptr(), 1, 8, 0, cap // 2, -1, 0,
                                           dw.data_ptr(), 8, _stream())
    assert rc == -5
    torch.cuda.synchronize()
