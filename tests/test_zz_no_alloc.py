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


def _both(lib, dy, ids, lo, hi, padding_idx):
    """(static result, workspace result) of one gradient call; dy [n, dim], ids [n]."""
    n, dim = dy.shape
    rows = hi - lo
    dt = _lib.DDL_DT_BF16 if dy.dtype == torch.bfloat16 else _lib.DDL_DT_F32
    i64 = 1 if ids.dtype == torch.int64 else 0
    # outputs and the reference workspace exist before the allocation-free call
    got = torch.full((rows, dim), 7, dtype=dy.dtype, device="cuda")
    ref = torch.full((rows, dim), 9, dtype=dy.dtype, device="cuda")
    work = torch.full((2 * rows + 1 + n,), -1, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.ddl_embedding_backward_static(dy.data_ptr(), dt, dim, dim, ids.data_ptr(), i64, n, lo, hi, padding_idx, 0,
                                           got.data_ptr(), dim, _stream())
    _lib.check(rc, "ddl_embedding_backward_static")
    assert torch.cuda.memory_allocated() == before
    rc = lib.ddl_embedding_backward(dy.data_ptr(), dt, dim, dim, ids.data_ptr(), i64, n, lo, hi, padding_idx, 0,
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
