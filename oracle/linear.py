"""ORACLE -- test infrastructure, not product code.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import it.

The local apply of the reference's linear layers (nn/linear.py:103,
nn/linear_ag.py:486: torch.nn.functional.linear(input, weight, bias)) as
y = x . w^T + b in fp32 (or fp64) on operands given as bf16 bit patterns.

The reference's tests check only forward/adjoint consistency of these layers
(tests/layers/test_linear.py:48-305), never forward values -- parity is
unpinned by the reference; here it is pinned by torch.nn.functional.linear on
CPU, by exact small-integer cases and by an fp64 evaluation.
"""

import numpy as np


def bf16_bits_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(x):
    """Round to nearest even, NaN -> 0x7FC0."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return np.where(np.isnan(np.asarray(x, dtype=np.float32)), np.uint16(0x7FC0), rounded)


def linear(x_bits, w_bits, bias_bits=None, dtype=np.float32):
    x = bf16_bits_to_f32(x_bits).astype(dtype)
    w = bf16_bits_to_f32(w_bits).astype(dtype)
    return linear_values(x, w, None if bias_bits is None else bf16_bits_to_f32(bias_bits).astype(dtype))


def linear_values(x, w, bias=None):
    """``linear`` on operands that are already values (any float dtype): the
    product and bias add alone, without the conversion from bit patterns.
    ``linear(xb, wb, bb, dtype)`` equals ``linear_values`` of the converted
    operands by construction; used where only the arithmetic is to be timed."""
    y = x.reshape(-1, x.shape[-1]) @ w.T
    if bias is not None:
        y = y + bias
    return y.reshape(x.shape[:-1] + (w.shape[0],))


def linear_backward(x_bits, w_bits, dy_bits, dtype=np.float64):
    """Adjoint of ``linear`` on bf16 bit patterns: returns ``(dx, dw, db)`` in
    ``dtype`` (exact sums, not rounded to bf16):
        dx = dy @ w        dw = dy.T @ x        db = dy.sum(0)
    which is what autograd derives for torch.nn.functional.linear
    (reference call sites nn/linear.py:103, nn/linear_ag.py:486).  Pinned by
    torch autograd on the same operands in tests/test_oracle_golden.py."""
    x = bf16_bits_to_f32(x_bits).astype(dtype)
    w = bf16_bits_to_f32(w_bits).astype(dtype)
    dy = bf16_bits_to_f32(dy_bits).astype(dtype)
    return dy @ w, dy.T @ x, dy.sum(axis=0)
