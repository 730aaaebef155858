"""ORACLE -- test infrastructure, not product code.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import it.

Row gather of the reference's DistributedEmbedding.forward
(nn/embedding.py:244-246: torch.nn.functional.embedding(input, weight, ...)) on
the local table, plus the shard window used for vocabulary-sharded tables:
out[t] = table[ids[t]-lo] if lo <= ids[t] < hi else 0.  Rows are moved as bit
patterns (bf16 tables are passed as uint16).

Pinned by torch.nn.functional.embedding on CPU (full window) and by a
per-token Python loop (windowed); ``renorm`` by torch.nn.functional.embedding
with ``max_norm`` on CPU.
"""

import numpy as np


def gather(table, ids, lo=0, hi=None):
    if hi is None:
        hi = lo + table.shape[0]
    ids = np.asarray(ids)
    hit = (ids >= lo) & (ids < hi)
    safe = np.where(hit, ids - lo, 0)
    out = table[safe.reshape(-1)].reshape(ids.shape + (table.shape[1],)).copy()
    out[~hit] = 0
    return out


def renorm(table, ids, lo, hi, max_norm, norm_type=2.0):
    """The renormalisation torch.nn.functional.embedding performs before the
    lookup when ``max_norm`` is given (the reference passes it through,
    nn/embedding.py:244-246): every row that is looked up and whose p-norm
    exceeds max_norm is multiplied by max_norm / (norm + 1e-7), once however
    often it is looked up.  Returns the new table (float64)."""
    out = np.asarray(table, dtype=np.float64).copy()
    ids = np.asarray(ids).reshape(-1)
    for row in np.unique(ids[(ids >= lo) & (ids < hi)]) - lo:
        norm = np.linalg.norm(out[row], ord=norm_type)
        if norm > max_norm:
            out[row] *= max_norm / (norm + 1e-7)
    return out


def backward(dy, ids, lo, hi, padding_idx=None, dtype=np.float64, scale_grad_by_freq=False):
    """Adjoint of ``gather`` with respect to the table: row r of the result is
    the sum of dy[t] over the tokens with ids[t] - lo == r (tokens outside the
    window and tokens equal to padding_idx add nothing) -- the dense gradient
    of torch.nn.functional.embedding (reference call site nn/embedding.py:244-246).
    ``dy`` holds values (not bit patterns); sums are exact in ``dtype``.
    With ``scale_grad_by_freq`` a row's sum is divided by the number of tokens
    that contributed to it (the option of that name of the same torch call).
    Pinned by torch autograd on CPU in tests/test_oracle_golden.py."""
    ids = np.asarray(ids).reshape(-1)
    dy = np.asarray(dy, dtype=dtype).reshape(ids.size, -1)
    out = np.zeros((hi - lo, dy.shape[1]), dtype=dtype)
    count = np.zeros(hi - lo, dtype=np.int64)
    for t, i in enumerate(ids):
        if lo <= i < hi and (padding_idx is None or i != padding_idx):
            out[i - lo] += dy[t]
            count[i - lo] += 1
    if scale_grad_by_freq:
        out /= np.maximum(count, 1)[:, None]
    return out
