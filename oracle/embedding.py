"""ORACLE -- test infrastructure, not product code.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import it.

Row gather of the reference's DistributedEmbedding.forward
(nn/embedding.py:244-246: torch.nn.functional.embedding(input, weight, ...)) on
the local table, plus the shard window used for vocabulary-sharded tables:
out[t] = table[ids[t]-lo] if lo <= ids[t] < hi else 0.  Rows are moved as bit
patterns (bf16 tables are passed as uint16).

Pinned by torch.nn.functional.embedding on CPU (full window) and by a
per-token Python loop (windowed).
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
