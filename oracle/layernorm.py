"""ORACLE -- test infrastructure, not product code.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import it.

Literal NumPy restatement of the distributed branch of the reference's
DistributedLayerNorm.forward (nn/layernorm.py:295-309) over all workers that
share a row:

  mean  = allreduce(local mean over the normalised dims) / num_reduce    :230-233
  var   = allreduce(local mean of (x - mean)**2)        / num_reduce    :246-247
  y     = (x - mean) / sqrt(var + eps)                                   :302
  y     = weight * y + bias                                              :309

The all-reduce is a sum over the list of shards.  Arithmetic is carried out in
the dtype given (float32 like the reference's default, or float64 to serve as
the exact answer).

Pinned by: torch.nn.functional.layer_norm on the concatenated tensor (the
reference's own test, tests/layers/test_layernorm.py:185-263) for equal shard
widths; the closed form of mean-of-means / mean-of-variances for unequal widths
(reference quirk: not the layer norm of the concatenated row; no reference test
covers it -- parity unpinned by the reference for that corner).
"""

import numpy as np


def forward_shards(shards, gammas, betas, eps, num_norm_dims=1, dtype=np.float32):
    """``shards``: list over the reduction group of arrays whose last
    ``num_norm_dims`` dims are the local part of the normalised dims.
    Returns the list of normalised shards."""
    axes = tuple(range(-num_norm_dims, 0))
    xs = [np.asarray(s, dtype=dtype) for s in shards]
    P = dtype(len(xs))
    mean = sum(x.mean(axis=axes, keepdims=True, dtype=dtype) for x in xs) / P
    var = sum(((x - mean) ** 2).mean(axis=axes, keepdims=True, dtype=dtype) for x in xs) / P
    outs = []
    for x, g, b in zip(xs, gammas, betas):
        y = (x - mean) / np.sqrt(var + dtype(eps))
        if g is not None:
            y = np.asarray(g, dtype=dtype) * y + np.asarray(b, dtype=dtype)
        outs.append(y.astype(dtype))
    return outs


def partial_stats(shard, num_norm_dims=1, dtype=np.float64):
    """Per-row {local mean, local sum of squared deviations from it}."""
    axes = tuple(range(-num_norm_dims, 0))
    x = np.asarray(shard, dtype=dtype)
    m = x.mean(axis=axes, keepdims=True)
    m2 = ((x - m) ** 2).sum(axis=axes, keepdims=True)
    rows = int(np.prod(x.shape[:x.ndim - num_norm_dims]))
    return np.stack([m.reshape(rows), m2.reshape(rows)], axis=1)
