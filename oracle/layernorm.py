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


def forward_rank(x, peer_mean_sum, peer_var_sum, num_reduce, gamma, beta, eps, num_norm_dims=1, dtype=np.float32):
    """One worker's share of ``forward_shards``, in the reference's order of
    operations, with the two all-reduces replaced by what they deliver: the sum
    of the OTHER workers' local means (``peer_mean_sum``) and of their local
    mean squared deviations from the global mean (``peer_var_sum``), both of
    shape ``x.shape[:-num_norm_dims] + (1,) * num_norm_dims``.

        m_loc = x.mean(dims)                 mean = (m_loc + peers) / P     :230-233
        v_loc = ((x - mean)**2).mean(dims)   var  = (v_loc + peers) / P     :246-247
        y = (x - mean) / sqrt(var + eps);  y = weight * y + bias             :302, :309

    Pinned in tests/test_oracle_golden.py against ``forward_shards``."""
    axes = tuple(range(-num_norm_dims, 0))
    x = np.asarray(x, dtype=dtype)
    P = dtype(num_reduce)
    mean = (x.mean(axis=axes, keepdims=True, dtype=dtype) + peer_mean_sum) / P
    var = (((x - mean) ** 2).mean(axis=axes, keepdims=True, dtype=dtype) + peer_var_sum) / P
    y = (x - mean) / np.sqrt(var + dtype(eps))
    if gamma is not None:
        y = np.asarray(gamma, dtype=dtype) * y + np.asarray(beta, dtype=dtype)
    return y.astype(dtype)


def partial_stats(shard, num_norm_dims=1, dtype=np.float64):
    """Per-row {local mean, local sum of squared deviations from it}."""
    axes = tuple(range(-num_norm_dims, 0))
    x = np.asarray(shard, dtype=dtype)
    m = x.mean(axis=axes, keepdims=True)
    m2 = ((x - m) ** 2).sum(axis=axes, keepdims=True)
    rows = int(np.prod(x.shape[:x.ndim - num_norm_dims]))
    return np.stack([m.reshape(rows), m2.reshape(rows)], axis=1)


def backward_shards(shards, gammas, dys, eps, num_norm_dims=1, dtype=np.float64):
    """Gradients of ``forward_shards`` with respect to the shards and the
    affine parameters: returns ``(dxs, dgammas, dbetas)``, lists over the
    reduction group.

    Every element of shard p enters the reference's mean and variance with
    weight a_p = 1 / (P n_p), and the all-reduce is its own adjoint, so with
    g = dy * gamma, xhat = (x - mean) * rstd, S1 = sum of g and S2 = sum of
    g * xhat over the WHOLE row (all shards):

        dx_p     = rstd * (g_p - a_p * (S1 + xhat_p * S2))
        dgamma_p = sum over rows of dy_p * xhat_p        dbeta_p = sum over rows of dy_p

    Pinned in tests/test_oracle_golden.py by torch autograd run through a
    literal torch restatement of nn/layernorm.py:230-309 (equal and unequal
    shard widths), and by torch.nn.functional.layer_norm for equal widths."""
    P = len(shards)
    xs = [np.asarray(s, dtype=dtype) for s in shards]
    ds = [np.asarray(d, dtype=dtype) for d in dys]
    lead = xs[0].shape[:xs[0].ndim - num_norm_dims]
    flat = [x.reshape(int(np.prod(lead)), -1) for x in xs]
    dflat = [d.reshape(int(np.prod(lead)), -1) for d in ds]
    ns = [f.shape[1] for f in flat]
    mean = sum(f.mean(axis=1) for f in flat) / P
    var = sum(((f - mean[:, None]) ** 2).mean(axis=1) for f in flat) / P
    rstd = 1.0 / np.sqrt(var + eps)
    gam = [np.ones(n, dtype=dtype) if g is None else np.asarray(g, dtype=dtype).reshape(-1) for g, n in zip(gammas, ns)]
    xhat = [(f - mean[:, None]) * rstd[:, None] for f in flat]
    g = [d * w[None, :] for d, w in zip(dflat, gam)]
    S1 = sum(v.sum(axis=1) for v in g)
    S2 = sum((v * h).sum(axis=1) for v, h in zip(g, xhat))
    dxs, dgs, dbs = [], [], []
    for p in range(P):
        a = 1.0 / (P * ns[p])
        dx = rstd[:, None] * (g[p] - a * (S1[:, None] + xhat[p] * S2[:, None]))
        dxs.append(dx.reshape(xs[p].shape))
        dgs.append((dflat[p] * xhat[p]).sum(axis=0))
        dbs.append(dflat[p].sum(axis=0))
    return dxs, dgs, dbs
