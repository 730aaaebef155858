"""DistributedEmbedding (reference: nn/embedding.py:12-246).

The table is partitioned along the embedding dimension as in the reference
(every id hits, :113-115); the lookup ``torch.nn.functional.embedding``
(:244-246) is replaced by the HIP gather kernel.  ``vocab_shard=(lo, hi)`` is an
extension for vocabulary-sharded tables: the local table then holds rows
``lo..hi-1`` and ids outside that window produce zero rows.
"""

import torch

from .. import config
from .. import hip_ops
from ..utilities.slicing import compute_subshape
from ..utilities.slicing import worker_layout
from ..utilities.torch import zero_volume_tensor
from .broadcast import Broadcast
from .module import Module


class _EmbeddingShard(torch.autograd.Function):
    """Row gather from the local table and its adjoint (the dense gradient
    autograd derives for ``F.embedding``: rows of ``grad_output`` summed per
    looked-up table row, the ``padding_idx`` row left at zero)."""

    @staticmethod
    def forward(ctx, weight, ids, lo, hi, padding_idx=None, scale_grad_by_freq=False):
        ctx.save_for_backward(ids)
        ctx.window = (lo, hi, padding_idx, scale_grad_by_freq)
        return hip_ops.embedding_gather(weight.detach(), ids, lo, hi)

    @staticmethod
    def backward(ctx, grad_output):
        (ids,) = ctx.saved_tensors
        lo, hi, padding_idx, scale_grad_by_freq = ctx.window
        dw = hip_ops.embedding_backward(grad_output.detach(), ids, lo, hi, padding_idx, scale_grad_by_freq)
        return dw, None, None, None, None, None


class DistributedEmbedding(Module):
    r"""Lookup table of ``num_embeddings`` vectors of size ``embedding_dim``
    whose last dimension is partitioned by the last dimension of ``P_x``.

    Signature of the reference.  ``padding_idx`` and ``scale_grad_by_freq``
    act on the gradient as they do in ``torch.nn.functional.embedding``;
    ``max_norm`` renormalises, in place and before the lookup, the rows that are
    looked up -- every worker its own columns by their own norm, as happens when
    the reference hands its local table to ``F.embedding``; ``sparse=True`` (a
    sparse gradient tensor) is refused.

    Without ``vocab_shard`` every id must lie in ``[0, num_embeddings)``; the
    kernel does not look (an id outside yields a zero row and no gradient).
    ``distdl_amd.config.check_embedding_ids = True`` (environment
    ``DISTDL_CHECK_EMBEDDING_IDS=1``) makes ``forward`` check the ids first and
    raise ``IndexError``, at the price of a device synchronisation per call.
    """

    def __init__(self, P_x, num_embeddings, embedding_dim, padding_idx=None,
                 max_norm=None, norm_type=2., scale_grad_by_freq=False, sparse=False,
                 _weight=None, _freeze=False, collect_state=False, device=None,
                 dtype=None, scale_backward=None, vocab_shard=None):
        super().__init__()
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        if padding_idx is not None:
            if padding_idx > 0:
                assert padding_idx < self.num_embeddings, 'Padding_idx must be within num_embeddings'
            elif padding_idx < 0:
                assert padding_idx >= -self.num_embeddings, 'Padding_idx must be within num_embeddings'
                padding_idx = self.num_embeddings + padding_idx
        if collect_state:
            raise NotImplementedError("collect_state=True is not part of this build")
        if sparse:
            raise NotImplementedError("sparse=True (a sparse gradient tensor) is not part of this build; "
                                      "the gradient of the table is dense")
        self.padding_idx = padding_idx
        self.max_norm = max_norm
        self.norm_type = norm_type
        self.scale_grad_by_freq = scale_grad_by_freq
        self.sparse = sparse
        self.collect_state = collect_state
        self.dtype = dtype
        self.P_x = P_x
        if not self.P_x.active:
            return

        if vocab_shard is None:
            vocab_shard = (0, num_embeddings)
        self.vocab_lo, self.vocab_hi = int(vocab_shard[0]), int(vocab_shard[1])
        if not 0 <= self.vocab_lo <= self.vocab_hi <= num_embeddings:
            raise ValueError(f"vocab_shard {vocab_shard} is not inside [0, {num_embeddings}]")
        rows_local = self.vocab_hi - self.vocab_lo

        # Workers with index 0 in every dimension but the last store the table.
        weight_partition_shape = [1] * P_x.dim
        weight_partition_shape[-1] = int(P_x.shape[-1])
        index_weight = [slice(0, 1)] * P_x.dim
        index_weight[-1] = slice(0, int(P_x.shape[-1]))
        weight_workers = worker_layout(P_x.shape)[tuple(index_weight)].reshape(-1).tolist()
        P_weight_base = P_x.create_partition_inclusive(weight_workers)
        self.P_weight = P_weight_base.create_cartesian_topology_partition(weight_partition_shape)
        P_weight_base.deactivate()
        self.broadcast = Broadcast(self.P_weight, self.P_x, scale_backward=scale_backward)

        embedding_dim_local = int(compute_subshape(P_x.shape[-1], P_x.index[-1], [embedding_dim])[0])
        dev = P_x.device if device is None else device
        if _weight is not None:
            assert _weight.shape[-1] == embedding_dim_local
            assert _weight.shape[-2] == rows_local
            if self.P_weight.active:
                self.weight = torch.nn.Parameter(_weight, requires_grad=not _freeze)
        elif self.P_weight.active:
            self.weight = torch.nn.Parameter(torch.empty((rows_local, embedding_dim_local), device=dev, dtype=dtype),
                                             requires_grad=not _freeze)
            self.reset_parameters()
        else:
            self.register_buffer('weight', zero_volume_tensor(device=dev, requires_grad=True, dtype=self.dtype))
        self.weight_buffer = None

    def reset_parameters(self, mean=0.0, std=1.0):
        """Every storing worker draws its own columns (the reference draws the
        whole table on the root worker and scatters it, :150-160)."""
        if self.P_weight.active:
            with torch.no_grad():
                torch.nn.init.normal_(self.weight, mean=mean, std=std)
        self._fill_padding_idx_with_zero()

    def extra_repr(self) -> str:
        return f'num_embeddings={self.num_embeddings}, embedding_dim={self.embedding_dim}'

    def _fill_padding_idx_with_zero(self):
        if self.padding_idx is not None and self.P_weight.active:
            if self.vocab_lo <= self.padding_idx < self.vocab_hi:
                with torch.no_grad():
                    self.weight[self.padding_idx - self.vocab_lo].fill_(0)

    def prefetch_weights(self):
        if self.P_x.size == 1:
            return
        self.weight_buffer = self.broadcast(self.weight)

    def forward(self, input):
        if not self.P_x.active:
            return zero_volume_tensor(device=self.P_x.device, dtype=self.dtype)
        if self.weight_buffer is None:
            weight = self.broadcast(self.weight)
        else:
            weight = self.weight_buffer
            self.weight_buffer = None
        if config.check_embedding_ids and input.numel() > 0:
            lo, hi = (int(v) for v in torch.aminmax(input))
            if lo < 0 or hi >= self.num_embeddings:
                raise IndexError(f"token ids span [{lo}, {hi}], outside the table's [0, {self.num_embeddings})")
        if self.max_norm is not None:
            # As F.embedding does: in place on the tensor that is looked up (every
            # worker scales its own columns by their own norm), outside autograd.
            hip_ops.embedding_renorm(weight.detach(), input, self.vocab_lo, self.vocab_hi, self.max_norm, self.norm_type)
        return _EmbeddingShard.apply(weight, input, self.vocab_lo, self.vocab_hi, self.padding_idx,
                                     bool(self.scale_grad_by_freq))
