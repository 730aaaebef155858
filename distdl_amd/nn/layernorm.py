"""DistributedLayerNorm (reference: nn/layernorm.py:15-321).

Constructor and ``forward`` signature are the reference's.  The arithmetic of
the distributed branch (reference :295-309: local mean, all-reduce, local mean
of squared deviations, all-reduce, normalise, affine -- six or more elementwise
kernels and two collectives) runs here as two HIP kernels around ONE gather of
per-row ``{mean, M2}`` pairs; the combination rule reproduces the reference's
mean of local means and mean of local variances exactly.  When the normalised
dimensions are not partitioned the reference calls
``torch.nn.functional.layer_norm`` (:310-319); here that is one HIP kernel.
Inputs may be float32, bfloat16 or float16, forward and backward; sums, means
and reciprocal deviations are float32 and results are rounded once.
"""

import numbers

import numpy as np
import torch

from .. import _lib
from .. import hip_ops
from ..utilities.slicing import compute_subshape
from ..utilities.slicing import range_index
from ..utilities.slicing import worker_layout
from ..utilities.torch import zero_volume_tensor
from .all_sum_reduce import AllSumReduce
from .broadcast import Broadcast
from .module import Module

STATS_TAG = "layernorm_stats"


BWD_SUMS_TAG = "layernorm_backward_sums"


def _shard_forward(input, weight, bias, P_reduce, part_cols, eps, part_cols_arr, stats_buffers, keep):
    """Forward of one shard: ``(y, x2d, mean, rstd, gamma)``; mean and rstd are
    None unless ``keep``.  ``stats_buffers``: the layer's cache of gathered
    statistics buffers ``[P, rows, 2]`` by row count (the stats kernel writes
    this worker's slot in place, the transport fills the others)."""
    x = input.detach()
    cols = int(part_cols[P_reduce.rank if P_reduce.active else 0])
    x2d = x.reshape(-1, cols)
    if x2d.shape[1] > 1 and x2d.stride(1) != 1:
        x2d = hip_ops.contiguous(x2d)
    gamma = None if weight is None else weight.detach().reshape(-1)
    beta = None if bias is None else bias.detach().reshape(-1)
    nparts = len(part_cols)
    if nparts > 1:
        rows = x2d.shape[0]
        gathered = stats_buffers.get(rows)
        if gathered is None or gathered.device != x2d.device:
            gathered = stats_buffers[rows] = torch.zeros((nparts, rows, 2), dtype=torch.float32, device=x2d.device)
        transport = P_reduce._world.transport
        if transport.peers_gathered_ahead(P_reduce, gathered, tag=STATS_TAG) and \
           hip_ops.ln_joined_supported(x2d, nparts, gamma, beta):
            # The peers' statistics are there already: one launch, one read of x.
            res = hip_ops.ln_stats_normalize(x2d, gathered, P_reduce.rank, part_cols, gamma, beta, eps, want_stats=keep,
                                             part_cols_arr=part_cols_arr)
        else:
            hip_ops.ln_partial_stats(x2d, out=gathered[P_reduce.rank])
            transport.allgather_into(P_reduce, gathered, tag=STATS_TAG)
            res = hip_ops.ln_normalize_affine(x2d, gathered, part_cols, gamma, beta, eps, want_stats=keep,
                                              part_cols_arr=part_cols_arr)
    else:
        res = hip_ops.layer_norm(x2d, gamma, beta, eps, want_stats=keep)
    if not keep:
        return res.view(input.shape), x2d, None, None, gamma
    y, mean, rstd = res
    return y.view(input.shape), x2d, mean, rstd, gamma


class _LayerNormShard(torch.autograd.Function):
    """Local shard of a layer norm whose statistics span ``P_reduce``, and its
    adjoint: the gradient autograd derives from the reference's forward
    (nn/layernorm.py:230-247, 295-309), whose all-reduces are self-adjoint."""

    @staticmethod
    def forward(ctx, input, weight, bias, P_reduce, part_cols, eps, part_cols_arr=None, stats_buffers=None):
        y, x2d, mean, rstd, gamma = _shard_forward(input, weight, bias, P_reduce, part_cols, eps, part_cols_arr,
                                                   {} if stats_buffers is None else stats_buffers, True)
        ctx.save_for_backward(x2d, mean, rstd, gamma)
        ctx.P_reduce, ctx.nparts, ctx.cols = P_reduce, len(part_cols), x2d.shape[1]
        ctx.param_shapes = (None if weight is None else weight.shape, None if bias is None else bias.shape)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        x2d, mean, rstd, gamma = ctx.saved_tensors
        need_x, need_w, need_b = ctx.needs_input_grad[:3]
        dy2d = grad_output.detach().reshape(-1, ctx.cols)
        if dy2d.dtype != x2d.dtype:
            dy2d = dy2d.to(x2d.dtype)
        if dy2d.shape[1] > 1 and dy2d.stride(1) != 1:
            dy2d = hip_ops.contiguous(dy2d)
        dx = dw = db = None
        w_shape, b_shape = ctx.param_shapes
        want_w, want_b = need_w and w_shape is not None, need_b and b_shape is not None
        fused = need_x and (want_w or want_b)        # two launches instead of four
        if need_x and ctx.nparts == 1 and hip_ops.ln_backward_one_pass_supported(dy2d, x2d, gamma):
            # rows held whole: this worker's sums are the row's sums, so dx comes out of the pass that forms them
            dx, dw, db = hip_ops.ln_backward_one_pass(dy2d, x2d, mean, rstd, gamma, 1.0 / ctx.cols, want_gamma=want_w,
                                                      want_beta=want_b)
            dx = dx.view(grad_output.shape)
        elif need_x:
            if fused:
                sums, work = hip_ops.ln_backward_partial_params(dy2d, x2d, mean, rstd, gamma)
            else:
                sums = hip_ops.ln_backward_partial(dy2d, x2d, mean, rstd, gamma)
            if ctx.nparts > 1:
                gathered = ctx.P_reduce._world.transport.allgather(ctx.P_reduce, sums, tag=BWD_SUMS_TAG).contiguous()
            else:
                gathered = sums.unsqueeze(0)
            weight_a = 1.0 / (ctx.nparts * ctx.cols)
            if fused:
                dx, dw, db = hip_ops.ln_backward_input_params(dy2d, x2d, mean, rstd, gamma, gathered, weight_a, work,
                                                              want_w, want_b)
            else:
                dx = hip_ops.ln_backward_input(dy2d, x2d, mean, rstd, gamma, gathered, weight_a)
            dx = dx.view(grad_output.shape)
        elif want_w or want_b:
            dw, db = hip_ops.ln_backward_params(dy2d, x2d, mean, rstd, want_w, want_b)
        dw = None if dw is None else dw.view(w_shape)
        db = None if db is None else db.view(b_shape)
        return dx, dw, db, None, None, None, None, None


class DistributedLayerNorm(Module):
    r"""Layer normalisation over the last ``len(normalized_shape)`` dimensions of
    a tensor partitioned by ``P_x``; those dimensions may themselves be
    partitioned.

    Parameters
    ----------
    P_x :
        Partition of the input (and output) tensor.
    normalized_shape :
        Global extent(s) of the normalised dimensions.
    elementwise_affine, eps :
        As ``torch.nn.LayerNorm``.
    collect_state, device, dtype, scale_backward :
        Accepted for signature compatibility; ``collect_state=True`` (gathering
        the parameters into the state dict) is not part of this build.
    """

    def __init__(self, P_x, normalized_shape, elementwise_affine=True, eps=1e-5,
                 collect_state=False, device=None, dtype=None, scale_backward=None):
        super().__init__()
        self.P_x = P_x
        if not self.P_x.active:
            return
        if collect_state:
            raise NotImplementedError("collect_state=True is not part of this build")
        if device is None:
            device = P_x.device
        self.eps = eps
        self.elementwise_affine = elementwise_affine
        self.collect_state = collect_state
        self.dtype = dtype
        if isinstance(normalized_shape, numbers.Integral):
            normalized_shape = (normalized_shape,)
        self.normalized_shape = tuple(int(n) for n in normalized_shape)
        num_dim = len(self.normalized_shape)

        # Dimensions the statistics run over, and the workers sharing them.
        self.dim_reduce = tuple(range(P_x.dim))[-num_dim:]
        self.allreduce = AllSumReduce(P_x, axes_reduce=self.dim_reduce)
        self.dim_reduce_slice = slice(P_x.dim - num_dim, P_x.dim)
        self.dim_bcast_slice = slice(0, P_x.dim - num_dim)
        reduce_shape = np.asarray(P_x.shape[self.dim_reduce_slice]).astype(int)
        self.num_reduce = int(np.prod(reduce_shape))

        # Columns held by every worker of the reduction group, in group order.
        self.part_cols = [int(np.prod(compute_subshape(reduce_shape, idx, self.normalized_shape)))
                          for idx in range_index(reduce_shape)]
        local_norm_shape = compute_subshape(reduce_shape, P_x.index[self.dim_reduce_slice], self.normalized_shape)
        self._part_cols_arr = _lib.i64_array(self.part_cols)     # what the normalize kernel's entry point takes
        self._checked_shape = None                               # last input shape found consistent with part_cols
        self._stats_buffers = {}                                 # rows -> gathered statistics buffer [P, rows, 2]
        self._call_plan = None                                   # what _forward_contiguous worked out for the last shape

        if self.elementwise_affine:
            # Parameters live on the workers with index 0 in every dimension that
            # is not normalised, and are broadcast along those dimensions.
            weight_partition_shape = np.copy(P_x.shape)
            weight_partition_shape[self.dim_bcast_slice] = 1
            index = [0] * P_x.dim
            for i in range(self.dim_reduce_slice.start, self.dim_reduce_slice.stop):
                index[i] = slice(0, int(P_x.shape[i]))
            storage_workers = worker_layout(P_x.shape)[tuple(index)].reshape(-1).tolist()
            P_w_base = P_x.create_partition_inclusive(storage_workers)
            P_w = P_w_base.create_cartesian_topology_partition(weight_partition_shape)
            P_w_base.deactivate()
            self.P_w = P_w
            self.broadcast = Broadcast(P_w, P_x, scale_backward=scale_backward)

            shape_local = [1] * P_x.dim
            shape_local[self.dim_reduce_slice] = [int(n) for n in local_norm_shape]
            if P_w.active:
                self.weight = torch.nn.Parameter(torch.empty(tuple(shape_local), device=device, dtype=dtype))
                self.bias = torch.nn.Parameter(torch.empty(tuple(shape_local), device=device, dtype=dtype))
            else:
                self.register_buffer('weight', zero_volume_tensor(device=device, requires_grad=True, dtype=dtype))
                self.register_buffer('bias', zero_volume_tensor(device=device, requires_grad=True, dtype=dtype))
            self.weight_buffer = None
            self.bias_buffer = None
        else:
            self.register_parameter('weight', None)
            self.register_parameter('bias', None)
        self.reset_parameters()

    def reset_parameters(self):
        if self.elementwise_affine and self.P_w.active:
            torch.nn.init.ones_(self.weight)
            torch.nn.init.zeros_(self.bias)

    def extra_repr(self) -> str:
        return f'normalized_shape={self.normalized_shape}'

    def prefetch_weights(self):
        """Fetches the parameters ahead of ``forward`` (reference :249-263)."""
        if self.P_x.size == 1 or not self.elementwise_affine:
            return
        self.weight_buffer = self.broadcast(self.weight)
        self.bias_buffer = self.broadcast(self.bias)

    def _forward_contiguous(self, input, weight, bias):
        """The forward of ``_shard_forward`` for a contiguous input when no
        gradient is recorded: everything that only depends on the input's
        shape (row and column counts, the gathered-statistics buffer and the
        address of this worker's slot in it) is worked out once per shape, and a
        call is the two entry points with the transport's gather between -- or
        the single-launch entry point when the peers' statistics are in the
        buffer beforehand."""
        plan = self._call_plan
        if plan is None or plan[0] != input.shape or plan[1] != input.dtype or plan[2] != input.device:
            P_reduce = self.allreduce.P_allreduce
            nparts = len(self.part_cols)
            cols = int(self.part_cols[P_reduce.rank if (nparts > 1 and P_reduce.active) else 0])
            rows = input.numel() // cols
            gathered = own = None
            if nparts > 1:
                gathered = self._stats_buffers.get(rows)
                if gathered is None or gathered.device != input.device:
                    gathered = self._stats_buffers[rows] = torch.zeros((nparts, rows, 2), dtype=torch.float32,
                                                                       device=input.device)
                own = gathered.data_ptr() + P_reduce.rank * rows * 8
            joinable = 1 < nparts <= 64 and cols <= 16384 and cols % 4 == 0     # what ddl_ln_stats_normalize takes
            plan = self._call_plan = (input.shape, input.dtype, input.device, rows, cols, hip_ops._LN_DTYPES[input.dtype],
                                      nparts, gathered, own, P_reduce, _lib.load(), joinable, 4 * input.element_size())
        _, _, _, rows, cols, dt, nparts, gathered, own, P_reduce, lib, joinable, quad = plan
        if weight is not None and (weight.numel() != cols or bias.numel() != cols):
            raise ValueError(f"DistributedLayerNorm parameters hold {weight.numel()} / {bias.numel()} elements, "
                             f"the local rows hold {cols}")
        y = torch.empty_like(input)
        stream = hip_ops._stream()
        gamma = None if weight is None else weight.data_ptr()
        beta = None if bias is None else bias.data_ptr()
        if nparts > 1 and joinable and input.data_ptr() % quad == 0 and \
           (weight is None or (weight.data_ptr() % quad == 0 and bias.data_ptr() % quad == 0)) and \
           P_reduce._world.transport.peers_gathered_ahead(P_reduce, gathered, tag=STATS_TAG):
            rc = lib.ddl_ln_stats_normalize(input.data_ptr(), dt, rows, cols, cols, gathered.data_ptr(), nparts, P_reduce.rank,
                                            self._part_cols_arr, gamma, beta, self.eps, y.data_ptr(), cols, None, None,
                                            stream)
            if rc:
                _lib.check(rc, "ddl_ln_stats_normalize")
        elif nparts > 1:
            rc = lib.ddl_ln_partial_stats(input.data_ptr(), dt, rows, cols, cols, own, stream)
            if rc:
                _lib.check(rc, "ddl_ln_partial_stats")
            P_reduce._world.transport.allgather_into(P_reduce, gathered, tag=STATS_TAG)
            rc = lib.ddl_ln_normalize_affine(input.data_ptr(), dt, rows, cols, cols, gathered.data_ptr(), nparts,
                                             self._part_cols_arr, gamma, beta, self.eps, y.data_ptr(), cols, None, None,
                                             stream)
            if rc:
                _lib.check(rc, "ddl_ln_normalize_affine")
        else:
            rc = lib.ddl_layer_norm(input.data_ptr(), dt, rows, cols, cols, gamma, beta, self.eps, y.data_ptr(), cols,
                                    None, None, stream)
            if rc:
                _lib.check(rc, "ddl_layer_norm")
        return y

    def forward(self, input):
        if not self.P_x.active:
            return input
        weight = bias = None
        if self.elementwise_affine:
            if self.weight_buffer is not None:
                weight, bias = self.weight_buffer, self.bias_buffer
                self.weight_buffer = self.bias_buffer = None
            elif self.broadcast.identity:      # every worker stores its own parameters: nothing to fetch
                weight, bias = self.weight, self.bias
            else:
                weight = self.broadcast(self.weight)
                bias = self.broadcast(self.bias)
        if input.dtype not in (torch.float32, torch.bfloat16, torch.float16):
            raise NotImplementedError(f"DistributedLayerNorm kernels take float32, bfloat16 and float16, got {input.dtype}")
        if weight is not None and weight.dtype != input.dtype:
            raise ValueError(f"DistributedLayerNorm parameters are {weight.dtype}, the input is {input.dtype}")
        if input.shape != self._checked_shape:
            local_cols = int(np.prod(input.shape[self.dim_reduce_slice.start - self.P_x.dim:]))
            mine = self.allreduce.P_allreduce.rank if self.num_reduce > 1 else 0
            if local_cols != self.part_cols[mine]:
                raise ValueError(f"input shard has {local_cols} normalised elements, the partition of "
                                 f"normalized_shape={self.normalized_shape} gives this worker {self.part_cols[mine]}")
            self._checked_shape = input.shape
        wants_grad = torch.is_grad_enabled() and (input.requires_grad or (weight is not None and weight.requires_grad) or
                                                  (bias is not None and bias.requires_grad))
        if not wants_grad:      # nothing to record: skip the autograd machinery and the statistics kept for backward
            if input.is_cuda and input.is_contiguous() and (weight is None or (weight.is_contiguous() and bias.is_contiguous())):
                return self._forward_contiguous(input, weight, bias)
            return _shard_forward(input, weight, bias, self.allreduce.P_allreduce, self.part_cols, self.eps,
                                  self._part_cols_arr, self._stats_buffers, False)[0]
        return _LayerNormShard.apply(input, weight, bias, self.allreduce.P_allreduce, self.part_cols, self.eps,
                                     self._part_cols_arr, self._stats_buffers)
