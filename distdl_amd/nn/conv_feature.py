"""Feature-space partitioned convolution (reference: nn/conv_feature.py:16-466).

What this build accelerates is the input staging in front of the local
convolution (reference forward, :399-410): zero padding on global boundaries,
halo exchange with the neighbours, cropping to the needed range.  When every
ghost slab is available before the call (solo transport) the padding, the ghost
fill and the packing of the outgoing slabs run as ONE kernel
(``ddl_halo_pad_exchange``); otherwise the padding kernel is followed by the
dimension-ordered HaloExchange layer.  The convolution itself stays the stock
``torch.nn.ConvNd`` the reference calls (:411).
"""

import numpy as np
import torch
import torch.nn.functional as F

from .. import hip_ops
from ..backends.stub_hip import buffer as _buffer
from ..utilities.slicing import assemble_slices
from ..utilities.slicing import compute_nd_slice_shape
from ..utilities.torch import TensorStructure
from ..utilities.torch import zero_volume_tensor
from .broadcast import Broadcast
from .halo_exchange import HaloExchange
from .mixins.conv_mixin import ConvMixin
from .mixins.halo_mixin import HaloMixin
from .module import Module


class _HaloStaging(torch.autograd.Function):
    """pad + exchange of one shard through the fused kernel.  With respect to
    the shard the operation is an embedding into the padded tensor (the ghost
    strips are filled from buffers, not from the shard), so its adjoint is the
    crop of the padded gradient -- a strided box copy."""

    @staticmethod
    def forward(ctx, input, plan, ghost_bufs, bulk_bufs):
        x = input.detach()
        if not x.is_contiguous():
            x = hip_ops.contiguous(x)
        ctx.plan = plan
        return plan.run(x, ghost_bufs, bulk_bufs)

    @staticmethod
    def backward(ctx, grad_output):
        plan = ctx.plan
        g = grad_output.detach()
        dx = torch.empty(plan.x_shape, dtype=g.dtype, device=g.device)
        inner = [slice(p[0], p[0] + n) for p, n in zip(plan.pad, plan.x_shape)]
        hip_ops.copy_box(g, inner, dx, [slice(0, n) for n in plan.x_shape])
        return dx, None, None, None


class _Crop(torch.autograd.Function):
    """``padded[slices]`` as a contiguous tensor (reference :410, where the
    slice is a view and the stock convolution makes the copy): one pass of the
    box kernel over the window.  Adjoint: the gradient placed into a zeroed
    tensor of the padded shape."""

    @staticmethod
    def forward(ctx, padded, slices):
        src = padded.detach()
        ctx.padded_shape, ctx.slices = tuple(src.shape), slices
        out = torch.empty([int(s.stop) - int(s.start) for s in slices], dtype=src.dtype, device=src.device)
        if out.numel():
            hip_ops.copy_box(src, slices, out, [slice(0, n) for n in out.shape])
        return out

    @staticmethod
    def backward(ctx, grad_output):
        g = grad_output.detach()
        dp = torch.empty(ctx.padded_shape, dtype=g.dtype, device=g.device)
        whole = hip_ops.BoxPlan(dp.shape, dp.stride(), [([0] * dp.dim(), list(dp.shape))])
        whole.zero(dp)
        if g.numel():
            hip_ops.copy_box(g, [slice(0, n) for n in g.shape], dp, ctx.slices)
        return dp, None


class DistributedFeatureConvBase(Module, HaloMixin, ConvMixin):
    r"""Convolution over a tensor partitioned in feature space only:
    ``P_x ~ 1 x 1 x P_{d-1} x ... x P_0``; the output reuses ``P_x``.  Weights
    live on worker 0 and are broadcast.  Arguments as the reference (and as the
    wrapped ``torch.nn.ConvNd``)."""

    TorchConvType = None
    num_dimensions = None

    def __init__(self, P_x, in_channels, out_channels, kernel_size, stride=1, padding=0, padding_mode='zeros',
                 dilation=1, groups=1, bias=True, buffer_manager=None, collect_state=False):
        super().__init__()
        self.P_x = P_x
        if buffer_manager is None:
            buffer_manager = self._distdl_backend.BufferManager()
        elif not isinstance(buffer_manager, self._distdl_backend.BufferManager):
            raise ValueError("Buffer manager type does not match backend.")
        self.buffer_manager = buffer_manager
        if not self.P_x.active:
            return
        if padding_mode != 'zeros':
            raise NotImplementedError("only zero padding is staged by the HIP kernels")

        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = self._expand_parameter(kernel_size)
        self.stride = self._expand_parameter(stride)
        self.padding = self._expand_parameter(padding)
        self.padding_mode = padding_mode
        self.dilation = self._expand_parameter(dilation)
        self.groups = groups
        self.use_bias = bias
        self.collect_state = collect_state

        # A stock layer provides the default initialisation of the parameters;
        # only worker 0 keeps them, the others receive them by broadcast.
        template = self.TorchConvType(in_channels=in_channels, out_channels=out_channels,
                                      kernel_size=self.kernel_size, stride=self.stride, padding=0,
                                      padding_mode='zeros', dilation=self.dilation, groups=groups, bias=bias,
                                      device=P_x.device)
        self._conv_fn = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}[self.num_dimensions]

        dims = len(self.P_x.shape)
        self.global_padding = np.concatenate([np.zeros(dims - len(self.padding), dtype=int),
                                              np.asarray(self.padding, dtype=int)])
        self.local_padding = self._compute_local_padding(np.stack([self.global_padding, self.global_padding], axis=1))

        P_wb = self.P_x.create_partition_inclusive([0])
        self.P_wb_cart = P_wb.create_cartesian_topology_partition([1])
        P_wb.deactivate()
        if self.P_wb_cart.active:
            self.weight = torch.nn.Parameter(template.weight.detach().clone())
            if bias:
                self.bias = torch.nn.Parameter(template.bias.detach().clone())
            else:
                self.register_buffer('bias', None)
        else:
            # Like the parameters they stand for, the empty tensors of the other
            # workers require gradients (reference :174-187): autograd then runs
            # the broadcast adjoint -- a collective -- on every worker.
            self.register_buffer('weight', zero_volume_tensor(device=P_x.device, requires_grad=True))
            if bias:
                self.register_buffer('bias', zero_volume_tensor(device=P_x.device, requires_grad=True))
            else:
                self.register_buffer('bias', None)

        self.w_broadcast = Broadcast(self.P_wb_cart, self.P_x, preserve_batch=False)
        if bias:
            self.b_broadcast = Broadcast(self.P_wb_cart, self.P_x, preserve_batch=False)

        self.needed_slices = None
        self.halo_layer = None
        self._staging_plan = None
        self._distdl_is_setup = False
        self._input_tensor_structure = TensorStructure()

    def _expand_parameter(self, param):
        param = np.atleast_1d(param)
        if len(param) == 1:
            param = np.ones(self.num_dimensions, dtype=int) * param[0]
        elif len(param) != self.num_dimensions:
            raise ValueError('Invalid parameter: ' + str(param))
        return tuple(int(p) for p in param)

    def _compute_local_padding(self, padding):
        """Explicit zero padding exists only on the sides of the shard that lie
        on the global boundary (reference :367-377)."""
        on_left = [k == 0 for k in self.P_x.index]
        on_right = [k == d - 1 for k, d in zip(self.P_x.index, self.P_x.shape)]
        return np.where(np.stack((on_left, on_right), axis=1), padding, 0)

    def _distdl_module_setup(self, input):
        """Halo geometry for the structure of ``input[0]``, computed on the
        explicitly padded global tensor with padding 0 (reference :263-328)."""
        self._distdl_is_setup = True
        self._input_tensor_structure = TensorStructure(input[0])
        if not self.P_x.active:
            return
        backend = self._distdl_backend
        x_global_structure = backend.assemble_global_tensor_structure(input[0], self.P_x)
        x_global_shape_after_pad = np.asarray(x_global_structure.shape) + 2 * self.global_padding
        padded = TensorStructure(input[0])
        padded.shape = np.asarray(input[0].shape) + np.sum(self.local_padding, axis=1)
        subtensor_shapes = backend.tensor_decomposition.compute_subtensor_shapes_unbalanced(padded, self.P_x)

        halo_shape, recv_buffer_shape, send_buffer_shape, needed_ranges = self._compute_exchange_info(
            x_global_shape_after_pad, self.kernel_size, self.stride, self._expand_parameter(0), self.dilation,
            self.P_x.active, self.P_x.shape, self.P_x.index, subtensor_shapes=subtensor_shapes)
        self.halo_shape = halo_shape
        self.recv_buffer_shape = recv_buffer_shape
        self.send_buffer_shape = send_buffer_shape
        self.halo_layer = HaloExchange(self.P_x, halo_shape, recv_buffer_shape, send_buffer_shape,
                                       buffer_manager=self.buffer_manager)
        self.needed_slices = assemble_slices(needed_ranges[:, 0], needed_ranges[:, 1])

        total_padding = self.local_padding + self.halo_shape
        self._pad_only_plan = hip_ops.HaloPadPlan(input[0].shape, total_padding,
                                                  np.zeros_like(total_padding), np.zeros_like(total_padding))
        self._staging_plan = hip_ops.HaloPadPlan(input[0].shape, total_padding, recv_buffer_shape, send_buffer_shape)

    def _distdl_module_teardown(self, input):
        self.needed_slices = None
        self.halo_layer = None
        self._staging_plan = None
        self._distdl_is_setup = False
        self._input_tensor_structure = TensorStructure()

    def _distdl_input_changed(self, input):
        return self._input_tensor_structure != TensorStructure(input[0])

    def _slab_views(self, padded_shape):
        """Ghost and bulk buffers of the halo layer as ``[dim][side]`` tables."""
        layer = self.halo_layer
        if layer.slices is None:
            SliceTable = self._distdl_backend.functional.halo_exchange.SliceTable
            layer.slices = SliceTable(layer._assemble_slices(padded_shape, layer.recv_buffer_shape,
                                                             layer.send_buffer_shape))
            layer.buffers = layer.allocate_halo_exchange_buffers(layer.buffer_manager, layer.slices,
                                                                 layer.recv_buffer_shape, layer.send_buffer_shape,
                                                                 self._input_tensor_structure.dtype)
        ghost, bulk = [], []
        for i in range(len(padded_shape)):
            lbs, lgs, rbs, rgs = layer.slices[i]
            lbb, lgb, rbb, rgb = layer.buffers[i]

            def view(buf, sl):
                return None if buf is None else buf.get_view(compute_nd_slice_shape(sl))
            ghost.append([view(lgb, lgs), view(rgb, rgs)])
            bulk.append([view(lbb, lbs), view(rbb, rbs)])
        return ghost, bulk

    def stage_input(self, input):
        """Padded, exchanged and cropped input of the local convolution."""
        total_padding = self.local_padding + self.halo_shape
        transport = self.P_x._world.transport
        if total_padding.sum() == 0 and self.P_x.size == 1:
            return input
        if getattr(transport, "ghosts_preloaded", False):
            ghost, bulk = self._fused_slabs(input)
            exchanged = _HaloStaging.apply(input, self._staging_plan, ghost, bulk)
        else:
            padded = _HaloStaging.apply(input, self._pad_only_plan, None, None)
            exchanged = self.halo_layer(padded)
        crop = tuple(slice(int(sl.start), int(sl.stop)) for sl in self.needed_slices)
        if all(sl.start == 0 and sl.stop == n for sl, n in zip(crop, exchanged.shape)):
            return exchanged
        # A window smaller than the padded tensor (strided or unbalanced
        # geometries): handed to the convolution as a contiguous tensor.
        return _Crop.apply(exchanged, crop)

    def _fused_slabs(self, input):
        """Ghost and bulk slabs of the fused pass as ``[dim][side]`` tables of
        views into pooled buffers.  The halo layer's four buffers are shared by
        all dimensions (reference buffer_allocator.py:69-74), which only works
        when dimensions are exchanged one after the other; one pass over all
        dimensions needs a slab per (dimension, side, kind), so it asks the
        same buffer manager for that many buffers (the first four are the halo
        layer's own: the two ways of staging never run together).  A slab's
        place in the pool is fixed by (dimension, side, kind), whether or not
        the slab exists, so two layers of one manager agree on which buffer
        is, say, the right ghost of dimension 3.  Pooled buffers are scratch:
        another layer of the same manager overwrites them, so ghost slabs that
        a caller seeds (solo transport) must be seeded again before each call
        unless this layer has the manager to itself.  Ghost views are zeroed
        when the layer first takes them, so slabs nobody seeded read as zeros."""
        plan = self._staging_plan
        slabs = getattr(self, "_fused_slab_cache", None)
        key = (tuple(input.shape), input.dtype, _buffer.reallocations())
        if slabs is None or slabs[0] != key:
            first_time = slabs is None
            wanted = [(d, s, kind, plan.slab_shape(d, s, kind))
                      for d in range(plan.ndim) for s in range(2) for kind in ("ghost", "bulk")]
            # dimensions in front of the first exchanged one take no place in the pool
            first = next((i for i, w in enumerate(wanted) if w[3] is not None), len(wanted)) // 4 * 4
            wanted = wanted[first:]
            while wanted and wanted[-1][3] is None:
                wanted.pop()
            pool = self.buffer_manager.request_buffers(len(wanted), dtype=input.dtype)
            for buf, w in zip(pool, wanted):
                if w[3] is not None:
                    buf.allocate_view(w[3])        # may reallocate: take the views only afterwards
            ghost = [[None, None] for _ in range(plan.ndim)]
            bulk = [[None, None] for _ in range(plan.ndim)]
            for buf, (d, s, kind, shape) in zip(pool, wanted):
                if shape is None:
                    continue
                view = buf.get_view(shape)
                if kind == "ghost" and first_time:
                    hip_ops.BoxPlan(view.shape, view.stride(), [([0] * view.dim(), list(view.shape))]).zero(view)
                (ghost if kind == "ghost" else bulk)[d][s] = view
            key = (tuple(input.shape), input.dtype, _buffer.reallocations())
            slabs = self._fused_slab_cache = (key, ghost, bulk)
        return slabs[1], slabs[2]

    def forward(self, input):
        if not self.P_x.active:
            return input
        weight = self.w_broadcast(self.weight)
        bias = self.b_broadcast(self.bias) if self.use_bias else None
        # The local convolution is the stock one the reference calls (:411).
        return self._conv_fn(self.stage_input(input), weight, bias, stride=self.stride, padding=0,
                             dilation=self.dilation, groups=self.groups)


class DistributedFeatureConv1d(DistributedFeatureConvBase):
    TorchConvType = torch.nn.Conv1d
    num_dimensions = 1


class DistributedFeatureConv2d(DistributedFeatureConvBase):
    TorchConvType = torch.nn.Conv2d
    num_dimensions = 2


class DistributedFeatureConv3d(DistributedFeatureConvBase):
    TorchConvType = torch.nn.Conv3d
    num_dimensions = 3
