"""Torch-tensor front end of the C ABI: device checks, pointer extraction and
the current HIP stream.  Nothing here computes; every function ends in one call
into ``libdistdl_hip.so`` and raises when that is impossible.
"""

import ctypes

import torch

from . import _lib

_ADD_DTYPES = {
    torch.float32: _lib.DDL_DT_F32,
    torch.float64: _lib.DDL_DT_F64,
    torch.bfloat16: _lib.DDL_DT_BF16,
    torch.float16: _lib.DDL_DT_F16,
    torch.int32: _lib.DDL_DT_I32,
    torch.int64: _lib.DDL_DT_I64,
}


# torch's raw-stream query costs a microsecond; building a torch.cuda.Stream
# object for every launch costs ten.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "distdl_amd: tensor on %s; the HIP path only accepts GPU tensors and there is no CPU fallback"
                % (t.device,))


def _ptr(t):
    return None if t is None else t.data_ptr()


class BoxPlan:
    """Box geometry of one strided tensor, converted to C arrays once.

    ``boxes`` is a list of ``(start, shape)`` pairs (or ``None`` for an absent
    box) in the coordinates of a tensor with the given shape / strides; the
    contiguous buffers on the other side are supplied per call.  Built where the
    reference builds its overlap lists (the forward pre-hook), used on every
    forward and adjoint call.
    """

    def __init__(self, tensor_shape, tensor_strides, boxes):
        self.ndim = len(tensor_shape)
        if self.ndim < 1 or self.ndim > _lib.DDL_MAX_DIMS:
            raise ValueError(f"tensors of rank {self.ndim} are not supported (1..{_lib.DDL_MAX_DIMS})")
        self.tensor_shape = tuple(int(s) for s in tensor_shape)
        self.tensor_strides = tuple(int(s) for s in tensor_strides)
        self.shape_arr = _lib.i64_array(self.tensor_shape)
        self.stride_arr = _lib.i64_array(self.tensor_strides)
        self.present = [b is not None for b in boxes]
        starts, shapes = [], []
        for b in boxes:
            if b is None:
                starts += [0] * self.ndim
                shapes += [0] * self.ndim
            else:
                starts += list(b[0])
                shapes += list(b[1])
        self.nbox = len(boxes)
        self.box_shapes = [None if b is None else tuple(int(v) for v in b[1]) for b in boxes]
        self.start_arr = _lib.i64_array(starts)
        self.boxshape_arr = _lib.i64_array(shapes)

    @classmethod
    def from_slices(cls, tensor, slice_list):
        boxes = []
        for sl in slice_list:
            if sl is None:
                boxes.append(None)
            else:
                boxes.append(([int(s.start) for s in sl], [int(s.stop) - int(s.start) for s in sl]))
        return cls(tensor.shape, tensor.stride(), boxes)

    def matches(self, tensor):
        return tuple(tensor.shape) == self.tensor_shape and tuple(tensor.stride()) == self.tensor_strides

    def _buf_ptrs(self, bufs, dtype, device):
        if len(bufs) != self.nbox:
            raise ValueError(f"expected {self.nbox} buffers, got {len(bufs)}")
        ptrs = []
        for buf, shape in zip(bufs, self.box_shapes):
            if buf is None or shape is None:
                ptrs.append(None)
                continue
            _require_gpu(buf)
            if buf.dtype != dtype or not buf.is_contiguous() or tuple(buf.shape) != shape:
                raise ValueError(f"buffer {tuple(buf.shape)}/{buf.dtype} does not match box {shape}/{dtype} "
                                 "or is not contiguous")
            ptrs.append(buf.data_ptr())
        return _lib.ptr_array(ptrs)

    def pack(self, tensor, bufs):
        """bufs[b][...] = tensor[box b]"""
        _require_gpu(tensor)
        if not self.matches(tensor):
            raise ValueError("tensor structure differs from the one this plan was built for")
        if self.nbox == 0:
            return
        ptrs = self._buf_ptrs(bufs, tensor.dtype, tensor.device)
        rc = _lib.load().ddl_pack_boxes(tensor.data_ptr(), self.shape_arr, self.stride_arr, self.ndim,
                                        tensor.element_size(), self.nbox, self.start_arr, self.boxshape_arr,
                                        ptrs, _stream())
        _lib.check(rc, "ddl_pack_boxes")

    def unpack(self, tensor, bufs, accumulate=False):
        """tensor[box b] = bufs[b]   (+= when accumulate)"""
        _require_gpu(tensor)
        if not self.matches(tensor):
            raise ValueError("tensor structure differs from the one this plan was built for")
        if self.nbox == 0:
            return
        ptrs = self._buf_ptrs(bufs, tensor.dtype, tensor.device)
        op, dt = _lib.DDL_OP_COPY, _lib.DDL_DT_BITS
        if accumulate:
            if tensor.dtype not in _ADD_DTYPES:
                raise ValueError(f"accumulating unpack is not available for {tensor.dtype}")
            op, dt = _lib.DDL_OP_ADD, _ADD_DTYPES[tensor.dtype]
        rc = _lib.load().ddl_unpack_boxes(tensor.data_ptr(), self.shape_arr, self.stride_arr, self.ndim,
                                          tensor.element_size(), self.nbox, self.start_arr, self.boxshape_arr,
                                          ptrs, op, dt, _stream())
        _lib.check(rc, "ddl_unpack_boxes")

    def zero(self, tensor):
        """tensor[box b] = 0 for every box"""
        _require_gpu(tensor)
        if not self.matches(tensor):
            raise ValueError("tensor structure differs from the one this plan was built for")
        if self.nbox == 0:
            return
        rc = _lib.load().ddl_zero_boxes(tensor.data_ptr(), self.shape_arr, self.stride_arr, self.ndim,
                                        tensor.element_size(), self.nbox, self.start_arr, self.boxshape_arr, _stream())
        _lib.check(rc, "ddl_zero_boxes")


def copy_box(src, src_slices, dst, dst_slices, accumulate=False):
    """dst[dst_slices] (+)= src[src_slices]; both strided, same box shape."""
    _require_gpu(src, dst)
    if src.dtype != dst.dtype:
        raise ValueError("copy_box: dtype mismatch")
    nd = src.dim()
    if dst.dim() != nd or len(src_slices) != nd or len(dst_slices) != nd:
        raise ValueError("copy_box: rank mismatch")
    box = _lib.ddl_box_t()
    box.ndim = nd
    soff = doff = 0
    for d in range(nd):
        n = int(src_slices[d].stop) - int(src_slices[d].start)
        if n != int(dst_slices[d].stop) - int(dst_slices[d].start):
            raise ValueError("copy_box: source and destination boxes differ in shape")
        if src_slices[d].start < 0 or src_slices[d].stop > src.shape[d] or \
           dst_slices[d].start < 0 or dst_slices[d].stop > dst.shape[d]:
            raise ValueError("copy_box: box outside tensor")
        box.shape[d] = n
        box.src_stride[d] = src.stride(d)
        box.dst_stride[d] = dst.stride(d)
        soff += int(src_slices[d].start) * src.stride(d)
        doff += int(dst_slices[d].start) * dst.stride(d)
    es = src.element_size()
    box.src = src.data_ptr() + soff * es
    box.dst = dst.data_ptr() + doff * es
    op, dt = _lib.DDL_OP_COPY, _lib.DDL_DT_BITS
    if accumulate:
        if src.dtype not in _ADD_DTYPES:
            raise ValueError(f"accumulating copy is not available for {src.dtype}")
        op, dt = _lib.DDL_OP_ADD, _ADD_DTYPES[src.dtype]
    rc = _lib.load().ddl_copy_boxes(ctypes.byref(box), 1, es, op, dt, _stream())
    _lib.check(rc, "ddl_copy_boxes")


def sum_boxes(srcs, src_slices, dst, dst_slices, divisor=1):
    """dst[dst_slices] = sum over q, in order, of srcs[q][src_slices] / divisor.

    One launch that reads every source once and writes the destination once;
    quotients and partial sums are rounded to the element type, as a chain of
    divisions and accumulating copies would round them.  All sources share
    shape and strides.  ``dst`` may be one of them when the slices coincide
    (scaling in place).  Sources that do not sit a multiple of 16 bytes apart,
    or more than 64 of them, go through the same arithmetic one source at a
    time (divided into a temporary, added by an accumulating box copy)."""
    srcs = list(srcs)
    if not srcs:
        raise ValueError("sum_boxes: no sources")
    first = srcs[0]
    _require_gpu(dst, *srcs)
    nd = first.dim()
    for t in srcs:
        if t.dtype != dst.dtype or tuple(t.shape) != tuple(first.shape) or t.stride() != first.stride():
            raise ValueError("sum_boxes: sources must agree in dtype, shape and strides with each other (dtype: and with dst)")
    if dst.dtype not in _ADD_DTYPES:
        raise ValueError(f"sums are not available for {dst.dtype}")
    if dst.dim() != nd or len(src_slices) != nd or len(dst_slices) != nd:
        raise ValueError("sum_boxes: rank mismatch")
    box = _lib.ddl_box_t()
    box.ndim = nd
    soff = doff = 0
    for d in range(nd):
        n = int(src_slices[d].stop) - int(src_slices[d].start)
        if n != int(dst_slices[d].stop) - int(dst_slices[d].start):
            raise ValueError("sum_boxes: source and destination boxes differ in shape")
        if src_slices[d].start < 0 or src_slices[d].stop > first.shape[d] or \
           dst_slices[d].start < 0 or dst_slices[d].stop > dst.shape[d]:
            raise ValueError("sum_boxes: box outside tensor")
        box.shape[d] = n
        box.src_stride[d] = first.stride(d)
        box.dst_stride[d] = dst.stride(d)
        soff += int(src_slices[d].start) * first.stride(d)
        doff += int(dst_slices[d].start) * dst.stride(d)
    es = dst.element_size()
    box.dst = dst.data_ptr() + doff * es
    ptrs = [t.data_ptr() + soff * es for t in srcs]
    one_launch = len(srcs) <= 64 and all((p - ptrs[0]) % 16 == 0 for p in ptrs)
    lib = _lib.load()
    dt = _ADD_DTYPES[dst.dtype]
    if one_launch:
        rc = lib.ddl_sum_boxes(ctypes.byref(box), _lib.ptr_array(ptrs), len(srcs), es, dt, float(divisor), _stream())
        _lib.check(rc, "ddl_sum_boxes")
        return
    # The same arithmetic source by source: the first one divided into dst, every other one divided into a
    # temporary of the box's shape and added to dst by an accumulating copy.
    rc = lib.ddl_sum_boxes(ctypes.byref(box), _lib.ptr_array(ptrs[:1]), 1, es, dt, float(divisor), _stream())
    _lib.check(rc, "ddl_sum_boxes")
    shape = [int(box.shape[d]) for d in range(nd)]
    whole = [slice(0, n) for n in shape]
    for t in srcs[1:]:
        if divisor == 1:
            copy_box(t, src_slices, dst, dst_slices, accumulate=True)
            continue
        tmp = torch.empty(shape, dtype=dst.dtype, device=dst.device)
        sum_boxes([t], src_slices, tmp, whole, divisor)
        copy_box(tmp, whole, dst, dst_slices, accumulate=True)


def scaled(t, divisor):
    """``t / divisor`` as a new tensor, through the sum kernel with one source
    (the scaling of a gradient ahead of an adjoint's sum)."""
    out = torch.empty(t.shape, dtype=t.dtype, device=t.device)
    if t.numel() == 0:
        return out
    src = t if t.is_contiguous() else contiguous(t)
    full = [slice(0, int(n)) for n in src.shape]
    sum_boxes([src], full, out, full, divisor)
    return out


def contiguous(t):
    """A row-major copy of a strided tensor, made by the box kernel."""
    if t.is_contiguous():
        return t
    _require_gpu(t)
    out = torch.empty(t.shape, dtype=t.dtype, device=t.device)
    if t.numel():
        full = [slice(0, int(n)) for n in t.shape]
        copy_box(t, full, out, full)
    return out


class HaloPadPlan:
    """Geometry of the fused pad + ghost fill + bulk pack call for one shard shape."""

    def __init__(self, x_shape, pad, recv, send):
        self.x_shape = tuple(int(s) for s in x_shape)
        self.ndim = len(self.x_shape)
        self.pad = [[int(p[0]), int(p[1])] for p in pad]
        self.recv = [[int(p[0]), int(p[1])] for p in recv]
        self.send = [[int(p[0]), int(p[1])] for p in send]
        self.padded_shape = tuple(s + p[0] + p[1] for s, p in zip(self.x_shape, self.pad))
        self.shape_arr = _lib.i64_array(self.x_shape)
        self.pad_arr = _lib.i64_array([v for p in self.pad for v in p])
        self.recv_arr = _lib.i64_array([v for p in self.recv for v in p])
        self.send_arr = _lib.i64_array([v for p in self.send for v in p])

    def slab_shape(self, dim, side, kind):
        """Shape of the ghost (kind='ghost') or bulk slab of (dim, side); None if empty."""
        widths = self.recv if kind == "ghost" else self.send
        w = widths[dim][side]
        if w == 0:
            return None
        shape = []
        for j in range(self.ndim):
            if j < dim:
                shape.append(self.padded_shape[j])
            elif j == dim:
                shape.append(w)
            else:
                shape.append(self.padded_shape[j] - self.recv[j][0] - self.recv[j][1])
        return tuple(shape)

    def run(self, x, ghost_bufs, bulk_bufs, out=None, kernel=_lib.DDL_HALO_AUTO):
        """ghost_bufs / bulk_bufs: ``[ndim][2]`` nested lists of tensors or None.
        ``kernel``: ``DDL_HALO_AUTO`` (library's choice), ``DDL_HALO_ROWS`` or
        ``DDL_HALO_LINES``; the results are identical."""
        _require_gpu(x)
        if tuple(x.shape) != self.x_shape or not x.is_contiguous():
            raise ValueError("halo_pad_exchange: input must be contiguous with the planned shape")
        if out is None:
            out = torch.empty(self.padded_shape, dtype=x.dtype, device=x.device)
        elif tuple(out.shape) != self.padded_shape or not out.is_contiguous() or out.dtype != x.dtype:
            raise ValueError("halo_pad_exchange: bad output tensor")
        gptr, bptr = [], []
        for d in range(self.ndim):
            for s in range(2):
                for kind, bufs, ptrs in (("ghost", ghost_bufs, gptr), ("bulk", bulk_bufs, bptr)):
                    buf = None if bufs is None else bufs[d][s]
                    shape = self.slab_shape(d, s, kind)
                    if buf is None or shape is None:
                        ptrs.append(None)
                        continue
                    _require_gpu(buf)
                    if tuple(buf.shape) != shape or not buf.is_contiguous() or buf.dtype != x.dtype:
                        raise ValueError(f"halo_pad_exchange: {kind} slab ({d},{s}) must be contiguous {shape}, "
                                         f"got {tuple(buf.shape)}")
                    ptrs.append(buf.data_ptr())
        rc = _lib.load().ddl_halo_pad_exchange(x.data_ptr(), out.data_ptr(), self.shape_arr, self.ndim,
                                               x.element_size(), self.pad_arr, self.recv_arr, self.send_arr,
                                               _lib.ptr_array(gptr), _lib.ptr_array(bptr), int(kernel), _stream())
        _lib.check(rc, "ddl_halo_pad_exchange")
        return out


_LN_DTYPES = {
    torch.float32: _lib.DDL_DT_F32,
    torch.bfloat16: _lib.DDL_DT_BF16,
    torch.float16: _lib.DDL_DT_F16,
}


def _ln_rows(x2d, name):
    """dtype code and row pitch of a 2-D LayerNorm operand (last stride 1)."""
    dt = _LN_DTYPES.get(x2d.dtype)
    if dt is None or x2d.dim() != 2 or (x2d.shape[1] > 1 and x2d.stride(1) != 1):
        raise ValueError(f"{name}: need a 2-D float32, bfloat16 or float16 tensor with unit column stride")
    return dt, (x2d.stride(0) if x2d.shape[0] > 1 else x2d.shape[1])


def _ln_params(x2d, gamma, beta, name):
    for p in (gamma, beta):
        if p is not None and (p.dtype != x2d.dtype or p.numel() != x2d.shape[1] or not p.is_contiguous()):
            raise ValueError(f"{name}: gamma / beta must be contiguous, of the input's dtype, with `cols` elements")


def ln_partial_stats(x2d, out=None):
    """{mean, M2} per row of a [rows, cols] view (last stride 1), fp32."""
    _require_gpu(x2d)
    dt, ld = _ln_rows(x2d, "ln_partial_stats")
    rows, cols = x2d.shape
    if out is None:
        out = torch.empty((rows, 2), dtype=torch.float32, device=x2d.device)
    rc = _lib.load().ddl_ln_partial_stats(x2d.data_ptr(), dt, rows, cols, ld, out.data_ptr(), _stream())
    _lib.check(rc, "ddl_ln_partial_stats")
    return out


def ln_normalize_affine(x2d, part_stats, part_cols, gamma, beta, eps, want_stats=False, part_cols_arr=None):
    """Combines [P, rows, 2] partial statistics and normalises x2d; returns y
    (and mean, rstd).  ``part_cols_arr``: ``part_cols`` already converted with
    ``_lib.i64_array`` (callers that run every step keep it)."""
    _require_gpu(x2d, part_stats, gamma, beta)
    dt, ld = _ln_rows(x2d, "ln_normalize_affine")
    rows, cols = x2d.shape
    nparts = len(part_cols)
    if part_stats.dtype != torch.float32 or tuple(part_stats.shape) != (nparts, rows, 2) or \
       not part_stats.is_contiguous():
        raise ValueError(f"ln_normalize_affine: part_stats must be contiguous fp32 [{nparts}, {rows}, 2]")
    _ln_params(x2d, gamma, beta, "ln_normalize_affine")
    y = torch.empty((rows, cols), dtype=x2d.dtype, device=x2d.device)
    mean = rstd = None
    if want_stats:
        mean = torch.empty((rows,), dtype=torch.float32, device=x2d.device)
        rstd = torch.empty((rows,), dtype=torch.float32, device=x2d.device)
    if part_cols_arr is None:
        part_cols_arr = _lib.i64_array(part_cols)
    rc = _lib.load().ddl_ln_normalize_affine(x2d.data_ptr(), dt, rows, cols, ld, part_stats.data_ptr(), nparts,
                                             part_cols_arr, _ptr(gamma), _ptr(beta), float(eps), y.data_ptr(), cols,
                                             _ptr(mean), _ptr(rstd), _stream())
    _lib.check(rc, "ddl_ln_normalize_affine")
    return (y, mean, rstd) if want_stats else y


def ln_joined_supported(x2d, nparts, gamma=None, beta=None):
    """Whether ``ln_stats_normalize`` takes these rows: at most 64 workers, rows
    of at most 16384 columns, columns and row pitch multiples of 4, x and the
    parameters aligned to four elements."""
    rows, cols = x2d.shape
    quad = 4 * x2d.element_size()
    return (nparts <= 64 and cols <= 16384 and cols % 4 == 0 and (rows <= 1 or x2d.stride(0) % 4 == 0) and
            x2d.data_ptr() % quad == 0 and
            (gamma is None or (gamma.data_ptr() % quad == 0 and beta.data_ptr() % quad == 0)))


def ln_stats_normalize(x2d, part_stats, my_part, part_cols, gamma, beta, eps, want_stats=False, part_cols_arr=None):
    """``ln_partial_stats`` into slot ``my_part`` of ``part_stats`` [P, rows, 2]
    and ``ln_normalize_affine`` on the completed table, in one launch and one
    read of x2d: for a worker whose peers' slots are filled before the call.
    Returns y (and mean, rstd), bit-equal to the two calls.  Rows the single
    launch does not take (see ``ln_joined_supported``) raise ``RuntimeError``."""
    _require_gpu(x2d, part_stats, gamma, beta)
    dt, ld = _ln_rows(x2d, "ln_stats_normalize")
    rows, cols = x2d.shape
    nparts = len(part_cols)
    if part_stats.dtype != torch.float32 or tuple(part_stats.shape) != (nparts, rows, 2) or \
       not part_stats.is_contiguous():
        raise ValueError(f"ln_stats_normalize: part_stats must be contiguous fp32 [{nparts}, {rows}, 2]")
    _ln_params(x2d, gamma, beta, "ln_stats_normalize")
    y = torch.empty((rows, cols), dtype=x2d.dtype, device=x2d.device)
    mean = rstd = None
    if want_stats:
        mean = torch.empty((rows,), dtype=torch.float32, device=x2d.device)
        rstd = torch.empty((rows,), dtype=torch.float32, device=x2d.device)
    if part_cols_arr is None:
        part_cols_arr = _lib.i64_array(part_cols)
    rc = _lib.load().ddl_ln_stats_normalize(x2d.data_ptr(), dt, rows, cols, ld, part_stats.data_ptr(), nparts, int(my_part),
                                            part_cols_arr, _ptr(gamma), _ptr(beta), float(eps), y.data_ptr(), cols,
                                            _ptr(mean), _ptr(rstd), _stream())
    _lib.check(rc, "ddl_ln_stats_normalize")
    return (y, mean, rstd) if want_stats else y


def layer_norm(x2d, gamma, beta, eps, want_stats=False):
    """Layer norm of rows held whole by this worker, one launch; returns y (and mean, rstd)."""
    _require_gpu(x2d, gamma, beta)
    dt, ld = _ln_rows(x2d, "layer_norm")
    rows, cols = x2d.shape
    _ln_params(x2d, gamma, beta, "layer_norm")
    y = torch.empty((rows, cols), dtype=x2d.dtype, device=x2d.device)
    mean = rstd = None
    if want_stats:
        mean = torch.empty((rows,), dtype=torch.float32, device=x2d.device)
        rstd = torch.empty((rows,), dtype=torch.float32, device=x2d.device)
    rc = _lib.load().ddl_layer_norm(x2d.data_ptr(), dt, rows, cols, ld, _ptr(gamma), _ptr(beta), float(eps),
                                    y.data_ptr(), cols, _ptr(mean), _ptr(rstd), _stream())
    _lib.check(rc, "ddl_layer_norm")
    return (y, mean, rstd) if want_stats else y


def _rows2d(t, name):
    if t.dtype not in _LN_DTYPES or t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise ValueError(f"{name}: need a 2-D float32, bfloat16 or float16 tensor with unit column stride")
    return t.stride(0) if t.shape[0] > 1 else t.shape[1]


def _ln_bwd_dtype(name, dy2d, x2d, gamma):
    """The element type of a LayerNorm backward call: dy, x and gamma must share it."""
    if dy2d.dtype != x2d.dtype or (gamma is not None and gamma.dtype != x2d.dtype):
        raise ValueError(f"{name}: dy, x and gamma must have one dtype")
    if dy2d.shape != x2d.shape:
        raise ValueError(f"{name}: dy {tuple(dy2d.shape)} and x {tuple(x2d.shape)} differ in shape")
    return _LN_DTYPES[x2d.dtype]


def ln_backward_partial(dy2d, x2d, mean, rstd, gamma):
    """Local {sum g, sum g xhat} per row, g = dy gamma: a [rows, 2] fp32 tensor."""
    _require_gpu(dy2d, x2d, mean, rstd, gamma)
    ld_dy, ld_x = _rows2d(dy2d, "ln_backward_partial"), _rows2d(x2d, "ln_backward_partial")
    dt = _ln_bwd_dtype("ln_backward_partial", dy2d, x2d, gamma)
    rows, cols = x2d.shape
    sums = torch.empty((rows, 2), dtype=torch.float32, device=x2d.device)
    rc = _lib.load().ddl_ln_bwd_partial(dy2d.data_ptr(), x2d.data_ptr(), dt, rows, cols, ld_dy, ld_x, mean.data_ptr(),
                                        rstd.data_ptr(), _ptr(gamma), sums.data_ptr(), _stream())
    _lib.check(rc, "ddl_ln_bwd_partial")
    return sums


def ln_backward_input(dy2d, x2d, mean, rstd, gamma, part_sums, weight):
    """dx from the gathered [P, rows, 2] sums; ``weight`` = 1 / (P * local columns)."""
    _require_gpu(dy2d, x2d, mean, rstd, gamma, part_sums)
    ld_dy, ld_x = _rows2d(dy2d, "ln_backward_input"), _rows2d(x2d, "ln_backward_input")
    rows, cols = x2d.shape
    if part_sums.dtype != torch.float32 or part_sums.dim() != 3 or tuple(part_sums.shape[1:]) != (rows, 2) or \
       not part_sums.is_contiguous():
        raise ValueError(f"ln_backward_input: part_sums must be contiguous fp32 [P, {rows}, 2]")
    dt = _ln_bwd_dtype("ln_backward_input", dy2d, x2d, gamma)
    dx = torch.empty((rows, cols), dtype=x2d.dtype, device=x2d.device)
    rc = _lib.load().ddl_ln_bwd_input(dy2d.data_ptr(), x2d.data_ptr(), dt, rows, cols, ld_dy, ld_x, mean.data_ptr(),
                                      rstd.data_ptr(), _ptr(gamma), part_sums.data_ptr(), part_sums.shape[0],
                                      float(weight), dx.data_ptr(), cols, _stream())
    _lib.check(rc, "ddl_ln_bwd_input")
    return dx


def ln_backward_params(dy2d, x2d, mean, rstd, want_gamma=True, want_beta=True):
    """(dgamma, dbeta) = column sums over the local rows of (dy xhat, dy)."""
    _require_gpu(dy2d, x2d, mean, rstd)
    ld_dy, ld_x = _rows2d(dy2d, "ln_backward_params"), _rows2d(x2d, "ln_backward_params")
    rows, cols = x2d.shape
    dt = _ln_bwd_dtype("ln_backward_params", dy2d, x2d, None)
    dg = torch.empty(cols, dtype=x2d.dtype, device=x2d.device) if want_gamma else None
    db = torch.empty(cols, dtype=x2d.dtype, device=x2d.device) if want_beta else None
    work = _ln_param_workspace(rows, cols, x2d.device)
    rc = _lib.load().ddl_ln_bwd_params(dy2d.data_ptr(), x2d.data_ptr(), dt, rows, cols, ld_dy, ld_x, mean.data_ptr(),
                                       rstd.data_ptr(), _ptr(dg), _ptr(db), work.data_ptr(), work.numel(), _stream())
    _lib.check(rc, "ddl_ln_bwd_params")
    return dg, db


def _ln_param_workspace(rows, cols, device):
    splits = max(1, min(256, (rows + 31) // 32))
    return torch.empty(2 * splits * cols, dtype=torch.float32, device=device)


def ln_backward_partial_params(dy2d, x2d, mean, rstd, gamma):
    """``ln_backward_partial`` plus, in the same pass, the partial column sums
    for the parameter gradients.  Returns (sums [rows, 2], workspace); hand the
    workspace to ``ln_backward_input_params``."""
    _require_gpu(dy2d, x2d, mean, rstd, gamma)
    ld_dy, ld_x = _rows2d(dy2d, "ln_backward_partial_params"), _rows2d(x2d, "ln_backward_partial_params")
    rows, cols = x2d.shape
    sums = torch.empty((rows, 2), dtype=torch.float32, device=x2d.device)
    work = _ln_param_workspace(rows, cols, x2d.device)
    dt = _ln_bwd_dtype("ln_backward_partial_params", dy2d, x2d, gamma)
    rc = _lib.load().ddl_ln_bwd_partial_params(dy2d.data_ptr(), x2d.data_ptr(), dt, rows, cols, ld_dy, ld_x,
                                               mean.data_ptr(), rstd.data_ptr(), _ptr(gamma), sums.data_ptr(),
                                               work.data_ptr(), work.numel(), _stream())
    _lib.check(rc, "ddl_ln_bwd_partial_params")
    return sums, work


def ln_backward_input_params(dy2d, x2d, mean, rstd, gamma, part_sums, weight, work, want_gamma=True, want_beta=True):
    """dx as ``ln_backward_input`` and, in the same launch, (dgamma, dbeta) from
    the workspace that ``ln_backward_partial_params`` filled."""
    _require_gpu(dy2d, x2d, mean, rstd, gamma, part_sums, work)
    ld_dy, ld_x = _rows2d(dy2d, "ln_backward_input_params"), _rows2d(x2d, "ln_backward_input_params")
    rows, cols = x2d.shape
    if part_sums.dtype != torch.float32 or part_sums.dim() != 3 or tuple(part_sums.shape[1:]) != (rows, 2) or \
       not part_sums.is_contiguous():
        raise ValueError(f"ln_backward_input_params: part_sums must be contiguous fp32 [P, {rows}, 2]")
    if work.dtype != torch.float32 or not work.is_contiguous():
        raise ValueError("ln_backward_input_params: the workspace must be a contiguous fp32 tensor")
    dt = _ln_bwd_dtype("ln_backward_input_params", dy2d, x2d, gamma)
    dx = torch.empty((rows, cols), dtype=x2d.dtype, device=x2d.device)
    dg = torch.empty(cols, dtype=x2d.dtype, device=x2d.device) if want_gamma else None
    db = torch.empty(cols, dtype=x2d.dtype, device=x2d.device) if want_beta else None
    rc = _lib.load().ddl_ln_bwd_input_params(dy2d.data_ptr(), x2d.data_ptr(), dt, rows, cols, ld_dy, ld_x, mean.data_ptr(),
                                             rstd.data_ptr(), _ptr(gamma), part_sums.data_ptr(), part_sums.shape[0],
                                             float(weight), dx.data_ptr(), cols, work.data_ptr(), work.numel(),
                                             _ptr(dg), _ptr(db), _stream())
    _lib.check(rc, "ddl_ln_bwd_input_params")
    return dx, dg, db


def ln_backward_one_pass_supported(dy2d, x2d, gamma, nparts=1):
    """Whether ``ln_backward_one_pass`` takes these rows: at most 64 workers,
    rows of at most 1024 columns, columns and pitches multiples of 4, dy, x and
    gamma aligned to four elements."""
    rows, cols = x2d.shape
    quad = 4 * x2d.element_size()
    return (nparts <= 64 and cols <= 1024 and cols % 4 == 0 and
            (rows <= 1 or (x2d.stride(0) % 4 == 0 and dy2d.stride(0) % 4 == 0)) and
            x2d.data_ptr() % quad == 0 and dy2d.data_ptr() % quad == 0 and (gamma is None or gamma.data_ptr() % quad == 0))


def ln_backward_one_pass(dy2d, x2d, mean, rstd, gamma, weight, part_sums=None, my_part=0, want_gamma=True, want_beta=True):
    """dx, (dgamma, dbeta) and this worker's row sums in one pass over dy and
    x: for rows this worker holds whole (``part_sums`` None) or whose other
    workers' sums are in ``part_sums`` [P, rows, 2] beforehand (slot ``my_part``
    is written).  Results as ``ln_backward_partial_params`` followed by
    ``ln_backward_input_params``."""
    _require_gpu(dy2d, x2d, mean, rstd, gamma, part_sums)
    ld_dy, ld_x = _rows2d(dy2d, "ln_backward_one_pass"), _rows2d(x2d, "ln_backward_one_pass")
    rows, cols = x2d.shape
    nparts = 1
    if part_sums is not None:
        if part_sums.dtype != torch.float32 or part_sums.dim() != 3 or tuple(part_sums.shape[1:]) != (rows, 2) or \
           not part_sums.is_contiguous():
            raise ValueError(f"ln_backward_one_pass: part_sums must be contiguous fp32 [P, {rows}, 2]")
        nparts = part_sums.shape[0]
    dt = _ln_bwd_dtype("ln_backward_one_pass", dy2d, x2d, gamma)
    work = _ln_param_workspace(rows, cols, x2d.device)
    dx = torch.empty((rows, cols), dtype=x2d.dtype, device=x2d.device)
    dg = torch.empty(cols, dtype=x2d.dtype, device=x2d.device) if want_gamma else None
    db = torch.empty(cols, dtype=x2d.dtype, device=x2d.device) if want_beta else None
    rc = _lib.load().ddl_ln_bwd_one_pass(dy2d.data_ptr(), x2d.data_ptr(), dt, rows, cols, ld_dy, ld_x, mean.data_ptr(),
                                         rstd.data_ptr(), _ptr(gamma), _ptr(part_sums), nparts, int(my_part), float(weight),
                                         dx.data_ptr(), cols, work.data_ptr(), work.numel(), _ptr(dg), _ptr(db), _stream())
    _lib.check(rc, "ddl_ln_bwd_one_pass")
    return dx, dg, db


def embedding_gather(weight, ids, lo, hi, out=None):
    """out[t] = weight[ids[t] - lo] if lo <= ids[t] < hi else 0."""
    _require_gpu(weight, ids)
    if weight.dim() != 2 or (weight.shape[1] > 1 and weight.stride(1) != 1):
        raise ValueError("embedding_gather: weight must be 2-D with unit column stride")
    if ids.dtype not in (torch.int64, torch.int32):
        raise ValueError("embedding_gather: ids must be int32 or int64")
    if weight.shape[0] != hi - lo:
        raise ValueError(f"embedding_gather: table has {weight.shape[0]} rows but the window is [{lo},{hi})")
    ids_c = contiguous(ids)
    dim = weight.shape[1]
    if out is None:
        out = torch.empty(tuple(ids.shape) + (dim,), dtype=weight.dtype, device=weight.device)
    elif not out.is_contiguous() or out.numel() != ids.numel() * dim or out.dtype != weight.dtype:
        raise ValueError("embedding_gather: bad output tensor")
    rc = _lib.load().ddl_embedding_gather(weight.data_ptr(), dim, weight.stride(0) if weight.shape[0] > 1 else dim,
                                          weight.element_size(), ids_c.data_ptr(),
                                          1 if ids.dtype == torch.int64 else 0, ids_c.numel(), int(lo), int(hi),
                                          out.data_ptr(), _stream())
    _lib.check(rc, "ddl_embedding_gather")
    return out


def embedding_renorm(weight, ids, lo, hi, max_norm, norm_type=2.0):
    """The ``max_norm`` step of ``F.embedding``: the rows of ``weight`` that
    ``ids`` name inside [lo, hi) and whose ``norm_type``-norm exceeds
    ``max_norm`` are scaled down to it, in place."""
    _require_gpu(weight, ids)
    if weight.dim() != 2 or (weight.shape[1] > 1 and weight.stride(1) != 1):
        raise ValueError("embedding_renorm: weight must be 2-D with unit column stride")
    if weight.dtype not in _LN_DTYPES:
        raise ValueError(f"embedding_renorm: tables are float32, bfloat16 or float16, got {weight.dtype}")
    if ids.dtype not in (torch.int64, torch.int32):
        raise ValueError("embedding_renorm: ids must be int32 or int64")
    if weight.shape[0] != hi - lo:
        raise ValueError(f"embedding_renorm: table has {weight.shape[0]} rows but the window is [{lo},{hi})")
    if weight.shape[0] == 0 or ids.numel() == 0:
        return weight
    ids_c = contiguous(ids)
    dim = weight.shape[1]
    flags = torch.empty(weight.shape[0], dtype=torch.int32, device=weight.device)
    rc = _lib.load().ddl_embedding_renorm(weight.data_ptr(), _LN_DTYPES[weight.dtype], dim,
                                          weight.stride(0) if weight.shape[0] > 1 else dim, ids_c.data_ptr(),
                                          1 if ids.dtype == torch.int64 else 0, ids_c.numel(), int(lo), int(hi),
                                          float(max_norm), float(norm_type), flags.data_ptr(), _stream())
    _lib.check(rc, "ddl_embedding_renorm")
    return weight


def embedding_backward(grad_output, ids, lo, hi, padding_idx=None, scale_grad_by_freq=False):
    """Gradient of :func:`embedding_gather` with respect to the ``[hi-lo, dim]``
    table; with ``scale_grad_by_freq`` every row's sum is divided by the number
    of tokens that looked the row up."""
    _require_gpu(grad_output, ids)
    if grad_output.dtype not in _LN_DTYPES:
        raise ValueError("embedding_backward: bfloat16, float16 or float32 gradients only")
    if ids.dtype not in (torch.int64, torch.int32):
        raise ValueError("embedding_backward: ids must be int32 or int64")
    dim = grad_output.shape[-1]
    if tuple(grad_output.shape[:-1]) != tuple(ids.shape):
        raise ValueError("embedding_backward: gradient and ids disagree in shape")
    dy = grad_output.reshape(-1, dim)
    if dim > 1 and dy.stride(1) != 1:
        dy = contiguous(dy)
    ids_c = contiguous(ids)
    rows, n_ids = int(hi) - int(lo), ids_c.numel()
    dw = torch.empty((rows, dim), dtype=grad_output.dtype, device=grad_output.device)
    work = torch.empty(3 * rows + 1 + n_ids, dtype=torch.int32, device=grad_output.device)
    dt = _LN_DTYPES[grad_output.dtype]
    rc = _lib.load().ddl_embedding_backward(dy.data_ptr(), dt, dim, dy.stride(0) if n_ids > 1 else dim, ids_c.data_ptr(),
                                            1 if ids.dtype == torch.int64 else 0, n_ids, int(lo), int(hi),
                                            -1 if padding_idx is None else int(padding_idx), 1 if scale_grad_by_freq else 0,
                                            dw.data_ptr(), dim, work.data_ptr(), work.numel(), _stream())
    _lib.check(rc, "ddl_embedding_backward")
    return dw


_LINEAR_DTYPES = {
    torch.bfloat16: _lib.DDL_DT_BF16,
    torch.float16: _lib.DDL_DT_F16,
    torch.float32: _lib.DDL_DT_F32,
}


def _padded_k(t, k8):
    """``t[rows, k]`` copied into a fresh ``[rows, k8]`` tensor whose extra columns are zero."""
    rows, k = t.shape
    out = torch.zeros((rows, k8), dtype=t.dtype, device=t.device)
    if rows > 0 and k > 0:
        full = [slice(0, rows), slice(0, k)]
        copy_box(t, full, out, full)
    return out


def linear(x, weight, bias=None, out=None):
    """y = x @ weight.T + bias with fp32 accumulation; operands and result
    bfloat16, float16 or float32 (all the same).  The 16-bit kernel wants the
    reduction length and the row pitches to be multiples of 8 and 16-byte
    aligned operands; operands that are not are copied into zero-padded
    temporaries first (zeros add nothing to the sums)."""
    _require_gpu(x, weight, bias)
    dt = _LINEAR_DTYPES.get(x.dtype)
    if dt is None or weight.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        raise ValueError("linear: operands must all be bfloat16, all float16 or all float32")
    if weight.dim() != 2 or x.shape[-1] != weight.shape[1]:
        raise ValueError(f"linear: x[..., {x.shape[-1]}] does not match weight {tuple(weight.shape)}")
    n, k = weight.shape
    x2 = x.reshape(-1, k)
    if x2.stride(1) != 1 and k > 1:
        x2 = contiguous(x2)
    if weight.stride(1) != 1 and k > 1:
        weight = contiguous(weight)
    if bias is not None and (bias.numel() != n or not bias.is_contiguous()):
        raise ValueError("linear: bias must be contiguous with out_features elements")
    m = x2.shape[0]
    if out is None:
        out = torch.empty(tuple(x.shape[:-1]) + (n,), dtype=x.dtype, device=x.device)
    elif not out.is_contiguous() or out.numel() != m * n or out.dtype != x.dtype:
        raise ValueError("linear: bad output tensor")
    if k == 0:
        # an empty sum: the bias alone (the kernels refuse K = 0)
        out.zero_()
        if bias is not None and m > 0:
            copy_box(bias.reshape(1, n).expand(m, n), [slice(0, m), slice(0, n)], out.view(m, n), [slice(0, m), slice(0, n)])
        return out
    if dt != _lib.DDL_DT_F32:
        def fits(t, rows):
            return k % 8 == 0 and t.data_ptr() % 16 == 0 and (rows <= 1 or t.stride(0) % 8 == 0)
        if not (fits(x2, m) and fits(weight, n)):
            k8 = _round_up(k, 8)
            x2, weight, k = _padded_k(x2, k8), _padded_k(weight, k8), k8
    rc = _lib.load().ddl_linear(x2.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(), dt, m, n, k,
                                x2.stride(0) if m > 1 else k, weight.stride(0) if n > 1 else k, n, _stream())
    _lib.check(rc, "ddl_linear")
    return out


def linear_bf16(x, weight, bias=None, out=None):
    """:func:`linear` restricted to bfloat16 operands."""
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or (bias is not None and bias.dtype != torch.bfloat16):
        raise ValueError("linear_bf16: operands must be bfloat16")
    return linear(x, weight, bias, out)


def _round_up(n, m):
    return (n + m - 1) // m * m


def transpose_2d(src, ld_dst=None):
    """``src[rows, cols]`` (16-bit elements, row stride arbitrary) -> a new
    ``[cols, ld_dst]`` tensor whose first ``rows`` columns hold the transpose;
    any further columns are zero."""
    _require_gpu(src)
    if src.dim() != 2 or src.element_size() != 2:
        raise ValueError("transpose_2d: a 2-D tensor of 16-bit elements is required")
    if src.stride(1) != 1 and src.shape[1] > 1:
        src = contiguous(src)
    rows, cols = src.shape
    ld_dst = rows if ld_dst is None else ld_dst
    alloc = torch.empty if ld_dst == rows else torch.zeros
    dst = alloc((cols, ld_dst), dtype=src.dtype, device=src.device)
    rc = _lib.load().ddl_transpose_2d(src.data_ptr(), dst.data_ptr(), rows, cols, src.stride(0) if rows > 1 else cols,
                                      ld_dst, 2, _stream())
    _lib.check(rc, "ddl_transpose_2d")
    return dst


def colsum(a):
    """Column sums of a 2-D bfloat16 / float16 / float32 tensor, fp32 accumulation, result in the tensor's type."""
    _require_gpu(a)
    dt = _LINEAR_DTYPES.get(a.dtype)
    if a.dim() != 2 or dt is None:
        raise ValueError("colsum: a 2-D bfloat16, float16 or float32 tensor is required")
    if a.stride(1) != 1 and a.shape[1] > 1:
        a = contiguous(a)
    rows, cols = a.shape
    out = torch.empty(cols, dtype=a.dtype, device=a.device)
    splits = max(1, min(64, (rows + 127) // 128))
    work = torch.empty(splits * max(cols, 1), dtype=torch.float32, device=a.device)
    rc = _lib.load().ddl_colsum(a.data_ptr(), dt, rows, cols, a.stride(0) if rows > 1 else cols, out.data_ptr(),
                                work.data_ptr(), work.numel(), _stream())
    _lib.check(rc, "ddl_colsum")
    return out


def colsum_bf16(a):
    """:func:`colsum` restricted to bfloat16."""
    if a.dim() != 2 or a.dtype != torch.bfloat16:
        raise ValueError("colsum_bf16: a 2-D bfloat16 tensor is required")
    return colsum(a)


def linear_backward(x, weight, grad_output, need_input=True, need_weight=True, need_bias=True):
    """Adjoint of :func:`linear`: ``(dx, dw, db)`` for ``y = x @ weight.T + bias``
    (entries not asked for are None).  Both products read their operands where
    they lie: the float32 one through strides, the 16-bit one through
    transposing LDS reads, which need row counts and pitches that are multiples
    of 8; 16-bit operands that do not qualify are transposed into temporaries
    whose row pitch is padded to a multiple of 8 with zeros, and the forward
    kernel runs on those."""
    _require_gpu(x, weight, grad_output)
    dt = _LINEAR_DTYPES.get(x.dtype)
    if dt is None or weight.dtype != x.dtype or grad_output.dtype != x.dtype:
        raise ValueError("linear_backward: operands must all be bfloat16, all float16 or all float32")
    n, k = weight.shape
    x2 = x.reshape(-1, k)
    dy = grad_output.reshape(-1, n)
    if dy.stride(1) != 1 and n > 1:
        dy = contiguous(dy)
    m = x2.shape[0]
    dx = dw = db = None
    if dt == _lib.DDL_DT_F32:
        if x2.stride(1) != 1 and k > 1:
            x2 = contiguous(x2)
        if weight.stride(1) != 1 and k > 1:
            weight = contiguous(weight)
        lib = _lib.load()
        ld_dy, ld_x, ld_w = (dy.stride(0) if m > 1 else n), (x2.stride(0) if m > 1 else k), (weight.stride(0) if n > 1 else k)
        if need_input:
            dx = torch.empty((m, k), dtype=x.dtype, device=x.device)
            if n == 0:
                dx.zero_()
            else:   # dx[m, j] = sum_n dy[m, n] w[n, j]: rows of the second operand are the columns of w
                rc = lib.ddl_gemm_f32(dy.data_ptr(), ld_dy, 1, weight.data_ptr(), 1, ld_w, None, dx.data_ptr(), k, m, k, n,
                                      _stream())
                _lib.check(rc, "ddl_gemm_f32")
            dx = dx.reshape(x.shape)
        if need_weight:
            dw = torch.empty((n, k), dtype=x.dtype, device=x.device)
            if m == 0:
                dw.zero_()
            else:   # dw[i, j] = sum_m dy[m, i] x[m, j]: both operands are read down their columns
                rc = lib.ddl_gemm_f32(dy.data_ptr(), 1, ld_dy, x2.data_ptr(), 1, ld_x, None, dw.data_ptr(), k, n, k, m,
                                      _stream())
                _lib.check(rc, "ddl_gemm_f32")
        if need_bias:
            db = colsum(dy)
        return dx, dw, db
    if x2.stride(1) != 1 and k > 1:
        x2 = contiguous(x2)
    if weight.stride(1) != 1 and k > 1:
        weight = contiguous(weight)
    ld_dy, ld_x, ld_w = (dy.stride(0) if m > 1 else n), (x2.stride(0) if m > 1 else k), (weight.stride(0) if n > 1 else k)
    if need_input:
        # dx[m, j] = sum_n dy[m, n] w[n, j]: dy is read along n, w down its columns
        if m and n and k and _along_k_ok(dy, ld_dy, n) and _along_rows_ok(weight, ld_w, k, n):
            dx = torch.empty((m, k), dtype=x.dtype, device=x.device)
            rc = _lib.load().ddl_gemm(dy.data_ptr(), ld_dy, 1, weight.data_ptr(), 1, ld_w, None, dx.data_ptr(), dt, k, m, k, n,
                                      _stream())
            _lib.check(rc, "ddl_gemm")
            dx = dx.reshape(x.shape)
        else:   # operands dy[M, N] and wT[K, N], padded
            np8 = _round_up(n, 8)
            w_t = transpose_2d(weight, np8)                       # [K, np8], padding columns zero
            dy_p = dy
            if np8 != n or (m > 1 and dy.stride(0) % 8 != 0) or dy.data_ptr() % 16 != 0:
                dy_p = _padded_k(dy, np8)
            dx = _linear_padded(dy_p, w_t, m, k, np8, dt).reshape(x.shape)
    if need_weight:
        # dw[i, j] = sum_m dy[m, i] x[m, j]: both operands are read down their columns
        if m and n and k and _along_rows_ok(dy, ld_dy, n, m) and _along_rows_ok(x2, ld_x, k, m):
            dw = torch.empty((n, k), dtype=x.dtype, device=x.device)
            rc = _lib.load().ddl_gemm(dy.data_ptr(), 1, ld_dy, x2.data_ptr(), 1, ld_x, None, dw.data_ptr(), dt, k, n, k, m,
                                      _stream())
            _lib.check(rc, "ddl_gemm")
        else:   # operands dyT[N, M] and xT[K, M], padded
            mp8 = _round_up(m, 8)
            dy_t = transpose_2d(dy, mp8)                          # [N, mp8]
            x_t = transpose_2d(x2, mp8)                           # [K, mp8]
            dw = _linear_padded(dy_t, x_t, n, k, mp8, dt)
    if need_bias:
        db = colsum(dy)
    return dx, dw, db


def _along_k_ok(t, pitch, depth):
    """Can the 16-bit product read ``t`` (rows contiguous along the reduction
    dimension of length ``depth``) where it lies?"""
    return depth % 8 == 0 and pitch % 8 == 0 and pitch <= 0x3FFFFF and t.data_ptr() % 16 == 0


def _along_rows_ok(t, pitch, rows, depth):
    """Can the 16-bit product read ``t`` down its columns (``rows`` of them, each
    of length ``depth`` along the reduction dimension) where it lies?"""
    return (rows % 8 == 0 and pitch % 8 == 0 and pitch <= 0x3FFFFF and t.data_ptr() % 16 == 0
            and (depth + 64) * pitch <= 0x3FFFFFFF)


def linear_bf16_backward(x, weight, grad_output, need_input=True, need_weight=True, need_bias=True):
    """:func:`linear_backward`; kept under the name of the first, bfloat16-only version."""
    return linear_backward(x, weight, grad_output, need_input, need_weight, need_bias)


def _linear_padded(a, b, m, n, k_padded, dt):
    """``a[m, k_padded] @ b[n, k_padded].T`` where the padding columns are zero."""
    out = torch.empty((m, n), dtype=a.dtype, device=a.device)
    if k_padded == 0 or m == 0 or n == 0:
        return out.zero_()
    rc = _lib.load().ddl_linear(a.data_ptr(), b.data_ptr(), None, out.data_ptr(), dt, m, n, k_padded,
                                a.stride(0) if m > 1 else k_padded, b.stride(0) if n > 1 else k_padded, n, _stream())
    _lib.check(rc, "ddl_linear")
    return out
