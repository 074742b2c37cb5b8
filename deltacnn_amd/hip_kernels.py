"""Functional wrappers over libdeltacnn_hip.so with the names, argument order and defaults
of the reference's ``src/deltacnn/cuda_kernels.py``: shape arithmetic, output allocation
(NHWC / ``torch.channels_last`` features, int32 ``[B,1,H,W]`` masks) and the C-ABI call on
torch's current stream.  Tensors are borrowed for the asynchronous launch; nothing
synchronises.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from . import _lib
from ._lib import DC_BF16, DC_F16, DC_F32, Geometry

_DTYPES = {torch.float32: DC_F32, torch.float16: DC_F16, torch.bfloat16: DC_BF16}

# Optional per-call tracer (see deltacnn_amd/trace.py): when set, every library call goes
# through ``tracer.run(op, fn, args, meta)`` which brackets it with events and records the
# shapes and mask populations that the algorithmic byte counts are computed from.
_TRACER = None


def set_tracer(tracer) -> None:
    global _TRACER
    _TRACER = tracer


def _call(op, fn, args, **meta):
    if _TRACER is None:
        _lib.check(fn(*args))
    else:
        _lib.check(_TRACER.run(op, fn, args, meta))


def _dtype(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise _lib.DeltaCNNError(-1, f"unsupported dtype {t.dtype} (float32, float16 and bfloat16 only)")


def _nhwc(t: torch.Tensor, name: str) -> torch.Tensor:
    """The kernels index features as [B][H][W][C]; refuse anything else instead of guessing."""
    if t.dim() != 4 or not t.is_contiguous(memory_format=torch.channels_last):
        raise _lib.DeltaCNNError(-2, f"{name} must be a 4-d channels_last tensor, got shape "
                                     f"{tuple(t.shape)} strides {t.stride()}")
    if not t.is_cuda:
        raise _lib.DeltaCNNError(-4, f"{name} must live on the GPU")
    return t


def _mask(m: torch.Tensor, name: str) -> torch.Tensor:
    if m.dtype != torch.int32 or not m.is_cuda or not (m.is_contiguous() or m.is_contiguous(
            memory_format=torch.channels_last)):
        raise _lib.DeltaCNNError(-2, f"{name} must be a dense int32 GPU tensor")
    return m


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _pixels(t: torch.Tensor) -> int:
    return t.shape[0] * t.shape[2] * t.shape[3]


def _pad4(padding: Sequence[int]):
    """(top, bottom, left, right), cuda_kernels.py:21-26."""
    if len(padding) == 2:
        return padding[0], padding[0], padding[1], padding[1]
    if len(padding) == 4:
        return tuple(padding)
    raise ValueError("Padding must be iterable of size 2 or 4")


def new_features(b, c, h, w, dtype, device) -> torch.Tensor:
    return torch.empty((b, c, h, w), dtype=dtype, device=device, memory_format=torch.channels_last)


def new_mask(b, h, w, device) -> torch.Tensor:
    return torch.empty((b, 1, h, w), dtype=torch.int32, device=device)


def conv_geometry(x_shape, kernel, c_out, stride, padding, dilation, groups, transposed=False,
                  out_hw=None) -> Geometry:
    b, c_in, h, w = x_shape
    t, bt, l, r = _pad4(padding)
    if out_hw is None:
        if transposed:
            oh = (h - 1) * stride[0] - 2 * t + dilation[0] * (kernel[0] - 1) + 1
            ow = (w - 1) * stride[1] - 2 * l + dilation[1] * (kernel[1] - 1) + 1
        else:
            oh = (h + t + bt - dilation[0] * (kernel[0] - 1) - 1) // stride[0] + 1
            ow = (w + l + r - dilation[1] * (kernel[1] - 1) - 1) // stride[1] + 1
    else:
        oh, ow = out_hw
    return Geometry(b, h, w, c_in, oh, ow, c_out, kernel[0], kernel[1], stride[0], stride[1],
                    dilation[0], dilation[1], t, l, bt, r, groups)


def _conv_like(transposed, x, filter, mask, bias, stride, padding, dilation, groups, c_out,
               create_out_mask, out_mask, out_shape, packed_filter, out, geometry, epilogue=None):
    lib = _lib.load()
    _nhwc(x, "x")
    if mask is None:
        raise _lib.DeltaCNNError(-4, "the delta kernels need an update mask (mask=None is the "
                                     "dense path of the reference and is not part of this library)")
    _mask(mask, "mask")
    out_c = filter.shape[3] if c_out is None else c_out
    g = geometry
    if g is None:
        hw = tuple(out_shape) if out_shape is not None and len(out_shape) == 2 else None
        g = conv_geometry(x.shape, (filter.shape[1], filter.shape[2]), out_c, stride, padding,
                          dilation, groups, transposed, hw)
        if isinstance(out_shape, list) and len(out_shape) == 0:
            out_shape.extend([g.out_h, g.out_w])
    if out is None:
        out = new_features(g.batch, out_c, g.out_h, g.out_w, x.dtype, x.device)
    if out_mask is None:
        out_mask = new_mask(g.batch, g.out_h, g.out_w, x.device)
    dt = _dtype(x)
    # `keep`: the tracer replays recorded calls later; buffers allocated here must outlive them
    meta = dict(g=g, esize=x.element_size(), in_mask=mask, out_mask=out_mask,
                mfma=packed_filter is not None, keep=(x, filter, packed_filter, bias, out))
    if epilogue is not None:
        prev, trunc, thr, act, mode = epilogue
        _call("conv_act", lib.dc_conv_act,
              (g, x.data_ptr(), filter.data_ptr(), _ptr(packed_filter), _ptr(bias), out.data_ptr(),
               mask.data_ptr(), out_mask.data_ptr(), prev.data_ptr(), _ptr(trunc), thr, act, mode,
               dt, _stream()), **meta)
    else:
        _call("deconv" if transposed else "conv", lib.dc_deconv if transposed else lib.dc_conv,
              (g, x.data_ptr(), filter.data_ptr(), _ptr(packed_filter), _ptr(bias), out.data_ptr(),
               mask.data_ptr(), out_mask.data_ptr(), dt, _stream()), **meta)
    if create_out_mask:
        return out, out_mask
    return out


def sparse_conv(x, filter, mask=None, bias=None, stride=(1, 1), padding=(0, 0), dilation=(1, 1),
                groups=1, c_out: int = None, create_out_mask=False, sub_tile_sparsity=True,
                out_mask=None, out_shape=None, *, packed_filter=None, out=None, geometry=None):
    """cuda_kernels.py:13-45.  ``filter`` is in the layout of ``process_filters()``.

    Keyword-only extras: ``packed_filter`` (from :func:`pack_filter`) selects the MFMA
    kernels, ``out`` / ``geometry`` let a layer reuse its buffers.
    """
    return _conv_like(False, x, filter, mask, bias, stride, padding, dilation, groups, c_out,
                      create_out_mask, out_mask, out_shape, packed_filter, out, geometry)


def sparse_conv_activation(x, filter, mask, bias, prev_out, truncated, threshold, activation,
                           truncation_mode, stride=(1, 1), padding=(0, 0), dilation=(1, 1),
                           groups=1, c_out=None, *, packed_filter=None, out=None, out_mask=None,
                           geometry=None):
    """``sparse_conv`` followed by ``sparse_activation`` on its output in one library call."""
    return _conv_like(False, x, filter, mask, bias, stride, padding, dilation, groups, c_out, True,
                      out_mask, None, packed_filter, out, geometry,
                      (prev_out, truncated, float(threshold), int(activation), int(truncation_mode)))


def sparse_conv_add(x, packed_filter, mask, bias, residual, mask_residual, geometry, out, out_mask,
                    weight_residual=1.0, weight_conv=1.0, prev_out=None, activation=0):
    """``sparse_add_tensors(residual, sparse_conv(x), prev_out, ..., activation)`` in the
    convolution's launch, for fp16 convolutions with a packed filter: pointwise ones (without
    activation) and small layers of any kernel size.  Returns ``None`` (nothing launched) when
    the shape has no fused form, so the caller can issue the two separate calls."""
    lib = _lib.load()
    _nhwc(x, "x")
    _nhwc(residual, "residual")
    if packed_filter is None or x.dtype not in (torch.float16, torch.bfloat16):
        return None
    activation = max(int(activation), 0)
    args = (geometry, x.data_ptr(), packed_filter.data_ptr(), _ptr(bias), _mask(mask, "mask").data_ptr(),
            residual.data_ptr(), _mask(mask_residual, "mask_residual").data_ptr(), out.data_ptr(),
            out_mask.data_ptr(), float(weight_residual), float(weight_conv), _ptr(prev_out), activation,
            _dtype(x), _stream())
    meta = dict(g=geometry, esize=2, in_mask=mask, in_mask_b=mask_residual, out_mask=out_mask, mfma=True)
    try:
        _call("conv_add", lib.dc_conv_add, args, **meta)
    except _lib.DeltaCNNError as e:
        if e.code == -3:
            return None
        raise
    return out, out_mask


def sparse_deconv_add(x, packed_filter, mask, residual, mask_residual, geometry, out, out_mask,
                      weight_residual=1.0, weight_conv=1.0):
    """``sparse_add_tensors(residual, sparse_deconv(x))`` (no activation) in the transposed
    convolution's launch (``dc_deconv_add``), for 16-bit layers with a packed filter that the
    LDS-halo kernel takes.  Returns ``None`` (nothing launched) when the shape has no fused form,
    so the caller can issue the two separate calls."""
    lib = _lib.load()
    _nhwc(x, "x")
    _nhwc(residual, "residual")
    if packed_filter is None or x.dtype not in (torch.float16, torch.bfloat16):
        return None
    args = (geometry, x.data_ptr(), packed_filter.data_ptr(), _mask(mask, "mask").data_ptr(), residual.data_ptr(),
            _mask(mask_residual, "mask_residual").data_ptr(), out.data_ptr(), out_mask.data_ptr(),
            float(weight_residual), float(weight_conv), _dtype(x), _stream())
    meta = dict(g=geometry, esize=2, in_mask=mask, in_mask_b=mask_residual, out_mask=out_mask, mfma=True)
    try:
        _call("deconv_add", lib.dc_deconv_add, args, **meta)
    except _lib.DeltaCNNError as e:
        if e.code == -3:
            return None
        raise
    return out, out_mask


def sparse_block(x, mask, dw_filter, dw_geometry, dw_prev_out, dw_truncated, dw_threshold, dw_activation,
                 project_packed, project_channels, out, out_mask, residual=None, residual_mask=None,
                 weight_residual=1.0, weight_conv=1.0, expand=None, truncation_mode=0, late_loads=False):
    """Depthwise 3x3 convolution + activation/truncation, 1x1 projection (+ residual sum) and,
    with ``expand = (packed_filter, channels, prev_out, truncated, threshold, activation, out,
    out_mask)``, the following 1x1 expansion + activation/truncation, in ONE launch (``dc_block``).
    Identical to the separate calls bit for bit; the depthwise output is never stored.  Returns
    ``False`` (nothing launched) for shapes the kernel does not take, so the caller can issue the
    separate calls.  ``late_loads``: fetch operands only once the masks are known (for large,
    mostly inactive maps; the default requests everything up front where the filters are small)."""
    lib = _lib.load()
    _nhwc(x, "x")
    if x.dtype != torch.float16 or project_packed is None:
        return False
    a = _lib.BlockArgs()
    a.flags = 1 if late_loads else 0
    a.input, a.mask, a.dw_filter = x.data_ptr(), _mask(mask, "mask").data_ptr(), dw_filter.data_ptr()
    a.dw_prev_out, a.dw_truncated = dw_prev_out.data_ptr(), dw_truncated.data_ptr()
    a.dw_threshold, a.dw_activation, a.dw_truncation_mode = float(dw_threshold), int(dw_activation), int(truncation_mode)
    a.project_packed_filter, a.project_channels = project_packed.data_ptr(), int(project_channels)
    a.residual, a.residual_mask = _ptr(residual), _ptr(residual_mask)
    a.weight_residual, a.weight_conv = float(weight_residual), float(weight_conv)
    a.out, a.out_mask = out.data_ptr(), out_mask.data_ptr()
    ex_mask, ce = None, 0
    if expand is not None:
        packed, ce, prev, trunc, thr, act, eout, ex_mask = expand
        if packed is None:
            return False
        a.expand_packed_filter, a.expand_channels = packed.data_ptr(), int(ce)
        a.expand_prev_out, a.expand_truncated = prev.data_ptr(), trunc.data_ptr()
        a.expand_threshold, a.expand_activation, a.expand_truncation_mode = float(thr), int(act), int(truncation_mode)
        a.expand_out, a.expand_out_mask = eout.data_ptr(), ex_mask.data_ptr()
    meta = dict(g=dw_geometry, esize=2, in_mask=mask, in_mask_b=residual_mask, out_mask=out_mask, ex_mask=ex_mask,
                Cp=int(project_channels), Ce=int(ce), keep=(a, x, dw_filter, project_packed, residual, expand))
    try:
        _call("block", lib.dc_block, (dw_geometry, ctypes.byref(a), DC_F16, _stream()), **meta)
    except _lib.DeltaCNNError as e:
        if e.code == -3:
            return False
        raise
    return True


def sparse_expand_depthwise(x, mask, expand_packed, expand_prev_out, expand_truncated, expand_threshold,
                            expand_activation, expand_out, expand_out_mask, dw_filter, dw_geometry, dw_prev_out,
                            dw_truncated, dw_threshold, dw_activation, dw_truncation_mode, out, out_mask,
                            opened: bool = False):
    """A 1x1 expansion with activation / maximum-norm truncation followed by a depthwise 3x3
    (stride 1 or 2, padding 1) with activation / truncation as TWO launches instead of three
    (``dc_expand_depthwise``): the expansion leaves its keep decision to the depthwise kernel,
    which reads whole pixel rows anyway and commits the expansion's cached state.  Layer states
    and the depthwise output are identical, bit for bit, to the separate calls.  Returns ``False``
    (nothing launched) for shapes without this form, so the caller can issue the separate calls.

    ``opened``: :func:`sparse_project_expand` has already run the expansion's convolution into
    ``expand_out`` / ``expand_truncated`` / ``expand_out_mask``; only the depthwise launch runs
    (``x`` is then the expansion's INPUT shape donor only and ``mask``, ``expand_packed`` are unused)."""
    lib = _lib.load()
    _nhwc(x, "x")
    if x.dtype not in (torch.float16, torch.bfloat16) or (expand_packed is None and not opened):
        return False
    a = _lib.ExpandDwArgs()
    if opened:
        a.input, a.mask, a.expand_packed_filter = None, None, None
        mask = expand_out_mask
    else:
        a.input, a.mask, a.expand_packed_filter = x.data_ptr(), _mask(mask, "mask").data_ptr(), expand_packed.data_ptr()
    a.expand_in_channels = int(x.shape[1])
    a.expand_prev_out, a.expand_truncated = expand_prev_out.data_ptr(), expand_truncated.data_ptr()
    a.expand_threshold, a.expand_activation, a.expand_truncation_mode = float(expand_threshold), int(expand_activation), 0
    a.expand_out, a.expand_out_mask = expand_out.data_ptr(), expand_out_mask.data_ptr()
    a.dw_filter, a.dw_prev_out, a.dw_truncated = dw_filter.data_ptr(), dw_prev_out.data_ptr(), dw_truncated.data_ptr()
    a.dw_threshold, a.dw_activation, a.dw_truncation_mode = float(dw_threshold), int(dw_activation), int(dw_truncation_mode)
    a.out, a.out_mask = out.data_ptr(), out_mask.data_ptr()
    meta = dict(g=dw_geometry, esize=x.element_size(), in_mask=mask, out_mask=out_mask, Ci=int(x.shape[1]),
                opened=opened, keep=(a, x, expand_packed, dw_filter))
    try:
        _call("expand_dw", lib.dc_expand_depthwise, (dw_geometry, ctypes.byref(a), _dtype(x), _stream()), **meta)
    except _lib.DeltaCNNError as e:
        if e.code == -3:
            return False
        raise
    return True


def sparse_project_expand(x, mask, project_packed, project_geometry, residual, residual_mask, out, out_mask,
                          expand_packed, expand_prev_out, expand_truncated, expand_activation, expand_out,
                          expand_out_mask, dw_geometry, dw_activation, dw_truncation_mode,
                          weight_residual: float = 1.0, weight_conv: float = 1.0):
    """The 1x1 projection that ends an inverted-residual block (+ the block's residual sum) and the
    next block's 1x1 expansion in ONE launch (``dc_project_expand``).  The expansion's activation is
    left open: the next call on its buffers has to be :func:`sparse_expand_depthwise` with
    ``opened=True``, which this call has verified to be accepted for ``dw_geometry``.  Together
    the two are identical, bit for bit, to the separate layer calls.  Returns ``False`` (nothing
    launched) for shapes without this form."""
    lib = _lib.load()
    _nhwc(x, "x")
    if x.dtype not in (torch.float16, torch.bfloat16) or project_packed is None or expand_packed is None:
        return False
    a = _lib.ProjectExpandArgs()
    a.input, a.mask, a.project_packed_filter = x.data_ptr(), _mask(mask, "mask").data_ptr(), project_packed.data_ptr()
    if residual is not None:
        a.residual, a.residual_mask = _nhwc(residual, "residual").data_ptr(), _mask(residual_mask, "residual_mask").data_ptr()
    a.weight_residual, a.weight_conv = float(weight_residual), float(weight_conv)
    a.out, a.out_mask = out.data_ptr(), out_mask.data_ptr()
    a.expand_packed_filter, a.expand_channels = expand_packed.data_ptr(), int(expand_out.shape[1])
    a.expand_prev_out, a.expand_truncated = expand_prev_out.data_ptr(), expand_truncated.data_ptr()
    a.expand_activation = int(expand_activation)
    a.expand_out, a.expand_out_mask = expand_out.data_ptr(), expand_out_mask.data_ptr()
    a.dw_geometry = ctypes.pointer(dw_geometry)
    a.dw_activation, a.dw_truncation_mode = int(dw_activation), int(dw_truncation_mode)
    meta = dict(g=project_geometry, esize=x.element_size(), in_mask=mask, in_mask_b=residual_mask, out_mask=out_mask,
                Ce=int(expand_out.shape[1]), keep=(a, x, project_packed, expand_packed, residual, dw_geometry))
    try:
        _call("project_expand", lib.dc_project_expand, (project_geometry, ctypes.byref(a), _dtype(x), _stream()), **meta)
    except _lib.DeltaCNNError as e:
        if e.code == -3:
            return False
        raise
    return True


def sparse_conv_group(items) -> bool:
    """Independent small 3x3 layers in ONE launch (``dc_conv_group``), plus one for the
    activations that their convolutions cannot finish themselves; or independent plain 1x1
    convolutions in one launch.  ``items``: 2 .. 8 dicts with
    ``x, mask, packed_filter, geometry, out, out_mask`` (and optionally ``bias``) and at most one of
    ``residual = (values, mask, weight_residual, weight_conv, prev_out or None, activation)`` --
    the operands of :func:`sparse_conv_add` -- and ``activation = (prev_out, truncated, threshold,
    activation, truncation_mode)`` -- those of :func:`sparse_conv_activation`.  Every item's
    results are identical, bit for bit, to the separate call's.  Returns ``False`` (nothing
    launched) when the group has no such form."""
    lib = _lib.load()
    n = len(items)
    if n < 2 or n > _lib.CONV_GROUP_MAX:
        return False
    dtype = items[0]["x"].dtype
    if dtype not in (torch.float16, torch.bfloat16):
        return False
    arr = (_lib.ConvItem * n)()
    metas, keep = [], []
    for a, it in zip(arr, items):
        x, packed = _nhwc(it["x"], "x"), it["packed_filter"]
        if packed is None or x.dtype != dtype:
            return False
        a.geometry = it["geometry"]
        a.input, a.mask, a.packed_filter = x.data_ptr(), _mask(it["mask"], "mask").data_ptr(), packed.data_ptr()
        a.bias = _ptr(it.get("bias"))
        a.out, a.out_mask = it["out"].data_ptr(), it["out_mask"].data_ptr()
        meta = dict(g=it["geometry"], in_mask=it["mask"], in_mask_b=None, out_mask=it["out_mask"], kind="conv")
        res, act = it.get("residual"), it.get("activation")
        if res is not None:
            values, rmask, wa, wb, prev, activation = res
            a.residual, a.residual_mask = _nhwc(values, "residual").data_ptr(), _mask(rmask, "residual mask").data_ptr()
            a.weight_residual, a.weight_conv = float(wa), float(wb)
            a.sum_prev_out, a.sum_activation = _ptr(prev), max(int(activation), 0)
            meta.update(kind="conv_add", in_mask_b=rmask)
            keep.append((values, prev))
        elif act is not None:
            prev, truncated, threshold, activation, mode = act
            a.prev_out, a.truncated = prev.data_ptr(), _ptr(truncated)
            a.threshold, a.activation, a.truncation_mode = float(threshold), int(activation), int(mode)
            meta.update(kind="conv_act")
            keep.append((prev, truncated))
        metas.append(meta)
        keep.append((x, packed, it.get("bias")))
    try:
        _call("conv_group", lib.dc_conv_group, (arr, n, _DTYPES[dtype], _stream()), items=metas,
              esize=items[0]["x"].element_size(), keep=(arr, keep))
    except _lib.DeltaCNNError as e:
        if e.code == -3:
            return False
        raise
    return True


def sparse_deconv(x, filter, mask=None, bias=None, stride=(1, 1), padding=(0, 0), dilation=(1, 1),
                  groups=1, c_out: int = None, create_out_mask=False, sub_tile_sparsity=True,
                  out_mask=None, out_shape=None, *, packed_filter=None, out=None, geometry=None):
    """cuda_kernels.py:47-78."""
    if len(padding) != 2:
        raise ValueError("Padding must be iterable of size 2")
    return _conv_like(True, x, filter, mask, bias, stride, padding, dilation, groups, c_out,
                      create_out_mask, out_mask, out_shape, packed_filter, out, geometry)


def pack_filter(filter: torch.Tensor, c_in: int, c_out: int, groups: int = 1,
                transposed: bool = False) -> Optional[torch.Tensor]:
    """One-time relayout of a processed fp16 filter, or of a bfloat16 filter in the fp32 layout,
    for the MFMA kernels; None if the shape has no packed form (fp32, grouped, or an input
    channel count that is neither a multiple of 8 nor a stem's: Cin <= 4 with a window up to
    8 x 8 and Cout <= 64)."""
    lib = _lib.load()
    if filter.dtype not in (torch.float16, torch.bfloat16):
        return None
    dt = _dtype(filter)
    g = Geometry(1, 1, 1, c_in, 1, 1, c_out, filter.shape[1], filter.shape[2], 1, 1, 1, 1, 0, 0, 0,
                 0, groups)
    nbytes = lib.dc_packed_filter_bytes(g, dt, int(transposed))
    if nbytes == 0:
        return None
    packed = torch.empty(nbytes // 2, dtype=filter.dtype, device=filter.device)
    _lib.check(lib.dc_pack_filter(g, filter.data_ptr(), packed.data_ptr(), dt, int(transposed), _stream()))
    return packed


def sparse_pooling(x, prev_x, kernel_size, mask=None, stride=(1, 1), padding=(0, 0),
                   dilation=(1, 1), create_out_mask=True, sub_tile_sparsity=True, out_mask=None,
                   pooling_mode_int=0, out_shape=None, *, out=None):
    """cuda_kernels.py:80-129.  The reference accumulates a 1x1 output in a float32 buffer and
    casts it back afterwards (:101-124); here the kernel writes the input dtype directly when
    the window is the whole unpadded map, and falls back to that protocol otherwise."""
    lib = _lib.load()
    _nhwc(x, "x")
    if mask is None:
        raise _lib.DeltaCNNError(-4, "sparse_pooling needs an update mask")
    hw = tuple(out_shape) if out_shape is not None and len(out_shape) == 2 else None
    g = conv_geometry(x.shape, kernel_size, x.shape[1], stride, padding, dilation, 1, False, hw)
    if isinstance(out_shape, list) and len(out_shape) == 0:
        out_shape.extend([g.out_h, g.out_w])
    is_global = g.out_h == 1 and g.out_w == 1
    vec = 16 // x.element_size()
    direct = (is_global and g.kernel_h == g.in_h and g.kernel_w == g.in_w and tuple(_pad4(padding)) == (0, 0, 0, 0)
              and tuple(dilation) == (1, 1) and x.shape[1] % vec == 0)
    if out is None:
        odt = torch.float32 if is_global and not direct else x.dtype
        out = new_features(g.batch, x.shape[1], g.out_h, g.out_w, odt, x.device)
    if out_mask is None:
        out_mask = new_mask(g.batch, g.out_h, g.out_w, x.device)
    _call("pool", lib.dc_pool,
          (g, x.data_ptr(), _ptr(prev_x), out.data_ptr(), _mask(mask, "mask").data_ptr(),
           out_mask.data_ptr(), int(pooling_mode_int), _dtype(x), _dtype(out), _stream()),
          g=g, esize=x.element_size(), in_mask=mask, out_mask=out_mask, mode=int(pooling_mode_int),
          keep=(x, prev_x, out))
    if out.dtype != x.dtype:
        out = out.to(dtype=x.dtype)
    if create_out_mask:
        return out, out_mask
    return out


def sparse_concat_conv(inputs, packed_filter, geometry, out, out_mask):
    """A 1x1 convolution over the channel concatenation of 2..4 delta tensors ``inputs = [(x,
    mask), ...]`` that is never formed (``dc_concat_conv``): identical to chained
    :func:`sparse_concatenate` calls followed by :func:`sparse_conv`.  ``geometry`` describes the
    convolution of the concatenated tensor.  Returns ``None`` (nothing launched) when the shapes
    have no fused form, so the caller can issue the separate calls."""
    lib = _lib.load()
    n = len(inputs)
    if packed_filter is None or not 2 <= n <= 4 or inputs[0][0].dtype not in (torch.float16, torch.bfloat16):
        return None
    for x, _ in inputs:
        _nhwc(x, "input")
    ptrs = (ctypes.c_void_p * n)(*[x.data_ptr() for x, _ in inputs])
    mptrs = (ctypes.c_void_p * n)(*[_mask(m, "mask").data_ptr() for _, m in inputs])
    chans = (ctypes.c_int32 * n)(*[x.shape[1] for x, _ in inputs])
    args = (geometry, n, ctypes.cast(ptrs, ctypes.c_void_p), ctypes.cast(mptrs, ctypes.c_void_p),
            ctypes.cast(chans, ctypes.c_void_p), packed_filter.data_ptr(), out.data_ptr(), out_mask.data_ptr(),
            _dtype(inputs[0][0]), _stream())
    try:
        _call("concat_conv", lib.dc_concat_conv, args, g=geometry, esize=2, in_mask=inputs[0][1], out_mask=out_mask,
              seg_masks=[m for _, m in inputs], seg_channels=[x.shape[1] for x, _ in inputs], mfma=True,
              keep=(ptrs, mptrs, chans, [x for x, _ in inputs]))
    except _lib.DeltaCNNError as e:
        if e.code == -3:
            return None
        raise
    return out, out_mask


def sparse_max_pooling_update(x, prev_x, kernel_size, mask, stride, out=None, out_mask=None):
    """Maximum pooling and the update of the layer's cached input (``prev_x[mask] += x``) in one
    launch (``dc_pool_update``), for windows that tile the map exactly.  Returns ``(out,
    out_mask)``, or ``None`` (nothing launched) for other shapes: the caller then issues
    :func:`sparse_pooling` and :func:`sparse_add_to_dense_tensor`."""
    lib = _lib.load()
    _nhwc(x, "x")
    g = conv_geometry(x.shape, kernel_size, x.shape[1], stride, (0, 0), (1, 1), 1, False, None)
    if out is None:
        out = new_features(g.batch, x.shape[1], g.out_h, g.out_w, x.dtype, x.device)
    if out_mask is None:
        out_mask = new_mask(g.batch, g.out_h, g.out_w, x.device)
    try:
        _call("pool_update", lib.dc_pool_update,
              (g, x.data_ptr(), prev_x.data_ptr(), out.data_ptr(), _mask(mask, "mask").data_ptr(), out_mask.data_ptr(),
               _dtype(x), _stream()),
              g=g, esize=x.element_size(), in_mask=mask, out_mask=out_mask, mode=0, keep=(x, prev_x, out))
    except _lib.DeltaCNNError as e:
        if e.code == -3:
            return None
        raise
    return out, out_mask


def sparse_activation(x, prev_x, truncated, mask, threshold, activation, truncation_mode):
    """cuda_kernels.py:132-133; in place on ``x``, ``prev_x``, ``truncated`` and ``mask``."""
    lib = _lib.load()
    _nhwc(x, "x")
    _call("densify" if truncation_mode < 0 else "activate_truncate", lib.dc_activate_truncate,
          (x.data_ptr(), prev_x.data_ptr(), _ptr(truncated), _mask(mask, "mask").data_ptr(),
           float(threshold), int(activation), int(truncation_mode), _pixels(x), x.shape[1],
           _dtype(x), _stream()),
          P=_pixels(x), C=x.shape[1], esize=x.element_size(), in_mask=mask, out_mask=mask)


def densify(delta, prev_out, out, mask):
    """DCDensify in one launch: ``prev_out += delta`` on active pixels, ``out = prev_out``
    everywhere (sparse_layers.py:1311-1325)."""
    lib = _lib.load()
    _nhwc(delta, "delta")
    _call("densify", lib.dc_densify,
          (delta.data_ptr(), prev_out.data_ptr(), out.data_ptr(), _mask(mask, "mask").data_ptr(), _pixels(delta),
           delta.shape[1], _dtype(delta), _stream()),
          P=_pixels(delta), C=delta.shape[1], esize=delta.element_size(), in_mask=mask, dense_copy=True)


def pooled_densify(x, mask, prev_out, out) -> bool:
    """Global average pooling of the delta ``x`` [B, C, H, W] followed by DCDensify on the pooled
    pixel, in one launch: ``prev_out`` [B, C, 1, 1] accumulates the pooled delta if any pixel of
    the map was updated, ``out`` receives the accumulated value.  Identical to
    ``sparse_pooling`` (average, whole map) followed by ``densify``.  False if the shape has no
    such form (nothing was launched): issue the two calls."""
    lib = _lib.load()
    _nhwc(x, "x")
    g = conv_geometry(x.shape, tuple(x.shape[2:]), x.shape[1], (1, 1), (0, 0), (1, 1), 1)
    try:
        _call("pool_densify", lib.dc_pool_densify,
              (g, x.data_ptr(), _mask(mask, "mask").data_ptr(), prev_out.data_ptr(), out.data_ptr(),
               _dtype(x), _stream()),
              g=g, esize=x.element_size(), in_mask=mask, keep=(x, prev_out, out))
    except _lib.DeltaCNNError as e:
        if e.code == -3:
            return False
        raise
    return True


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ weight.T + bias`` for a few rows ``x`` [rows, in_features] with torch.nn.Linear's
    weight layout [out_features, in_features]: fp32 accumulation, one rounding to the input
    type; returns a new [rows, out_features] tensor.  The library's kernel for the classifier
    behind DCDensify (which the reference leaves to torch, example/mobilenet_deltacnn.py:225)."""
    lib = _lib.load()
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise _lib.DeltaCNNError(-2, f"linear: x {tuple(x.shape)} against weight {tuple(weight.shape)}")
    if not (x.is_cuda and x.is_contiguous() and weight.is_contiguous() and weight.dtype == x.dtype
            and (bias is None or (bias.dtype == x.dtype and bias.is_contiguous()))):
        raise _lib.DeltaCNNError(-2, "linear: contiguous GPU operands of one dtype expected")
    out = torch.empty((x.shape[0], weight.shape[0]), dtype=x.dtype, device=x.device)
    _call("linear", lib.dc_linear,
          (x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(), x.shape[0], x.shape[1],
           weight.shape[0], _dtype(x), _stream()),
          rows=x.shape[0], in_f=x.shape[1], out_f=weight.shape[0], esize=x.element_size(), keep=(x, out))
    return out


def sparsify(input, prev_in, delta, mask, threshold):
    """cuda_kernels.py:136-137."""
    lib = _lib.load()
    _nhwc(input, "input")
    _nhwc(delta, "delta")
    _call("sparsify", lib.dc_sparsify,
          (input.data_ptr(), prev_in.data_ptr(), delta.data_ptr(), _mask(mask, "mask").data_ptr(),
           float(threshold), _pixels(input), input.shape[1], _dtype(input), _stream()),
          P=_pixels(input), C=input.shape[1], esize=input.element_size(), out_mask=mask)


def sparse_add_tensors(a, b, prev_out, out, mask_a, mask_b, mask_out, weight_a, weight_b,
                       activation, dense_out):
    """cuda_kernels.py:140-141."""
    lib = _lib.load()
    _nhwc(a, "a")
    _nhwc(b, "b")
    if a.shape != b.shape:
        raise _lib.DeltaCNNError(-2, f"shape mismatch {tuple(a.shape)} vs {tuple(b.shape)}")
    _call("add", lib.dc_add,
          (a.data_ptr(), b.data_ptr(), _ptr(prev_out), out.data_ptr(),
           _mask(mask_a, "mask_a").data_ptr(), _mask(mask_b, "mask_b").data_ptr(), _ptr(mask_out),
           float(weight_a), float(weight_b), int(activation), int(bool(dense_out)), _pixels(a),
           a.shape[1], _dtype(a), _stream()),
          P=_pixels(a), C=a.shape[1], esize=a.element_size(), in_mask=mask_a, in_mask_b=mask_b,
          out_mask=None if dense_out else mask_out, with_prev=prev_out is not None,
          dense_out=bool(dense_out))


def sparse_add_upsampled(a, b, prev_out, out, mask_a, mask_b, mask_out, weight_a, weight_b, activation, scale):
    """``sparse_add_tensors(a, sparse_upsample(b, scale))`` without the upsampled tensor
    (cuda_kernels.py:132-141 after :152-167): b and mask_b are `scale` times smaller."""
    lib = _lib.load()
    _nhwc(a, "a")
    _nhwc(b, "b")
    bt, c, h, w = a.shape
    scale = int(scale)
    if tuple(b.shape) != (bt, c, h // scale, w // scale) or h % scale or w % scale:
        raise _lib.DeltaCNNError(-2, f"sparse_add_upsampled: {tuple(b.shape)} x{scale} does not give {tuple(a.shape)}")
    _call("add", lib.dc_add_upsampled,
          (a.data_ptr(), b.data_ptr(), _ptr(prev_out), out.data_ptr(), _mask(mask_a, "mask_a").data_ptr(),
           _mask(mask_b, "mask_b").data_ptr(), mask_out.data_ptr(), float(weight_a), float(weight_b),
           int(activation), bt, h, w, c, scale, _dtype(a), _stream()),
          P=_pixels(a), C=c, esize=a.element_size(), in_mask=mask_a, in_mask_b=mask_b, out_mask=mask_out,
          with_prev=prev_out is not None, dense_out=False, b_scale=scale)


def sparse_add_group(items) -> bool:
    """Independent sums in ONE launch (``dc_add_group``).  ``items``: 2 .. 8 tuples ``(a, b,
    prev_out, out, mask_a, mask_b, mask_out, weight_a, weight_b, activation, scale)`` -- the
    arguments of :func:`sparse_add_upsampled`; scale 1: those of :func:`sparse_add_tensors`
    without ``dense_out``.  Every item's results are identical, bit for bit, to the separate
    call's.  Returns ``False`` (nothing launched) when the group has no such form."""
    lib = _lib.load()
    n = len(items)
    if n < 2 or n > _lib.CONV_GROUP_MAX:
        return False
    dtype = items[0][0].dtype
    if dtype not in (torch.float16, torch.bfloat16):
        return False
    arr = (_lib.AddItem * n)()
    metas = []
    for it, (a, b, prev_out, out, mask_a, mask_b, mask_out, wa, wb, activation, scale) in zip(arr, items):
        _nhwc(a, "a")
        _nhwc(b, "b")
        bt, c, h, w = a.shape
        scale = int(scale)
        if a.dtype != dtype or b.dtype != dtype:
            return False
        if tuple(b.shape) != (bt, c, h // scale, w // scale) or h % scale or w % scale:
            raise _lib.DeltaCNNError(-2, f"sparse_add_group: {tuple(b.shape)} x{scale} does not give {tuple(a.shape)}")
        it.a, it.b, it.prev_out, it.out = a.data_ptr(), b.data_ptr(), _ptr(prev_out), out.data_ptr()
        it.mask_a, it.mask_b = _mask(mask_a, "mask_a").data_ptr(), _mask(mask_b, "mask_b").data_ptr()
        it.mask_out = mask_out.data_ptr()
        it.weight_a, it.weight_b, it.activation = float(wa), float(wb), int(activation)
        it.batch, it.height, it.width, it.channels, it.scale = bt, h, w, c, scale
        metas.append(dict(P=_pixels(a), C=c, in_mask=mask_a, in_mask_b=mask_b, out_mask=mask_out,
                          with_prev=prev_out is not None, b_scale=scale))
    try:
        _call("add_group", lib.dc_add_group, (arr, n, _DTYPES[dtype], _stream()), items=metas,
              esize=items[0][0].element_size(), keep=(arr, items))
    except _lib.DeltaCNNError as e:
        if e.code == -3:
            return False
        raise
    return True


def sparse_add_to_dense_tensor(a, b, mask_a, activation=0):
    """cuda_kernels.py:144-145: ``b[px] += a[px]`` on active pixels."""
    lib = _lib.load()
    _nhwc(a, "a")
    _call("add_to_dense", lib.dc_add_to_dense,
          (a.data_ptr(), b.data_ptr(), _mask(mask_a, "mask_a").data_ptr(), int(activation),
           _pixels(a), a.shape[1], _dtype(a), _stream()),
          P=_pixels(a), C=a.shape[1], esize=a.element_size(), in_mask=mask_a)


def sparse_mul_add(x, x_mask, out, out_mask, scale, bias):
    """cuda_kernels.py:148-149: per-channel ``x*scale (+bias)`` on active pixels."""
    lib = _lib.load()
    _nhwc(x, "x")
    scale = scale.reshape(-1).to(x.dtype).contiguous()
    bias = None if bias is None else bias.reshape(-1).to(x.dtype).contiguous()
    _call("mul_add", lib.dc_mul_add,
          (x.data_ptr(), _mask(x_mask, "x_mask").data_ptr(), out.data_ptr(), out_mask.data_ptr(),
           scale.data_ptr(), _ptr(bias), _pixels(x), x.shape[1], _dtype(x), _stream()),
          P=_pixels(x), C=x.shape[1], esize=x.element_size(), in_mask=x_mask)


def sparse_upsample(input, mask_in, scale, out=None):
    """cuda_kernels.py:152-167."""
    lib = _lib.load()
    _nhwc(input, "input")
    b, c, h, w = input.shape
    scale = int(scale)
    if out is None:
        out_t = new_features(b, c, h * scale, w * scale, input.dtype, input.device)
        mask_out = new_mask(b, h * scale, w * scale, input.device)
    else:
        out_t, mask_out = out
    _call("upsample", lib.dc_upsample,
          (input.data_ptr(), out_t.data_ptr(), _mask(mask_in, "mask_in").data_ptr(),
           mask_out.data_ptr(), b, h, w, c, scale, _dtype(input), _stream()),
          P=b * h * w, C=c, esize=input.element_size(), in_mask=mask_in, scale=scale,
          keep=(input, out_t, mask_out))
    return out_t, mask_out


def sparse_concatenate(a, b, out=None):
    """cuda_kernels.py:170-185."""
    lib = _lib.load()
    a, mask_a = a
    b, mask_b = b
    _nhwc(a, "a")
    _nhwc(b, "b")
    if out is None:
        out_t = new_features(a.shape[0], a.shape[1] + b.shape[1], a.shape[2], a.shape[3], a.dtype,
                             a.device)
        mask_out = new_mask(a.shape[0], a.shape[2], a.shape[3], a.device)
    else:
        out_t, mask_out = out
    _call("concat", lib.dc_concat,
          (a.data_ptr(), b.data_ptr(), out_t.data_ptr(), _mask(mask_a, "mask_a").data_ptr(),
           _mask(mask_b, "mask_b").data_ptr(), mask_out.data_ptr(), _pixels(a), a.shape[1],
           b.shape[1], _dtype(a), _stream()),
          P=_pixels(a), C=a.shape[1], Cb=b.shape[1], esize=a.element_size(), in_mask=mask_a,
          in_mask_b=mask_b, out_mask=mask_out, keep=(a, b, out_t))
    return out_t, mask_out
