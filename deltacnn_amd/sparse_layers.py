"""Stateful DeltaCNN layers over the gfx950 HIP kernels.

Same classes, constructor arguments and frame protocol as the reference's
``src/deltacnn/sparse_layers.py``: every layer caches accumulated dense state from earlier
frames and exchanges ``(delta, mask)`` tuples (``delta``: NHWC features whose inactive
pixels are undefined, ``mask``: int32 ``[B,1,H,W]``).  A plain ``Tensor`` input takes the
dense pass-through branch like in the reference.

Backends (``DCConv2d.backend``): ``DCBackend.deltacnn`` runs the HIP kernels of
libdeltacnn_hip.so -- there is no other implementation of the delta path in this package;
``DCBackend.cudnn`` is the dense torch model (MIOpen on ROCm).  ``delta_cudnn`` (a
training aid of the reference) is not provided.
"""
from __future__ import annotations

import json
from collections import OrderedDict
from enum import Enum

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from . import hip_kernels as hk
from .filter_conversion import convert_filter_out_channels_last, convert_half_filter


def convert_activation_string(name, **kwargs):
    """sparse_layers.py:20-34: (dense torch callable, kernel activation id)."""
    if name is None or name == "" or name.lower() == "linear":
        return None, -1
    key = name.lower()
    if key == "relu":
        return torch.nn.ReLU(), 1
    if key == "relu6":
        return torch.nn.ReLU6(), 2
    if key == "leaky":
        return torch.nn.LeakyReLU(kwargs.get("leaky_relu_negative_slope", 1e-2)), 3
    if key == "sigmoid":
        return torch.nn.Sigmoid(), 4
    if key == "swish":
        return (lambda x: torch.sigmoid(x).mul_(x)), 5
    raise Exception(f"Activation {name} not implemented")


class _NamedChoice:
    """Enum mix-in: look a member up by its (case-insensitive) name."""

    @classmethod
    def parse_string(cls, text):
        member = cls.__members__.get(str(text).lower())
        if member is None:
            raise Exception(f"invalid {cls.__name__} value {text!r}; one of {', '.join(cls.__members__)}")
        return member


class DCBackend(_NamedChoice, Enum):
    """Which implementation a convolution layer runs (sparse_layers.py:64-75)."""
    cudnn = 0        # dense torch layers
    deltacnn = 1     # the delta kernels
    delta_cudnn = 2  # the reference's training aid; not provided here


class DCTruncation(_NamedChoice, Enum):
    """How an activation layer decides that an update is too small to pass on
    (sparse_layers.py:102-117)."""
    none = -1
    max = 0
    norm = 1
    rms = 2


class _ThresholdFile:
    """Per-layer thresholds on disk: one JSON object {"0": t0, "1": t1, ...} numbered in the
    order the layers registered (the file format of the reference, sparse_layers.py:157-186)."""

    def __init__(self, path):
        self.path = path

    def read(self):
        with open(self.path) as f:
            table = json.load(f)
        return [table[str(i)] for i in range(len(table))]

    def write(self, values):
        with open(self.path, "w+") as f:
            json.dump(dict(enumerate(values)), f)


class DCThreshold:
    """Registry of per-layer thresholds keyed by module (sparse_layers.py:122-208).

    A layer registers its threshold on its first frame (`set` never overwrites) and looks it
    up on every later frame, so a file loaded after frame 0 overrides the defaults.
    """
    t = OrderedDict()    # layer -> threshold, in registration order
    t_default = 0.0      # what a layer without a delta_threshold of its own registers
    path = None          # JSON file for load_thresholds
    scale = 1.0          # factor applied to the file's values
    initialized = False  # load_thresholds has run since the last reset

    @classmethod
    def get(cls, key, default=0.0):
        return cls.t.get(key, default)

    @classmethod
    def set(cls, key, val):
        cls.t.setdefault(key, val)

    @classmethod
    def load_thresholds(cls):
        """Once per reset: overwrite the registered thresholds with `path`'s values times
        `scale`.  File and registry are aligned at their ENDS: a shorter file describes the
        layers registered last, a longer one loses its leading entries."""
        already, cls.initialized = cls.initialized, True
        if already or cls.path is None:
            return
        values = _ThresholdFile(cls.path).read()
        layers = list(cls.t)
        if len(values) != len(layers):
            print(f"WARNING: {cls.path} holds {len(values)} thresholds, the model registered {len(layers)}")
        for layer, value in zip(reversed(layers), reversed(values)):
            cls.t[layer] = value * cls.scale

    @classmethod
    def save_thresholds(cls, name):
        _ThresholdFile(f"thresholds_{name}.json").write(list(cls.t.values()))

    @classmethod
    def reset(cls):
        """Forget every registered layer and the file."""
        cls.path, cls.initialized = None, False
        cls.t.clear()


class DCModule(nn.Module):
    """Base of every stateful layer.  `temp_buffers` lists all cache tensors of all layers
    (class level, sparse_layers.py:212), `reset_layers` returns a model to "no frame seen"."""
    temp_buffers = []
    # Intermediate (delta, mask) outputs live in per-layer buffers that are reused frame after
    # frame (the reference allocates with torch.empty on every call, cuda_kernels.py:34-37):
    # a returned delta tuple is valid until the same layer runs its next frame.  Dense results
    # (DCDensify, dense_out) are fresh tensors per call like in the reference.
    reuse_buffers = True

    def __init__(self):
        super().__init__()

    @classmethod
    def get_temp_buffer_numel(cls):
        return sum(buf.numel() for buf in cls.temp_buffers)

    @staticmethod
    def _cache(tensor):
        """Book a per-layer cache tensor in the class-level list and hand it back."""
        DCModule.temp_buffers.append(tensor)
        return tensor

    def _take_index(self, owner):
        """First frame of a layer: number it within `owner`, the class that holds the `idx`
        counter of its kind."""
        owner.idx += 1
        self.idx = owner.idx

    def reset(self):
        DCModule.temp_buffers = []

    def process_filters(self):
        for layer in self.modules():
            if type(layer) in (DCConv2d, DCConvTranspose2d):
                layer.process_filters()

    def reset_layers(self):
        # nn.Module.modules() walks the whole tree and yields each module once
        for layer in self.modules():
            if layer is not self and isinstance(layer, DCModule):
                layer.reset()
        DCModule.temp_buffers.clear()


def _pair(v):
    if isinstance(v, int):
        return (v, v)
    v = tuple(v)
    return v + v if len(v) == 1 else v


def to_tuple(*args):
    """ints and 1-sequences become (v, v); longer sequences pass as tuples.  One argument
    returns its pair, several return the list of pairs (sparse_layers.py:241-253)."""
    pairs = [_pair(a) for a in args]
    return pairs[0] if len(pairs) == 1 else pairs


def _matches(buf, like) -> bool:
    """A reusable buffer still fits: same shape, dtype and device as `like`."""
    return buf is not None and buf.shape == like.shape and buf.dtype == like.dtype and buf.device == like.device


def _is_depthwise(m) -> bool:
    return m.groups == m.out_channels and m.groups == m.in_channels and m.groups > 1


class _DeltaConvBase:
    """State and delta-path forward shared by DCConv2d and DCConvTranspose2d."""
    _transposed = False

    def _init_delta(self, delta_threshold, name, activation, dense_out, backend, kwargs):
        self.prev_in = None
        self.prev_out = None
        self.delta_threshold = delta_threshold if delta_threshold is not None else DCThreshold.t_default
        self.name = name
        self.backend = backend if backend is not None else DCConv2d.backend
        self.activation, self.activation_int = convert_activation_string(activation, **kwargs)
        self.dense_out = dense_out
        self.densify_layer = None
        self.activation_layer = None
        if self.dense_out:
            self.densify_layer = DCDensify(activation=activation, name=self.name)
        elif self.activation is not None:
            self.activation_layer = DCActivation(self.name, delta_threshold=delta_threshold,
                                                 activation=activation)
        self.conv_idx = -1
        self.dense_in = False
        self.frame_idx = -1
        self.out_shape = []
        self.in_shape = None
        self.kwargs = kwargs
        self.filters_processed = False
        self._packed = None
        self._plan = None
        assert kwargs.get("leaky_relu_negative_slope", 0.1) == 0.1, \
            "Leaky ReLU implementation uses hard coded negative slope of 0.1"

    def init_first_iter(self, input):
        """First call: take the layer's number from the class-level call counter
        (sparse_layers.py:341), note what kind of input arrives and register the threshold of a
        fused activation."""
        dense = isinstance(input, Tensor)
        self.dense_in = dense
        self.in_shape = (input if dense else input[0]).shape
        self.conv_idx = DCConv2d.conv_idx
        if self.backend != DCBackend.cudnn and self.activation is not None:
            DCThreshold.set(self, self.delta_threshold)

    def forward(self, input):
        # the class-level counter advances on every call of every convolution (:425); a layer
        # is on its first frame while it has not copied a number from it yet (:427)
        DCConv2d.conv_idx += 1
        self.frame_idx += 1
        first_iter = self.conv_idx < 0
        if first_iter:
            self.init_first_iter(input)
        if self.backend == DCBackend.deltacnn:
            return self._forward_delta_conv(input, first_iter)
        if self.backend == DCBackend.cudnn:
            return self._forward_dense(input)
        raise NotImplementedError("the delta_cudnn training backend is not part of this package")

    def _forward_dense(self, input):
        out = self._conv_forward_dense(input)
        return self.activation(out) if self.activation is not None else out

    def _make_plan(self, shape, dtype, device):
        pad = self.padding4 if getattr(self, "padding4", None) is not None else self.padding
        w = self.weight
        g = hk.conv_geometry(shape, (w.shape[1], w.shape[2]), self.out_channels, self.stride, pad,
                             self.dilation, self.groups, self._transposed)
        plan = {"shape": tuple(shape), "dtype": dtype, "g": g, "out": None, "out_mask": None}
        if DCModule.reuse_buffers:
            plan["out"] = hk.new_features(g.batch, g.out_c, g.out_h, g.out_w, dtype, device)
            plan["out_mask"] = hk.new_mask(g.batch, g.out_h, g.out_w, device)
        return plan

    def _plan_for(self, shape, dtype, device):
        """Geometry and reusable output buffers for an input of this shape."""
        if self._plan is None or self._plan["shape"] != tuple(shape) or self._plan["dtype"] != dtype:
            self._plan = self._make_plan(shape, dtype, device)
            self.in_shape = torch.Size(shape)
        return self._plan

    def _packed_filter(self):
        """The filter in matrix-core fragment order (made once), or None if it has no such form."""
        if self._packed is None:
            made = hk.pack_filter(self.weight.data, self.in_channels, self.out_channels, self.groups,
                                  self._transposed)
            self._packed = False if made is None else made
        return None if self._packed is False else self._packed

    def _prepare(self, input):
        if type(input) == Tensor:
            raise TypeError("the deltacnn backend propagates (delta, mask) tuples: put a "
                            "DCSparsify in front of the first convolution")
        if not self.filters_processed:
            raise RuntimeError("call process_filters() on the model (after moving it to the GPU "
                               "in channels_last) before the first frame")
        x, mask = input
        plan = self._plan_for(x.shape, x.dtype, x.device)
        bias = self.bias if self.frame_idx <= 0 else None
        pad = self.padding4 if getattr(self, "padding4", None) is not None else self.padding
        return x, mask, plan, self._packed_filter(), bias, pad

    def conv_delta(self, input):
        """The convolution alone: ``(delta, mask) -> (out, out_mask)`` without the layer's
        activation / densify stage (bias is applied while ``frame_idx <= 0``)."""
        x, mask, plan, packed, bias, pad = self._prepare(input)
        fn = hk.sparse_deconv if self._transposed else hk.sparse_conv
        return fn(x=x, filter=self.weight, mask=mask, bias=bias, stride=self.stride, padding=pad,
                  dilation=self.dilation, groups=self.groups, c_out=self.out_channels,
                  create_out_mask=True, out_mask=plan["out_mask"], packed_filter=packed,
                  out=plan["out"], geometry=plan["g"])

    def _forward_delta_conv(self, input, first_iter):
        act = self.activation_layer
        fuse = (act is not None and not act.first_iter and not self._transposed
                and DCConv2d.fuse_activation and act.inplace)
        if fuse:
            # activation/truncation runs as the epilogue of the convolution call
            x, mask, plan, packed, bias, pad = self._prepare(input)
            return hk.sparse_conv_activation(
                x, self.weight, mask, bias, act.prev_out, act.out_truncated,
                DCThreshold.get(act), act.activation_int, act.truncation_mode.value, self.stride,
                pad, self.dilation, self.groups, self.out_channels, packed_filter=packed,
                out=plan["out"], out_mask=plan["out_mask"], geometry=plan["g"])
        out, out_mask = self.conv_delta(input)
        if self.dense_out:
            return self.densify_layer((out, out_mask))
        if act is not None:
            return act((out, out_mask))
        return out, out_mask

    def reset(self):
        DCModule.reset(self)
        DCConv2d.conv_idx = -1
        self.conv_idx = self.frame_idx = -1
        self.prev_in = self.prev_out = None
        self.out_shape = []

    def process_filters(self):
        """Once per layer: move the weights into the layout the kernels read
        (filter_conversion.py; sparse_layers.py:648-675).  The torch layout is kept in
        ``orig_weights``; fp16 weights are padded to even channel counts and pair-swizzled,
        fp32 weights become [Cin][Kh][Kw][Cout]."""
        if self.filters_processed:
            return
        self.orig_weights = self.weight.data.clone()
        half = self.weight.data.dtype == torch.float16
        (self.process_filters_half if half else self.process_filters_single)()

    def process_filters_half(self):
        layer = self.half()
        if self.backend == DCBackend.deltacnn:
            layer.weight.data = convert_half_filter(layer.weight.data, pixel_wise=_is_depthwise(self),
                                                    transposed=self._transposed)
            self._filters_ready()
        return layer

    def process_filters_single(self):
        if self.backend == DCBackend.deltacnn:
            self.weight.data = convert_filter_out_channels_last(self.weight.data, transposed=self._transposed)
            self._filters_ready()
        return self

    def _filters_ready(self):
        self.filters_processed = True
        self._packed = None


class DCConv2d(_DeltaConvBase, nn.Conv2d, DCModule):
    """Delta convolution (sparse_layers.py:261-675)."""
    backend = DCBackend.deltacnn
    conv_idx = -1
    fuse_activation = True
    fuse_expansion = True  # expand_depthwise(): 1x1 expansion + activation -> depthwise 3x3 + activation in two launches
    fuse_projection = True  # project_expand(): projection (+ residual sum) + next expansion (left open) in one launch
    fuse_blocks = True  # fused_block(): depthwise -> projection (-> expansion) in one launch
    fuse_groups = True  # conv_group() / residual_group(): the same layer of several parallel branches in one launch
    # ... while the two 1x1 filters together stay below this many bytes: every 16-pixel workgroup
    # of that launch reads both in full, and one compute unit pulls only a few GB/s out of the
    # far caches, so larger layers are faster as separate launches that spread their filter over
    # many workgroups
    fuse_blocks_max_filter_bytes = 32 << 10
    # ... and up to this many output pixels (one stream at a time: the latency regime, where a
    # launch saved is time saved).  On larger maps -- many streams as a batch -- the separate
    # kernels are bandwidth-efficient and faster than the one-launch form (measured at 32 streams:
    # 0.77 ms per step against 0.93 ms).
    fuse_blocks_max_pixels = 16384

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, padding_mode="zeros", delta_threshold=None, name=None,
                 activation=None, dense_out=False, backend=None, use_logging=None, **kwargs):
        kernel_size, stride, padding, dilation = to_tuple(kernel_size, stride, padding, dilation)
        self.padding4 = None
        pad2 = padding
        if len(padding) == 4:  # (top, bottom, left, right), cuda_kernels.py:24-26
            self.padding4, pad2 = tuple(padding), (0, 0)
        nn.Conv2d.__init__(self, in_channels, out_channels, kernel_size, stride, pad2, dilation,
                           groups, bias, padding_mode)
        self._init_delta(delta_threshold, name, activation, dense_out, backend, kwargs)

    def __repr__(self):
        return f"DCConv2d{self.conv_idx} cin={self.in_channels} cout={self.out_channels}"

    def _conv_forward_dense(self, input):
        if self.padding4 is not None:
            t, b, l, r = self.padding4
            input = torch.nn.functional.pad(input, (l, r, t, b))
        return self._conv_forward(input, self.weight, self.bias)


class DCConvTranspose2d(_DeltaConvBase, nn.ConvTranspose2d, DCModule):
    """Delta transposed convolution (sparse_layers.py:678-1083).  ``output_padding`` does not
    enter the output size of the delta path (cuda_kernels.py:56-57)."""
    _transposed = True

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0,
                 output_padding=0, groups=1, bias=True, dilation=1, padding_mode="zeros",
                 delta_threshold=None, name=None, activation=None, store_prev_in=False,
                 dense_out=False, backend=None, use_logging=None, **kwargs):
        kernel_size, stride, padding, dilation = to_tuple(kernel_size, stride, padding, dilation)
        nn.ConvTranspose2d.__init__(self, in_channels, out_channels, kernel_size, stride, padding,
                                    output_padding, groups, bias, dilation, padding_mode)
        self.padding4 = None
        self._init_delta(delta_threshold, name, activation, dense_out, backend, kwargs)

    def _conv_forward_dense(self, input):
        return nn.ConvTranspose2d.forward(self, input)


class DCAdd(DCModule):
    """Weighted sum of two delta tensors over the union of their masks, optionally followed by
    an activation on the accumulated sum or by a dense output (sparse_layers.py:1086-1182)."""
    idx = -1
    fuse_into_conv = True

    def __init__(self, activation: str = None, dense_out=False, weight_a=None, weight_b=None, name=""):
        super().__init__()
        self.activation, self.activation_int = convert_activation_string(activation)
        self.name, self.dense_out = name, dense_out
        self.weight_a, self.weight_b = (1.0 if w is None else w for w in (weight_a, weight_b))
        self._forget()

    def _forget(self):
        self.idx = -1
        self.first_iter = True
        self.prev_out = self.out = self.mask_out = None

    def _needs_sum_cache(self):
        """An activation or a dense output works on the accumulated sum of all frames."""
        return self.dense_out or self.activation is not None

    def _result_buffers(self, like, like_mask):
        """(delta, mask) buffers for the result: per-layer and reused between frames, except the
        dense_out result, which is a fresh tensor per call."""
        if not DCModule.reuse_buffers:
            return torch.empty_like(like), torch.empty_like(like_mask)
        if not _matches(self.mask_out, like_mask):
            self.mask_out = torch.empty_like(like_mask)
        if self.dense_out:
            return torch.empty_like(like), self.mask_out
        if not _matches(self.out, like):
            self.out = torch.empty_like(like)
        return self.out, self.mask_out

    def forward(self, a, b, weight_a=None, weight_b=None):
        wa = self.weight_a if weight_a is None else weight_a
        wb = self.weight_b if weight_b is None else weight_b
        if isinstance(a, Tensor):  # dense operands: plain arithmetic
            total = wa * a + wb * b
            return total if self.activation is None else self.activation(total)
        (delta_a, mask_a), (delta_b, mask_b) = a, b
        if self.first_iter:
            self.first_iter = False
            self._take_index(DCAdd)
            if self._needs_sum_cache():
                self.prev_out = self._cache(torch.zeros_like(delta_a))
        out, mask_out = self._result_buffers(delta_a, mask_a)
        hk.sparse_add_tensors(delta_a, delta_b, self.prev_out, out, mask_a, mask_b, mask_out, wa, wb,
                              self.activation_int, self.dense_out)
        return out if self.dense_out else (out, mask_out)

    def after_conv(self, a, conv, conv_input):
        """``self(a, conv(conv_input))`` with the addition fused into the convolution's kernel
        when that is possible (fp16 convolution without activation of its own -- pointwise, or a
        small layer of any kernel size, which may also carry this layer's activation -- and no
        dense_out); otherwise exactly the two separate layer calls."""
        fusable = (DCAdd.fuse_into_conv and type(a) != Tensor and not self.first_iter
                   and not self.dense_out and isinstance(conv, DCConv2d) and conv.activation is None
                   and not conv.dense_out and conv.backend == DCBackend.deltacnn
                   and conv.frame_idx >= 0 and type(conv_input) != Tensor)
        if fusable:
            # conv.frame_idx >= 0: the convolution has seen its first frame, no bias from here on;
            # not self.first_iter: this layer's accumulated sum exists if it has an activation
            val_a, mask_a = a
            x, mask, plan, packed, _, _ = conv._prepare(conv_input)
            g = plan["g"]
            if packed is not None and tuple(val_a.shape) == (g.batch, g.out_c, g.out_h, g.out_w):
                if not _matches(self.out, val_a):
                    self.out = torch.empty_like(val_a)
                if not _matches(self.mask_out, mask_a):
                    self.mask_out = torch.empty_like(mask_a)
                res = hk.sparse_conv_add(x, packed, mask, None, val_a, mask_a, plan["g"], self.out,
                                         self.mask_out, self.weight_a, self.weight_b,
                                         self.prev_out if self.activation is not None else None,
                                         self.activation_int if self.activation is not None else 0)
                if res is not None:
                    DCConv2d.conv_idx += 1
                    conv.frame_idx += 1
                    return res
        return self(a, conv(conv_input))

    def conv_first(self, conv, conv_input, b):
        """``self(conv(conv_input), b)`` for a transposed convolution ``conv`` without activation:
        the addition runs in the convolution's kernel (``dc_deconv_add``) when this layer has unit
        weights, no activation and no dense_out -- the sum is then commutative bit for bit, and
        the kernel takes ``b`` as its residual operand; otherwise exactly the two layer calls."""
        fusable = (DCAdd.fuse_into_conv and type(b) != Tensor and type(conv_input) != Tensor and not self.first_iter
                   and not self.dense_out and self.activation is None and self.weight_a == 1.0 and self.weight_b == 1.0
                   and isinstance(conv, DCConvTranspose2d) and conv.activation is None and not conv.dense_out
                   and conv.backend == DCBackend.deltacnn and conv.frame_idx >= 0)
        if fusable:
            val_b, mask_b = b
            x, mask, plan, packed, _, _ = conv._prepare(conv_input)
            g = plan["g"]
            if packed is not None and tuple(val_b.shape) == (g.batch, g.out_c, g.out_h, g.out_w):
                if not _matches(self.out, val_b):
                    self.out = torch.empty_like(val_b)
                if not _matches(self.mask_out, mask_b):
                    self.mask_out = torch.empty_like(mask_b)
                res = hk.sparse_deconv_add(x, packed, mask, val_b, mask_b, g, self.out, self.mask_out)
                if res is not None:
                    DCConv2d.conv_idx += 1
                    conv.frame_idx += 1
                    return res
        return self(conv(conv_input), b)

    def after_upsample(self, a, b, upsample):
        """``self(a, upsample(b))`` with the nearest upsampling folded into the addition's kernel
        (the upsampled tensor is never stored) when both operands are delta tensors and this
        layer has no dense_out; otherwise exactly the two separate layer calls."""
        fusable = (DCAdd.fuse_into_conv and type(a) != Tensor and type(b) != Tensor and not self.first_iter
                   and not self.dense_out and isinstance(upsample, DCUpsamplingNearest2d))
        if not fusable:
            return self(a, upsample(b))
        val_a, mask_a = a
        val_b, mask_b = b
        if not _matches(self.out, val_a):
            self.out = torch.empty_like(val_a)
        if not _matches(self.mask_out, mask_a):
            self.mask_out = torch.empty_like(mask_a)
        hk.sparse_add_upsampled(val_a, val_b, self.prev_out if self.activation is not None else None, self.out,
                                mask_a, mask_b, self.mask_out, self.weight_a, self.weight_b,
                                self.activation_int if self.activation is not None else 0, upsample.scale_factor)
        return self.out, self.mask_out

    def reset(self):
        super().reset()
        self._forget()
        DCAdd.idx = -1


def _steady(conv) -> bool:
    """A convolution layer of the delta backend that has seen its first frame (no bias from here
    on) and owns processed fp16 filters."""
    return (isinstance(conv, DCConv2d) and conv.backend == DCBackend.deltacnn and conv.frame_idx >= 0
            and conv.filters_processed and conv.weight.dtype == torch.float16 and not conv.dense_out)


def _steady_activation(conv):
    """The convolution's fused activation layer if it can run inside another kernel: past its
    first frame, in place, truncation mode max."""
    act = conv.activation_layer
    if act is None or act.first_iter or not act.inplace or act.truncation_mode != DCTruncation.max:
        return None
    return act


def fused_block_wanted(depthwise, project, expand, hidden_shape, dtype) -> bool:
    """The policy part of :func:`fused_block`, decidable before the block's hidden tensor exists:
    the class switches, the layers' steady state, filter bytes and pixel count."""
    if not DCConv2d.fuse_blocks or dtype != torch.float16:
        return False
    if not (_steady(depthwise) and _steady(project) and (expand is None or _steady(expand))):
        return False
    if _steady_activation(depthwise) is None or project.activation is not None or not _is_depthwise(depthwise):
        return False
    filter_bytes = 2 * project.out_channels * (project.in_channels + (expand.out_channels if expand is not None else 0))
    if filter_bytes > DCConv2d.fuse_blocks_max_filter_bytes:
        return False
    g = depthwise._plan_for(hidden_shape, dtype, depthwise.weight.device)["g"]
    return g.batch * g.out_h * g.out_w <= DCConv2d.fuse_blocks_max_pixels


class OpenExpansion:
    """What :func:`project_expand` hands to the next block in place of its expansion's output: the
    expansion's convolution has run with its activation left open, and :func:`expand_depthwise`
    has to finish it (``opened=`` this object) before anything else touches the two layers."""

    def __init__(self, expand, depthwise):
        self.expand, self.depthwise = expand, depthwise


def _closing_pair(expand, depthwise, dtype):
    """The conditions of :func:`expand_depthwise` on the two layers themselves."""
    for conv in (expand, depthwise):
        if not (isinstance(conv, DCConv2d) and conv.backend == DCBackend.deltacnn and conv.frame_idx >= 0
                and conv.filters_processed and not conv.dense_out):
            return None
    act_e, act_d = expand.activation_layer, depthwise.activation_layer
    if (act_e is None or act_e.first_iter or not act_e.inplace or act_e.truncation_mode != DCTruncation.max
            or act_d is None or act_d.first_iter or not act_d.inplace):
        return None
    if (not _is_depthwise(depthwise) or depthwise.padding4 is not None
            or (expand.kernel_size, expand.stride, expand.padding, expand.groups) != ((1, 1), (1, 1), (0, 0), 1)):
        return None
    if dtype not in (torch.float16, torch.bfloat16) or dtype != expand.weight.dtype:
        return None
    return act_e, act_d


def project_expand(project, add, residual, expand, depthwise, input):
    """``add(residual, project(input))`` (``add`` / ``residual`` may be None) and the convolution of
    the NEXT block's 1x1 expansion ``expand`` in one launch (``dc_project_expand``), on frames after
    the first.  The expansion's activation is left open; ``depthwise`` is the layer behind it, which
    finishes it.  Returns ``(block_output, opened)`` -- the block's ``(delta, mask)`` exactly as
    the separate layer calls return it, and an :class:`OpenExpansion` that MUST be the next thing
    handed to :func:`expand_depthwise` -- or ``None`` when the layers are not in a state or of a
    shape the kernel takes; nothing has happened then.  Switch: ``DCConv2d.fuse_projection``."""
    if not (DCConv2d.fuse_projection and DCConv2d.fuse_expansion) or isinstance(input, Tensor):
        return None
    x, mask = input
    acts = _closing_pair(expand, depthwise, x.dtype)
    if acts is None:
        return None
    act_e, act_d = acts
    if not (isinstance(project, DCConv2d) and project.backend == DCBackend.deltacnn and project.frame_idx >= 0
            and project.filters_processed and not project.dense_out and project.activation is None
            and project.weight.dtype == x.dtype
            and (project.kernel_size, project.stride, project.padding, project.groups) == ((1, 1), (1, 1), (0, 0), 1)):
        return None
    if add is not None and (not DCAdd.fuse_into_conv or add.first_iter or add.dense_out or add.activation is not None
                            or residual is None or isinstance(residual, Tensor)):
        return None
    plan_p = project._plan_for(x.shape, x.dtype, x.device)
    packed_p, packed_e = project._packed_filter(), expand._packed_filter()
    if packed_p is None or packed_e is None or plan_p["out"] is None:
        return None
    plan_e = expand._plan_for(plan_p["out"].shape, x.dtype, x.device)
    if plan_e["out"] is None:
        return None
    plan_d = depthwise._plan_for(plan_e["out"].shape, x.dtype, x.device)
    # everything the closing call will need, before the launch that cannot be taken back
    if plan_d["out"] is None or any(not _matches(t, plan_e["out"]) for t in (act_e.prev_out, act_e.out_truncated)) \
            or any(not _matches(t, plan_d["out"]) for t in (act_d.prev_out, act_d.out_truncated)):
        return None
    out, out_mask = plan_p["out"], plan_p["out_mask"]
    res_v = res_m = None
    wa = wb = 1.0
    if add is not None:
        res_v, res_m = residual
        if tuple(res_v.shape) != tuple(out.shape):
            return None
        if not _matches(add.out, res_v):
            add.out = torch.empty_like(res_v)
        if not _matches(add.mask_out, res_m):
            add.mask_out = torch.empty_like(res_m)
        out, out_mask, wa, wb = add.out, add.mask_out, add.weight_a, add.weight_b
    done = hk.sparse_project_expand(
        x, mask, packed_p, plan_p["g"], res_v, res_m, out, out_mask, packed_e, act_e.prev_out, act_e.out_truncated,
        act_e.activation_int, plan_e["out"], plan_e["out_mask"], plan_d["g"], act_d.activation_int,
        act_d.truncation_mode.value, wa, wb)
    if not done:
        return None
    DCConv2d.conv_idx += 1  # the projection's own forward call; the expansion counts when it is finished
    project.frame_idx += 1
    return (out, out_mask), OpenExpansion(expand, depthwise)


def concat_conv(conv, inputs):
    """``conv(cat(inputs))`` for a 1x1 DCConv2d (with or without activation) over the channel
    concatenation of 2..4 delta tensors, on frames after the first: the convolution reads the
    tensors where they lie (``dc_concat_conv``), no DCConcatenate launch runs, and the layer's own
    activation follows as in its forward call.  Returns what the layer returns, or ``None`` when
    the layer is not in a state or of a shape the kernel takes; nothing has happened then and the
    caller concatenates and calls the layer.  Switch: ``DCConcatenate.fuse_into_conv``."""
    if not DCConcatenate.fuse_into_conv or any(isinstance(x, Tensor) for x in inputs) or not 2 <= len(inputs) <= 4:
        return None
    x0 = inputs[0][0]
    if not (isinstance(conv, DCConv2d) and not conv._transposed and conv.backend == DCBackend.deltacnn
            and conv.frame_idx >= 0 and conv.conv_idx >= 0 and conv.filters_processed and not conv.dense_out
            and conv.weight.dtype == x0.dtype
            and (conv.kernel_size, conv.stride, conv.padding, conv.groups) == ((1, 1), (1, 1), (0, 0), 1)):
        return None
    act = conv.activation_layer
    if act is not None and act.first_iter:
        return None
    b, _, h, w = x0.shape
    if any(x.shape[0] != b or x.shape[2:] != x0.shape[2:] or x.dtype != x0.dtype for x, _ in inputs):
        return None
    total = sum(x.shape[1] for x, _ in inputs)
    plan = conv._plan_for((b, total, h, w), x0.dtype, x0.device)
    packed = conv._packed_filter()
    if packed is None or plan["out"] is None:
        return None
    done = hk.sparse_concat_conv(list(inputs), packed, plan["g"], plan["out"], plan["out_mask"])
    if done is None:
        return None
    DCConv2d.conv_idx += 1  # what the layer's own forward call would have counted
    conv.frame_idx += 1
    return done if act is None else act(done)


def expand_depthwise(expand, depthwise, input, opened=None):
    """``depthwise(expand(input))`` for a 1x1 expansion DCConv2d and a 3x3 depthwise DCConv2d
    (stride 1 or 2), both with a truncating activation, as TWO launches instead of three on frames
    after the first: the expansion's convolution leaves its keep decision to the depthwise
    kernel (``dc_expand_depthwise``).  Returns the depthwise layer's ``(delta, mask)`` -- exactly
    what the separate layer calls return, all layer states included -- or ``None`` when the
    layers are not in a state or of a shape the kernels take; nothing has happened then and the
    caller runs the layers one by one.  Switch: ``DCConv2d.fuse_expansion``.

    ``opened``: the :class:`OpenExpansion` of a :func:`project_expand` call that has already run
    the expansion's convolution on ``input``; only the depthwise launch remains, and it cannot be
    declined any more."""
    if opened is not None:
        if opened.expand is not expand or opened.depthwise is not depthwise:
            raise RuntimeError("an open expansion has to be finished by the layers it was opened for")
    elif not DCConv2d.fuse_expansion or isinstance(input, Tensor):
        return None
    x, mask = input
    acts = _closing_pair(expand, depthwise, x.dtype)
    if acts is None:
        if opened is not None:
            raise RuntimeError("the layers of an open expansion changed state before it was finished")
        return None
    act_e, act_d = acts
    plan_e = expand._plan_for(x.shape, x.dtype, x.device)
    packed = expand._packed_filter()
    plan_d = None if plan_e["out"] is None else depthwise._plan_for(plan_e["out"].shape, x.dtype, x.device)
    if packed is None or plan_d is None or plan_d["out"] is None:
        if opened is not None:  # the expansion's state already holds T: there is no way back
            raise RuntimeError("the layers of an open expansion lost their buffers before it was finished")
        return None
    done = hk.sparse_expand_depthwise(
        x, mask, packed, act_e.prev_out, act_e.out_truncated, DCThreshold.get(act_e), act_e.activation_int,
        plan_e["out"], plan_e["out_mask"], depthwise.weight, plan_d["g"], act_d.prev_out, act_d.out_truncated,
        DCThreshold.get(act_d), act_d.activation_int, act_d.truncation_mode.value, plan_d["out"], plan_d["out_mask"],
        opened=opened is not None)
    if not done:
        if opened is not None:
            raise RuntimeError("dc_expand_depthwise declined to finish an expansion that dc_project_expand left open")
        return None
    for conv in (expand, depthwise):
        DCConv2d.conv_idx += 1  # what the layers' own forward calls would have counted
        conv.frame_idx += 1
    return plan_d["out"], plan_d["out_mask"]


def fused_block(dw_input, depthwise, project, add=None, residual=None, expand=None):
    """One launch for ``depthwise`` (3x3 depthwise DCConv2d with activation) -> ``project`` (1x1
    DCConv2d without activation) [-> ``add(residual, .)``, a DCAdd without activation]
    [-> ``expand`` (1x1 DCConv2d with the same activation)], on frames after the first.

    Returns ``(block_output, expanded)`` -- two ``(delta, mask)`` tuples, ``expanded`` is None
    without ``expand`` -- exactly what the separate layer calls return, or ``None`` when the
    layers are not in a state or of a shape the kernel takes; nothing has happened then and the
    caller runs the layers one by one.  Switch: ``DCConv2d.fuse_blocks``."""
    if not DCConv2d.fuse_blocks or isinstance(dw_input, Tensor):
        return None
    if not (_steady(depthwise) and _steady(project) and (expand is None or _steady(expand))):
        return None
    act_a = _steady_activation(depthwise)
    if act_a is None or project.activation is not None or not _is_depthwise(depthwise):
        return None
    if add is not None and (add.first_iter or add.dense_out or add.activation is not None
                            or residual is None or isinstance(residual, Tensor)):
        return None
    act_c = None
    if expand is not None:
        act_c = _steady_activation(expand)
        if act_c is None or act_c.activation_int != act_a.activation_int:
            return None
    x, mask = dw_input
    if x.dtype != torch.float16 or depthwise.padding4 is not None:
        return None
    filter_bytes = 2 * project.out_channels * (project.in_channels + (expand.out_channels if expand is not None else 0))
    if filter_bytes > DCConv2d.fuse_blocks_max_filter_bytes:
        return None
    plan_a = depthwise._plan_for(x.shape, x.dtype, x.device)
    g = plan_a["g"]
    if g.batch * g.out_h * g.out_w > DCConv2d.fuse_blocks_max_pixels:
        return None
    hidden_shape = (g.batch, g.out_c, g.out_h, g.out_w)
    plan_b = project._plan_for(hidden_shape, x.dtype, x.device)
    if plan_b["out"] is None or (project.kernel_size, project.stride, project.padding) != ((1, 1), (1, 1), (0, 0)):
        return None
    out, out_mask = plan_b["out"], plan_b["out_mask"]
    res_delta = res_mask = None
    if add is not None:
        res_delta, res_mask = residual
        if tuple(res_delta.shape) != tuple(out.shape):
            return None
        if not _matches(add.out, res_delta):
            add.out = torch.empty_like(res_delta)
        if not _matches(add.mask_out, res_mask):
            add.mask_out = torch.empty_like(res_mask)
        out, out_mask = add.out, add.mask_out
    ex = None
    if expand is not None:
        plan_c = expand._plan_for(out.shape, x.dtype, x.device)
        if plan_c["out"] is None or (expand.kernel_size, expand.stride, expand.padding) != ((1, 1), (1, 1), (0, 0)):
            return None
        ex = (expand._packed_filter(), expand.out_channels, act_c.prev_out, act_c.out_truncated,
              DCThreshold.get(act_c), act_c.activation_int, plan_c["out"], plan_c["out_mask"])
    done = hk.sparse_block(x, mask, depthwise.weight, g, act_a.prev_out, act_a.out_truncated,
                           DCThreshold.get(act_a), act_a.activation_int, project._packed_filter(),
                           project.out_channels, out, out_mask, res_delta, res_mask,
                           add.weight_a if add is not None else 1.0, add.weight_b if add is not None else 1.0, ex)
    if not done:
        return None
    for conv in (depthwise, project) + ((expand,) if expand is not None else ()):
        DCConv2d.conv_idx += 1  # what the layers' own forward calls would have counted
        conv.frame_idx += 1
    return (out, out_mask), ((ex[6], ex[7]) if ex is not None else None)


def _group_ready(conv, input) -> bool:
    """A 16-bit delta convolution past its first frame (no bias any more) on a delta input."""
    return (DCConv2d.fuse_groups and isinstance(conv, DCConv2d) and conv.backend == DCBackend.deltacnn
            and conv.frame_idx >= 0 and conv.filters_processed and not conv.dense_out
            and conv.weight.dtype in (torch.float16, torch.bfloat16) and not isinstance(input, Tensor))


def _group_item(conv, input):
    """The convolution part of a dc_conv_group item, or None if the layer has no packed filter."""
    x, mask, plan, packed, _, _ = conv._prepare(input)
    if packed is None:
        return None, None
    g = plan["g"]
    return dict(x=x, mask=mask, packed_filter=packed, geometry=g), plan


def conv_group(convs, inputs):
    """``[conv(x) for conv, x in zip(convs, inputs)]`` for layers that do not depend on each other
    -- the same layer of several parallel branches -- as ONE launch (+ one for the activations the
    convolution kernel cannot finish) where ``dc_conv_group`` takes them; the separate layer calls
    otherwise.  Results are identical either way.  Switch: ``DCConv2d.fuse_groups``."""
    items, results = [], []
    ok = len(convs) >= 2 and all(_group_ready(c, x) for c, x in zip(convs, inputs))
    if ok:
        for conv, x in zip(convs, inputs):
            item, plan = _group_item(conv, x)
            act = conv.activation_layer
            if item is None or (conv.activation is not None and (_steady_activation(conv) is None
                                                                 or not DCConv2d.fuse_activation)):
                ok = False
                break
            g = plan["g"]
            out = plan["out"] if plan["out"] is not None else hk.new_features(
                g.batch, g.out_c, g.out_h, g.out_w, item["x"].dtype, item["x"].device)
            out_mask = plan["out_mask"] if plan["out_mask"] is not None else hk.new_mask(
                g.batch, g.out_h, g.out_w, item["x"].device)
            item.update(out=out, out_mask=out_mask)
            if act is not None:
                item["activation"] = (act.prev_out, act.out_truncated, DCThreshold.get(act), act.activation_int,
                                      act.truncation_mode.value)
            items.append(item)
            results.append((out, out_mask))
    if ok and hk.sparse_conv_group(items):
        for conv in convs:
            DCConv2d.conv_idx += 1
            conv.frame_idx += 1
        return results
    return [conv(x) for conv, x in zip(convs, inputs)]


def residual_group(adds, residuals, convs, conv_inputs):
    """``[add(r, conv(x)) for ...]`` for independent (DCAdd, residual, convolution without
    activation, input) quadruples -- the block ends of several parallel branches -- as ONE
    launch where ``dc_conv_group`` takes them; ``add.after_conv`` per branch otherwise.  Results
    are identical either way.  Switch: ``DCConv2d.fuse_groups``."""
    items, results = [], []
    ok = len(convs) >= 2 and DCAdd.fuse_into_conv and all(
        _group_ready(c, x) and c.activation is None and not isinstance(r, Tensor) and not a.first_iter
        and not a.dense_out for a, r, c, x in zip(adds, residuals, convs, conv_inputs))
    if ok:
        for add, res, conv, x in zip(adds, residuals, convs, conv_inputs):
            item, plan = _group_item(conv, x)
            val, mask = res
            g = plan["g"] if plan is not None else None
            if item is None or tuple(val.shape) != (g.batch, g.out_c, g.out_h, g.out_w):
                ok = False
                break
            if not _matches(add.out, val):
                add.out = torch.empty_like(val)
            if not _matches(add.mask_out, mask):
                add.mask_out = torch.empty_like(mask)
            with_act = add.activation is not None
            item.update(out=add.out, out_mask=add.mask_out,
                        residual=(val, mask, add.weight_a, add.weight_b, add.prev_out if with_act else None,
                                  add.activation_int if with_act else 0))
            items.append(item)
            results.append((add.out, add.mask_out))
    if ok and hk.sparse_conv_group(items):
        for conv in convs:
            DCConv2d.conv_idx += 1
            conv.frame_idx += 1
        return results
    return [a.after_conv(r, c, x) for a, r, c, x in zip(adds, residuals, convs, conv_inputs)]


def add_group(adds, firsts, seconds, upsamples):
    """``[add(a, b) if up is None else add.after_upsample(a, b, up) for ...]`` for DCAdd layers
    that do not depend on each other -- the sums of one level of a multi-resolution exchange -- as
    ONE launch where ``dc_add_group`` takes them; the separate layer calls otherwise.  Results are
    identical either way.  Switch: ``DCConv2d.fuse_groups``."""
    def separate():
        return [add(a, b) if up is None else add.after_upsample(a, b, up)
                for add, a, b, up in zip(adds, firsts, seconds, upsamples)]
    ok = (DCConv2d.fuse_groups and len(adds) >= 2 and DCAdd.fuse_into_conv
          and all(not isinstance(a, Tensor) and not isinstance(b, Tensor) and not add.first_iter and not add.dense_out
                  and (up is None or isinstance(up, DCUpsamplingNearest2d))
                  for add, a, b, up in zip(adds, firsts, seconds, upsamples)))
    if not ok:
        return separate()
    items, results = [], []
    for add, (val_a, mask_a), (val_b, mask_b), up in zip(adds, firsts, seconds, upsamples):
        if not _matches(add.out, val_a):
            add.out = torch.empty_like(val_a)
        if not _matches(add.mask_out, mask_a):
            add.mask_out = torch.empty_like(mask_a)
        with_act = add.activation is not None
        items.append((val_a, val_b, add.prev_out if with_act else None, add.out, mask_a, mask_b, add.mask_out,
                      add.weight_a, add.weight_b, add.activation_int if with_act else 0,
                      1 if up is None else up.scale_factor))
        results.append((add.out, add.mask_out))
    return results if hk.sparse_add_group(items) else separate()


class DCConcatenate(DCModule):
    """Channel concatenation of two delta tensors (sparse_layers.py:1185-1194)."""
    fuse_into_conv = True  # a 1x1 convolution behind a chain of concatenations reads the tensors where they lie

    def __init__(self, name=""):
        super().__init__()
        self.name = name
        self.out = None

    def forward(self, a, b):
        if type(a) == Tensor:
            return torch.cat((a, b), dim=1)
        if not DCModule.reuse_buffers:
            return hk.sparse_concatenate(a, b)
        if self.out is not None and (self.out[0].shape[0] != a[0].shape[0]
                                     or self.out[0].shape[2:] != a[0].shape[2:]
                                     or self.out[0].dtype != a[0].dtype):
            self.out = None
        self.out = hk.sparse_concatenate(a, b, self.out)
        return self.out

    def reset(self):
        super().reset()
        self.out = None


class DCSparsify(DCModule):
    """Dense frame -> (delta, mask) against the cached accumulated input
    (sparse_layers.py:1197-1273).  With ``dilation > 1`` the per-pixel test is replaced by a
    torch expression over a dilation x dilation neighbourhood (:1233-1244)."""
    idx = -1

    def __init__(self, name="", delta_threshold=None, dilation=-1):
        super().__init__()
        self.name = name
        self.dilation = dilation
        self.delta_threshold = DCThreshold.t_default if delta_threshold is None else delta_threshold
        self._forget()

    def _forget(self):
        self.idx = -1
        self.frame_idx = -1
        self.prev_in = None
        self.mask = None
        self.delta = None

    def _first_frame(self, frame):
        """Everything is new: the frame itself is the delta, every pixel is active."""
        DCThreshold.set(self, self.delta_threshold)
        self._take_index(DCSparsify)
        self.prev_in = self._cache(frame.clone())
        b, _, h, w = frame.shape
        return frame, torch.ones((b, 1, h, w), dtype=torch.int32, device=frame.device)

    def _neighbourhood_delta(self, frame, threshold):
        k = self.dilation
        delta = frame - self.prev_in
        peak = F.max_pool2d(delta.abs().amax(dim=1, keepdim=True), k, stride=1, padding=(k - 1) // 2)
        active = peak > threshold
        self.prev_in = torch.where(active, frame, self.prev_in)
        return delta, active.to(torch.int32)

    def forward(self, input):
        if DCConv2d.backend != DCBackend.deltacnn:
            return input
        self.frame_idx += 1
        if self.idx < 0:
            return self._first_frame(input)
        threshold = DCThreshold.get(self)
        if self.dilation > 1:
            return self._neighbourhood_delta(input, threshold)
        b, _, h, w = input.shape
        if self.mask is None or self.mask.shape != (b, 1, h, w) or self.mask.device != input.device:
            self.mask = hk.new_mask(b, h, w, input.device)
        if not DCModule.reuse_buffers:
            delta = torch.empty_like(input)
        else:
            if not _matches(self.delta, input):
                self.delta = torch.empty_like(input)
            delta = self.delta
        hk.sparsify(input, self.prev_in, delta, self.mask, threshold)
        return delta, self.mask

    def reset(self):
        super().reset()
        self._forget()
        DCSparsify.idx = -1


class DCDensify(DCModule):
    """(delta, mask) -> dense accumulated tensor (sparse_layers.py:1276-1333).  With
    ``clone_out`` (default) every call returns a NEW tensor, so results collected over frames
    stay distinct; ``clone_out=False`` returns the accumulator itself."""
    idx = -1
    fuse_pooling = True  # pooled_dense(): a preceding global average pooling joins the launch

    def __init__(self, activation: str = None, name="", clone_out=True):
        super().__init__()
        self.name = name
        self.activation, self.activation_int = convert_activation_string(activation)
        self.clone_out = clone_out
        self.prev_out = None
        self.idx = -1

    def forward(self, input):
        if isinstance(input, Tensor):
            return input
        delta, mask = input
        if self.prev_out is None or not _matches(self.prev_out, delta):
            if self.prev_out is None:
                self._take_index(DCDensify)
            self.prev_out = self._cache(torch.zeros_like(delta))  # bias arrives with the frame-0 delta
        if self.clone_out:
            dense = torch.empty_like(self.prev_out)
            hk.densify(delta, self.prev_out, dense, mask)  # accumulate and copy in one launch
        else:
            hk.sparse_activation(delta, self.prev_out, None, mask, -1, -1, DCTruncation.none.value)
            dense = self.prev_out
        return dense if self.activation is None else self.activation(dense)

    def reset(self):
        super().reset()
        self.prev_out = None


def pooled_dense(pool, densify, input):
    """``densify(pool(input))`` for a global average pooling followed by a DCDensify, in one
    launch on frames after the first: the pooled delta goes straight into the densify layer's
    accumulator and never exists in memory.  Returns the dense ``[B, C, 1, 1]`` tensor (a new
    tensor per call, as DCDensify returns), or ``None`` when the layers are not in a state or
    of a shape the kernel takes; nothing has happened then and the caller runs the two layers.
    Switch: ``DCDensify.fuse_pooling``."""
    if not DCDensify.fuse_pooling or isinstance(input, Tensor):
        return None
    if not isinstance(pool, DCAdaptiveAveragePooling) or tuple(pool.output_size) != (1, 1):
        return None
    if not isinstance(densify, DCDensify) or densify.activation is not None or not densify.clone_out:
        return None
    delta, mask = input
    acc = densify.prev_out
    if (acc is None or tuple(acc.shape) != (delta.shape[0], delta.shape[1], 1, 1) or acc.dtype != delta.dtype
            or acc.device != delta.device):
        return None
    dense = torch.empty_like(acc)
    if not hk.pooled_densify(delta, mask, acc, dense):
        return None
    pool.first_iter = False
    return dense


class Linear(nn.Linear):
    """torch.nn.Linear (same parameters, same state dict) whose forward runs the library's
    dense-layer kernel on a few rows of a GPU tensor -- the classifier behind DCDensify, which
    the reference leaves to torch (example/mobilenet_deltacnn.py:196-199, 225) and which a GEMM
    library serves with several launch latencies at one row per stream.  Everything else
    (CPU tensors, training, more than ``max_rows`` rows, feature counts that do not fill 16-byte
    vectors) goes to torch.  Switch: ``Linear.use_library``."""
    use_library = True
    max_rows = 64

    def forward(self, input):
        w = self.weight
        if (Linear.use_library and input.is_cuda and input.dim() == 2 and input.dtype == w.dtype
                and input.dtype in (torch.float16, torch.bfloat16, torch.float32)
                and input.shape[0] <= Linear.max_rows and input.shape[1] % (16 // input.element_size()) == 0
                and not (torch.is_grad_enabled() and (input.requires_grad or w.requires_grad))):
            return hk.linear(input.contiguous(), w.contiguous(), self.bias)
        return F.linear(input, w, self.bias)


class DCUpsamplingNearest2d(DCModule):
    """Nearest upsampling by an integer factor (sparse_layers.py:1336-1359): an updated pixel
    updates its scale x scale copies."""
    idx = -1

    def __init__(self, scale_factor=2, name=""):
        super().__init__()
        self.scale_factor = int(scale_factor)
        self.torch_upsample = nn.UpsamplingNearest2d(scale_factor=scale_factor)
        self.name = name
        self.idx = -1
        self.out = None

    def forward(self, input):
        if isinstance(input, Tensor):
            return self.torch_upsample(input)
        delta, mask = input
        b, c, h, w = delta.shape
        k = self.scale_factor
        if self.out is not None:
            have = self.out[0]
            if have.shape != (b, c, h * k, w * k) or have.dtype != delta.dtype or have.device != delta.device:
                self.out = None
        self.out = hk.sparse_upsample(delta, mask, k, self.out)
        return self.out

    def reset(self):
        super().reset()
        self.out = None


class DCActivation(DCModule):
    """Non-linearity on accumulated values with truncation of small updates
    (sparse_layers.py:1362-1425).  State: ``prev_out`` = accumulated pre-activation values,
    ``out_truncated`` = updates withheld so far."""
    idx = -1
    truncation_default = DCTruncation.max

    def __init__(self, name="", inplace=True, delta_threshold=None, activation="relu",
                 truncation_mode: DCTruncation = None):
        super().__init__()
        self.activation, self.activation_int = convert_activation_string(activation)
        if self.activation is None:
            raise ValueError("DCActivation needs a non-linear activation")
        self.name = name
        self.inplace = inplace
        self.delta_threshold = DCThreshold.t_default if delta_threshold is None else delta_threshold
        self.truncation_mode = DCActivation.truncation_default if truncation_mode is None else truncation_mode
        self.idx = -1
        self._forget()

    def _forget(self):
        self.first_iter = True
        self.prev_out = None
        self.out_truncated = None

    def _first_frame(self, values, mask):
        """Dense frame: remember the pre-activation values, nothing withheld yet; the mask
        passes through untouched."""
        self.first_iter = False
        DCThreshold.set(self, self.delta_threshold)
        if self.idx < 0:
            self._take_index(DCActivation)
        self.prev_out = self._cache(values.clone())
        self.out_truncated = self._cache(torch.zeros_like(values))
        return self.activation(values), mask

    def forward(self, input):
        if isinstance(input, Tensor):
            return self.activation(input)
        values, mask = input
        if self.first_iter:
            return self._first_frame(values, mask)
        if not self.inplace:
            values, mask = values.clone(), mask.clone()
        hk.sparse_activation(values, self.prev_out, self.out_truncated, mask, DCThreshold.get(self),
                             self.activation_int, self.truncation_mode.value)
        return values, mask

    def reset(self):
        super().reset()
        self.idx = -1
        self._forget()
        DCActivation.idx = -1


class DCMaxPooling(nn.MaxPool2d, DCModule):
    """Delta max pooling; caches the accumulated input (sparse_layers.py:1428-1474).
    ``padding`` may be a pair or (left, right, top, bottom) as torch.nn.functional.pad takes it
    (:1439-1441)."""

    fuse_cache_update = True  # windows that tile the map: pooling and cache update in one launch

    def __init__(self, kernel_size, stride=(1, 1), padding=(0, 0), dilation=(1, 1)):
        kernel_size, stride, padding, dilation = to_tuple(kernel_size, stride, padding, dilation)
        nn.MaxPool2d.__init__(self, kernel_size, stride=stride, padding=padding, dilation=dilation)
        self.out_shape = []
        self.first_iter = True
        self.prev_in = None

    def _dense(self, x):
        """Plain tensors: torch pooling; four-sided padding is applied beforehand (zeros, as the
        reference pads) and the window then runs unpadded."""
        pad = self.padding
        if len(pad) == 4:
            x, pad = F.pad(x, pad), 0
        return F.max_pool2d(x, self.kernel_size, self.stride, pad, self.dilation, self.ceil_mode)

    def forward(self, input):
        if isinstance(input, Tensor):
            return self._dense(input)
        delta, mask = input
        if self.first_iter:
            self.first_iter = False
            self.prev_in = self._cache(torch.zeros_like(delta))
        if (DCMaxPooling.fuse_cache_update and tuple(self.kernel_size) == tuple(self.stride) and not any(self.padding)
                and tuple(self.dilation) == (1, 1)):
            pooled = hk.sparse_max_pooling_update(delta, self.prev_in, self.kernel_size, mask, self.stride)
            if pooled is not None:  # the pooling kernel has moved the cache along as well
                return pooled
        pooled = hk.sparse_pooling(delta, self.prev_in, self.kernel_size, mask, self.stride, self.padding,
                                   self.dilation, create_out_mask=True, pooling_mode_int=0)
        hk.sparse_add_to_dense_tensor(delta, self.prev_in, mask)  # the cache follows the input
        return pooled

    def reset(self):
        DCModule.reset(self)
        self.first_iter = True
        self.prev_in = None


class DCAdaptiveAveragePooling(nn.AdaptiveAvgPool2d, DCModule):
    """Global average pooling of deltas (sparse_layers.py:1477-1513): the mean is linear, so the
    delta of the mean is the mean of the deltas and no cache is needed.  Output size 1x1 only."""

    def __init__(self, output_size=None):
        output_size = to_tuple(output_size)
        nn.AdaptiveAvgPool2d.__init__(self, output_size=output_size)
        self.out_shape = output_size
        self.first_iter = True
        self.prev_in = None

    def get_target_size(self, input):
        """(window, stride, padding, dilation) of the pooling call that produces one pixel."""
        if tuple(self.output_size) != (1, 1):
            raise AssertionError("only output_size 1x1 is supported on delta tensors")
        return tuple(input.shape[2:]), (1, 1), (0, 0), (1, 1)

    def forward(self, input):
        if isinstance(input, Tensor):
            return nn.AdaptiveAvgPool2d.forward(self, input)
        delta, mask = input
        self.first_iter = False
        window, stride, padding, dilation = self.get_target_size(delta)
        return hk.sparse_pooling(delta, None, window, mask, stride, padding, dilation,
                                 create_out_mask=True, pooling_mode_int=1)

    def reset(self):
        DCModule.reset(self)
        self.first_iter = True
        self.prev_in = None


class DCBatchNorm2d(nn.BatchNorm2d, DCModule):
    """Inference batch norm on deltas (sparse_layers.py:1516-1585).  y = x * scale + offset is
    affine: a delta only needs the scale, the offset enters once with the first frame (and on
    every dense tensor)."""

    def __init__(self, num_features, eps=1e-5, momentum=0.1, affine=True,
                 track_running_stats=True, inplace=True):
        nn.BatchNorm2d.__init__(self, num_features, eps, momentum, affine, track_running_stats)
        self.inplace = inplace
        self.first_iter = True
        self.scale = self.offset = None

    def convert_to_scale_offset(self, input=None):
        """Fold running statistics and affine parameters into per-channel scale and offset,
        shaped [1, C, 1, 1]."""
        inv_std = torch.rsqrt(self.running_var + self.eps)
        gain = self.weight * inv_std
        shift = self.bias - self.running_mean * gain
        self.scale, self.offset = gain.view(1, -1, 1, 1), shift.view(1, -1, 1, 1)

    def forward(self, input):
        is_delta = isinstance(input, tuple)
        first, self.first_iter = self.first_iter, False
        if first:
            self.convert_to_scale_offset()
        with_offset = first or not is_delta
        if not is_delta:
            out = input.mul_(self.scale) if self.inplace else input * self.scale
            return out.add_(self.offset) if with_offset else out
        delta, mask = input
        shift = self.offset if with_offset else None
        if self.inplace:
            out, out_mask = delta, mask
        else:
            out, out_mask = torch.empty_like(delta), mask.clone()
        hk.sparse_mul_add(delta, mask, out, out_mask, self.scale, shift)
        return out, out_mask

    def reset(self):
        DCModule.reset(self)
        self.first_iter = True
