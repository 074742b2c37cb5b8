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


class DCBackend(Enum):
    cudnn = 0
    deltacnn = 1
    delta_cudnn = 2

    @classmethod
    def parse_string(cls, x):
        try:
            return cls[x.lower()]
        except KeyError:
            raise Exception(f"invalid backend {x}")


class DCTruncation(Enum):
    none = -1
    max = 0
    norm = 1
    rms = 2

    @classmethod
    def parse_string(cls, x):
        try:
            return cls[x.lower()]
        except KeyError:
            raise Exception(f"invalid truncation mode {x}")


class DCThreshold:
    """Registry of per-layer thresholds keyed by module (sparse_layers.py:122-208).

    Layers register their threshold on their first frame and look it up on every later
    frame, so a JSON file loaded after frame 0 overrides the defaults.
    """
    t_default = 0.0
    t = OrderedDict()
    path = None
    initialized = False
    scale = 1.0

    @classmethod
    def get(cls, key, default=0.0):
        return cls.t.get(key, default)

    @classmethod
    def set(cls, key, val):
        if key not in cls.t:
            cls.t[key] = val

    @classmethod
    def load_thresholds(cls):
        if cls.initialized:
            return
        cls.initialized = True
        if cls.path is None:
            return
        with open(cls.path) as f:
            thresholds = json.load(f)
        if len(thresholds) != len(cls.t):
            print(f"WARNING: thresholds file contains different number of thresholds. "
                  f"file: {len(thresholds)} expected {len(cls.t)}")
        skip = len(cls.t) - len(thresholds)
        for i, key in enumerate(cls.t.keys()):
            if i >= skip:
                cls.t[key] = thresholds[str(i - skip)] * cls.scale

    @classmethod
    def save_thresholds(cls, name):
        with open(f"thresholds_{name}.json", "w+") as f:
            json.dump({i: v for i, v in enumerate(cls.t.values())}, f)

    @classmethod
    def reset(cls):
        cls.t.clear()
        cls.initialized = False
        cls.path = None


class DCModule(nn.Module):
    temp_buffers = []
    # Layers keep their output / mask buffers between frames instead of allocating per call
    # (the reference allocates with torch.empty on every call, cuda_kernels.py:34-37).  A
    # returned delta tensor is therefore valid until the same layer runs its next frame.
    reuse_buffers = True

    def __init__(self):
        super().__init__()

    @classmethod
    def get_temp_buffer_numel(cls):
        return sum(x.numel() for x in cls.temp_buffers)

    def reset(self):
        DCModule.temp_buffers = []

    def process_filters(self):
        for mod in list(self.modules()):
            if type(mod) in [DCConv2d, DCConvTranspose2d]:
                mod.process_filters()

    def reset_layers(self):
        for module in self.modules():
            if module is not self and isinstance(module, DCModule):
                module.reset()
        DCModule.temp_buffers.clear()


def to_tuple(*args):
    result = []
    for x in args:
        if type(x) == int:
            result.append((x, x))
        elif len(x) == 1:
            result.append((x[0], x[0]))
        else:
            result.append(tuple(x))
    return result[0] if len(result) == 1 else result


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
        self.conv_idx = DCConv2d.conv_idx
        self.dense_in = type(input) == Tensor
        self.in_shape = input.shape if type(input) == Tensor else input[0].shape
        if self.activation is not None and self.backend != DCBackend.cudnn:
            DCThreshold.set(self, self.delta_threshold)

    def forward(self, input):
        DCConv2d.conv_idx += 1
        self.frame_idx += 1
        first_iter = self.conv_idx == -1
        if first_iter:
            self.init_first_iter(input)
        if self.backend == DCBackend.cudnn:
            return self._forward_dense(input)
        if self.backend == DCBackend.delta_cudnn:
            raise NotImplementedError("the delta_cudnn training backend is not part of this package")
        return self._forward_delta_conv(input, first_iter)

    def _forward_dense(self, input):
        out = self._conv_forward_dense(input)
        return self.activation(out) if self.activation is not None else out

    def _make_plan(self, x):
        pad = self.padding4 if getattr(self, "padding4", None) is not None else self.padding
        w = self.weight
        g = hk.conv_geometry(x.shape, (w.shape[1], w.shape[2]), self.out_channels, self.stride, pad,
                             self.dilation, self.groups, self._transposed)
        plan = {"shape": tuple(x.shape), "dtype": x.dtype, "g": g, "out": None, "out_mask": None}
        if DCModule.reuse_buffers:
            plan["out"] = hk.new_features(g.batch, g.out_c, g.out_h, g.out_w, x.dtype, x.device)
            plan["out_mask"] = hk.new_mask(g.batch, g.out_h, g.out_w, x.device)
        return plan

    def _prepare(self, input):
        if type(input) == Tensor:
            raise TypeError("the deltacnn backend propagates (delta, mask) tuples: put a "
                            "DCSparsify in front of the first convolution")
        if not self.filters_processed:
            raise RuntimeError("call process_filters() on the model (after moving it to the GPU "
                               "in channels_last) before the first frame")
        x, mask = input
        if self._plan is None or self._plan["shape"] != tuple(x.shape) or self._plan["dtype"] != x.dtype:
            self._plan = self._make_plan(x)
            self.in_shape = x.shape
        if self._packed is None:
            self._packed = hk.pack_filter(self.weight.data, self.in_channels, self.out_channels,
                                          self.groups, self._transposed)
            if self._packed is None:
                self._packed = False
        packed = self._packed if self._packed is not False else None
        bias = self.bias if self.frame_idx <= 0 else None
        pad = self.padding4 if getattr(self, "padding4", None) is not None else self.padding
        return x, mask, self._plan, packed, bias, pad

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
        self.frame_idx = -1
        self.conv_idx = -1
        self.prev_out = None
        self.prev_in = None
        self.out_shape = []
        DCConv2d.conv_idx = -1

    def process_filters_half(self):
        self.orig_weights = self.weight.data.clone()
        result = self.half()
        if self.backend == DCBackend.deltacnn:
            result.weight.data = convert_half_filter(result.weight.data, pixel_wise=_is_depthwise(self),
                                                     transposed=self._transposed)
            self.filters_processed = True
            self._packed = None
        return result

    def process_filters_single(self):
        self.orig_weights = self.weight.data.clone()
        if self.backend == DCBackend.deltacnn:
            self.weight.data = convert_filter_out_channels_last(self.weight.data,
                                                                transposed=self._transposed)
            self.filters_processed = True
            self._packed = None
        return self

    def process_filters(self):
        if self.filters_processed:
            return
        if self.weight.data.dtype == torch.float16:
            self.process_filters_half()
        else:
            self.process_filters_single()


class DCConv2d(_DeltaConvBase, nn.Conv2d, DCModule):
    """Delta convolution (sparse_layers.py:261-675)."""
    backend = DCBackend.deltacnn
    conv_idx = -1
    fuse_activation = True

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
    """Sum of two delta tensors with union mask (sparse_layers.py:1086-1182)."""
    idx = -1
    fuse_into_conv = True

    def __init__(self, activation: str = None, dense_out=False, weight_a=None, weight_b=None, name=""):
        super().__init__()
        self.name = name
        self.dense_out = dense_out
        self.activation, self.activation_int = convert_activation_string(activation)
        self.idx = -1
        self.prev_out = None
        self.mask_out = None
        self.out = None
        self.weight_a = 1.0 if weight_a is None else weight_a
        self.weight_b = 1.0 if weight_b is None else weight_b
        self.first_iter = True

    def forward(self, a, b, weight_a=None, weight_b=None):
        w_a = self.weight_a if weight_a is None else weight_a
        w_b = self.weight_b if weight_b is None else weight_b
        if type(a) == Tensor:
            c = w_a * a + w_b * b
            return self.activation(c) if self.activation is not None else c
        val_a, mask_a = a
        val_b, mask_b = b
        if self.first_iter:
            self.first_iter = False
            DCAdd.idx += 1
            self.idx = DCAdd.idx
            if self.dense_out or self.activation is not None:
                self.prev_out = torch.zeros_like(val_a)
                DCModule.temp_buffers.append(self.prev_out)
        if self.mask_out is None or self.mask_out.shape != mask_a.shape:
            self.mask_out = torch.empty_like(mask_a)
        if DCModule.reuse_buffers and not self.dense_out:
            if self.out is None or self.out.shape != val_a.shape or self.out.dtype != val_a.dtype:
                self.out = torch.empty_like(val_a)
            out = self.out
        else:
            out = torch.empty_like(val_a)
        mask_out = self.mask_out if DCModule.reuse_buffers else torch.empty_like(mask_a)
        hk.sparse_add_tensors(val_a, val_b, self.prev_out, out, mask_a, mask_b, mask_out, w_a, w_b,
                              self.activation_int, self.dense_out)
        if self.dense_out:
            return out
        return out, mask_out

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
                if self.out is None or self.out.shape != val_a.shape or self.out.dtype != val_a.dtype:
                    self.out = torch.empty_like(val_a)
                if self.mask_out is None or self.mask_out.shape != mask_a.shape:
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
        if self.out is None or self.out.shape != val_a.shape or self.out.dtype != val_a.dtype:
            self.out = torch.empty_like(val_a)
        if self.mask_out is None or self.mask_out.shape != mask_a.shape:
            self.mask_out = torch.empty_like(mask_a)
        hk.sparse_add_upsampled(val_a, val_b, self.prev_out if self.activation is not None else None, self.out,
                                mask_a, mask_b, self.mask_out, self.weight_a, self.weight_b,
                                self.activation_int if self.activation is not None else 0, upsample.scale_factor)
        return self.out, self.mask_out

    def reset(self):
        super().reset()
        self.idx = -1
        self.mask_out = None
        self.out = None
        self.prev_out = None
        self.first_iter = True
        DCAdd.idx = -1


class DCConcatenate(DCModule):
    """Channel concatenation of two delta tensors (sparse_layers.py:1185-1194)."""

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
    (sparse_layers.py:1197-1273)."""
    idx = -1

    def __init__(self, name="", delta_threshold=None, dilation=-1):
        super().__init__()
        self.name = name
        self.prev_in = None
        self.idx = -1
        self.delta_threshold = delta_threshold if delta_threshold is not None else DCThreshold.t_default
        self.dilation = dilation
        self.frame_idx = -1
        self.mask = None
        self.delta = None

    def forward(self, input):
        if DCConv2d.backend != DCBackend.deltacnn:
            return input
        first_iter = self.idx == -1
        self.frame_idx += 1
        if first_iter:
            if self not in DCThreshold.t:
                DCThreshold.set(self, self.delta_threshold)
            DCSparsify.idx += 1
            self.idx = DCSparsify.idx
            self.prev_in = input.clone()
            DCModule.temp_buffers.append(self.prev_in)
            return input, torch.ones_like(input[:, :1], dtype=torch.int)
        threshold = DCThreshold.get(self)
        if self.dilation > 1:
            x = input - self.prev_in
            mask = torch.max(torch.abs(x), dim=1, keepdim=True)[0]
            k = self.dilation
            mask = torch.max_pool2d(mask, (k, k), stride=(1, 1), padding=((k - 1) // 2, (k - 1) // 2)) > threshold
            self.prev_in = torch.where(mask, input, self.prev_in)
            return x, mask.int()
        if self.mask is None or self.mask.shape[2:] != input.shape[2:] or self.mask.shape[0] != input.shape[0]:
            self.mask = torch.empty_like(input[:, :1], dtype=torch.int)
        if DCModule.reuse_buffers:
            if self.delta is None or self.delta.shape != input.shape or self.delta.dtype != input.dtype:
                self.delta = torch.empty_like(input)
            x = self.delta
        else:
            x = torch.empty_like(input)
        hk.sparsify(input, self.prev_in, x, self.mask, threshold)
        return x, self.mask

    def reset(self):
        super().reset()
        self.idx = -1
        self.frame_idx = -1
        self.prev_in = None
        self.mask = None
        self.delta = None
        DCSparsify.idx = -1


class DCDensify(DCModule):
    """(delta, mask) -> dense accumulated tensor (sparse_layers.py:1276-1333)."""
    idx = -1

    def __init__(self, activation: str = None, name="", clone_out=True):
        super().__init__()
        self.name = name
        self.activation, self.activation_int = convert_activation_string(activation)
        self.prev_out = None
        self.out = None
        self.idx = -1
        self.clone_out = clone_out

    def forward(self, input):
        if type(input) == Tensor:
            return input
        input, mask = input
        if self.prev_out is None:
            DCDensify.idx += 1
            self.idx = DCDensify.idx
            self.prev_out = torch.zeros_like(input)
            DCModule.temp_buffers.append(self.prev_out)
        if self.clone_out:  # accumulate and copy in one launch
            out = self.out if DCModule.reuse_buffers and self.out is not None else torch.empty_like(self.prev_out)
            if DCModule.reuse_buffers:
                self.out = out
            hk.densify(input, self.prev_out, out, mask)
        else:
            hk.sparse_activation(input, self.prev_out, None, mask, -1, -1, DCTruncation.none.value)
            out = self.prev_out
        if self.activation is not None:
            return self.activation(out)
        return out

    def reset(self):
        super().reset()
        self.prev_out = None
        self.out = None


class DCUpsamplingNearest2d(DCModule):
    """Nearest upsampling by an integer factor (sparse_layers.py:1336-1359)."""
    idx = -1

    def __init__(self, scale_factor=2, name=""):
        super().__init__()
        self.name = name
        self.scale_factor = int(scale_factor)
        self.idx = -1
        self.out = None
        self.torch_upsample = nn.UpsamplingNearest2d(scale_factor=scale_factor)

    def forward(self, input):
        if type(input) == Tensor:
            return self.torch_upsample(input)
        val, mask = input
        if self.out is not None and (self.out[0].shape[0] != val.shape[0]
                                     or self.out[0].shape[1] != val.shape[1]
                                     or self.out[0].shape[2] != val.shape[2] * self.scale_factor
                                     or self.out[0].shape[3] != val.shape[3] * self.scale_factor
                                     or self.out[0].dtype != val.dtype):
            self.out = None
        self.out = hk.sparse_upsample(val, mask, self.scale_factor, self.out)
        return self.out

    def reset(self):
        super().reset()
        self.out = None


class DCActivation(DCModule):
    """Non-linearity on accumulated values with truncation of small updates
    (sparse_layers.py:1362-1425)."""
    idx = -1
    truncation_default = DCTruncation.max

    def __init__(self, name="", inplace=True, delta_threshold=None, activation="relu",
                 truncation_mode: DCTruncation = None):
        super().__init__()
        self.name = name
        self.idx = -1
        self.prev_out = None
        self.inplace = inplace
        self.out_truncated = None
        self.activation, self.activation_int = convert_activation_string(activation)
        if self.activation is None:
            raise ValueError("DCActivation needs a non-linear activation")
        self.delta_threshold = delta_threshold if delta_threshold is not None else DCThreshold.t_default
        self.first_iter = True
        self.truncation_mode = truncation_mode if truncation_mode is not None else DCActivation.truncation_default

    def forward(self, input):
        if type(input) == Tensor:
            return self.activation(input)
        val, mask = input
        if self.first_iter:
            self.first_iter = False
            if self not in DCThreshold.t:
                DCThreshold.set(self, self.delta_threshold)
            if self.idx < 0:
                DCActivation.idx += 1
                self.idx = DCActivation.idx
            self.prev_out = val.clone()
            self.out_truncated = torch.zeros_like(val)
            DCModule.temp_buffers.append(self.prev_out)
            DCModule.temp_buffers.append(self.out_truncated)
            return self.activation(val), mask
        threshold = DCThreshold.get(self)
        if not self.inplace:
            val = val.clone()
            mask = mask.clone()
        hk.sparse_activation(val, self.prev_out, self.out_truncated, mask, threshold,
                             self.activation_int, self.truncation_mode.value)
        return val, mask

    def reset(self):
        super().reset()
        self.idx = -1
        self.prev_out = None
        self.out_truncated = None
        self.first_iter = True
        DCActivation.idx = -1


class DCMaxPooling(nn.MaxPool2d, DCModule):
    """Delta max pooling; caches the accumulated input (sparse_layers.py:1428-1474)."""

    def __init__(self, kernel_size, stride=(1, 1), padding=(0, 0), dilation=(1, 1)):
        kernel_size, stride, padding, dilation = to_tuple(kernel_size, stride, padding, dilation)
        nn.MaxPool2d.__init__(self, kernel_size, stride=stride, padding=padding, dilation=dilation)
        self.first_iter = True
        self.out_shape = []
        self.prev_in = None

    def forward(self, input):
        if type(input) == Tensor:
            old_padding = self.padding
            if len(self.padding) == 4:
                input = torch.nn.functional.pad(input, self.padding)
                self.padding = 0
            out = nn.MaxPool2d.forward(self, input)
            self.padding = old_padding
            return out
        x, mask = input
        if self.first_iter:
            self.first_iter = False
            self.prev_in = torch.zeros_like(x)
            DCModule.temp_buffers.append(self.prev_in)
        out = hk.sparse_pooling(x, self.prev_in, self.kernel_size, mask, self.stride, self.padding,
                                self.dilation, create_out_mask=True, pooling_mode_int=0)
        hk.sparse_add_to_dense_tensor(x, self.prev_in, mask)
        return out

    def reset(self):
        DCModule.reset(self)
        self.first_iter = True
        self.prev_in = None


class DCAdaptiveAveragePooling(nn.AdaptiveAvgPool2d, DCModule):
    """Global average pooling of deltas (sparse_layers.py:1477-1513); output size 1x1 only."""

    def __init__(self, output_size=None):
        output_size = to_tuple(output_size)
        nn.AdaptiveAvgPool2d.__init__(self, output_size=output_size)
        self.first_iter = True
        self.out_shape = output_size
        self.prev_in = None

    def get_target_size(self, input):
        assert self.output_size[0] == 1 and self.output_size[1] == 1
        return tuple(input.shape[2:]), (1, 1), (0, 0), (1, 1)

    def forward(self, input):
        if type(input) == Tensor:
            return nn.AdaptiveAvgPool2d.forward(self, input)
        x, mask = input
        self.first_iter = False
        kernel_size, stride, padding, dilation = self.get_target_size(x)
        return hk.sparse_pooling(x, None, kernel_size, mask, stride, padding, dilation,
                                 create_out_mask=True, pooling_mode_int=1)

    def reset(self):
        DCModule.reset(self)
        self.first_iter = True
        self.prev_in = None


class DCBatchNorm2d(nn.BatchNorm2d, DCModule):
    """Inference batch norm on deltas: scale on every frame, offset on the first only
    (sparse_layers.py:1516-1585)."""

    def __init__(self, num_features, eps=1e-5, momentum=0.1, affine=True,
                 track_running_stats=True, inplace=True):
        nn.BatchNorm2d.__init__(self, num_features, eps, momentum, affine, track_running_stats)
        self.first_iter = True
        self.scale = None
        self.offset = None
        self.inplace = inplace

    def convert_to_scale_offset(self, input):
        bn_scale = self.weight * torch.rsqrt(self.running_var + self.eps)
        self.scale = bn_scale[None, :, None, None]
        self.offset = (-self.running_mean * bn_scale + self.bias)[None, :, None, None]

    def forward(self, input):
        use_offset = False
        mask = None
        dense = True
        if type(input) == tuple:
            input, mask = input
            dense = False
        else:
            use_offset = True
        if self.first_iter:
            self.first_iter = False
            use_offset = True
            self.convert_to_scale_offset(input)
        if dense:
            out = input.mul_(self.scale) if self.inplace else input * self.scale
            if use_offset:
                out.add_(self.offset)
            return out
        bias = self.offset if use_offset else None
        if self.inplace:
            hk.sparse_mul_add(input, mask, input, mask, self.scale, bias)
            return input, mask
        out = torch.empty_like(input)
        out_mask = mask.clone()
        hk.sparse_mul_add(input, mask, out, out_mask, self.scale, bias)
        return out, out_mask

    def reset(self):
        DCModule.reset(self)
        self.first_iter = True
