"""Stateful CPU restatement of the DeltaCNN layer protocol (sparse_layers.py).

TEST INFRASTRUCTURE: layer classes with the constructor signatures of the
reference's ``DC*`` modules, running entirely on ``oracle.delta_ops``.  A model
builder that takes a layer namespace can be instantiated once over the shipped
HIP layers and once over this module and compared frame by frame.

Differences to the shipped layers, on purpose: weights stay in torch layout
(``process_filters`` is a no-op), thresholds are plain per-layer floats, and
nothing is pre-allocated or cached beyond what the protocol requires.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import delta_ops as ops

_ACT = {None: (None, -1), "": (None, -1), "linear": (None, -1), "relu": (1, 1), "relu6": (2, 2),
        "leaky": (3, 3), "sigmoid": (4, 4), "swish": (5, 5)}


def _act_id(name):
    """convert_activation_string, sparse_layers.py:20-34."""
    key = name.lower() if isinstance(name, str) else name
    if key not in _ACT:
        raise Exception(f"Activation {name} not implemented")
    return _ACT[key][1]


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


class DCThreshold:
    t_default = 0.0


class DCModule(nn.Module):
    def reset(self):
        pass

    def process_filters(self):
        pass

    def reset_layers(self):
        for m in self.modules():
            if m is not self and isinstance(m, DCModule):
                m.reset()


class DCSparsify(DCModule):
    """sparse_layers.py:1197-1273."""

    def __init__(self, name="", delta_threshold=None, dilation=-1):
        super().__init__()
        self.delta_threshold = DCThreshold.t_default if delta_threshold is None else delta_threshold
        self.dilation = dilation
        self.prev_in = None

    def forward(self, x):
        if self.prev_in is None:
            self.prev_in = x.clone()
            return x, torch.ones_like(x[:, :1], dtype=torch.int32)
        if self.dilation > 1:
            return ops.sparsify_dilated(x, self.prev_in, self.delta_threshold, self.dilation)
        return ops.sparsify(x, self.prev_in, self.delta_threshold)

    def reset(self):
        self.prev_in = None


class DCActivation(DCModule):
    """sparse_layers.py:1362-1425."""
    truncation_default = ops.TRUNC_MAX

    def __init__(self, name="", inplace=True, delta_threshold=None, activation="relu",
                 truncation_mode=None):
        super().__init__()
        self.act = _act_id(activation)
        self.delta_threshold = DCThreshold.t_default if delta_threshold is None else delta_threshold
        self.mode = DCActivation.truncation_default if truncation_mode is None else truncation_mode
        self.mode = getattr(self.mode, "value", self.mode)
        self.prev_out = None
        self.out_truncated = None

    def forward(self, inp):
        if isinstance(inp, torch.Tensor):
            return ops.activation(inp, self.act)
        val, mask = inp
        if self.prev_out is None:
            self.prev_out = val.clone()
            self.out_truncated = torch.zeros_like(val)
            return ops.activation(val, self.act), mask
        val, mask = val.clone(), mask.clone()
        ops.activate_truncate(val, self.prev_out, self.out_truncated, mask,
                              self.delta_threshold, self.act, self.mode)
        return val, mask

    def reset(self):
        self.prev_out = None
        self.out_truncated = None


class DCDensify(DCModule):
    """sparse_layers.py:1276-1333."""

    def __init__(self, activation=None, name="", clone_out=True):
        super().__init__()
        self.act = _act_id(activation)
        self.prev_out = None

    def forward(self, inp):
        if isinstance(inp, torch.Tensor):
            return inp
        val, mask = inp
        if self.prev_out is None:
            self.prev_out = torch.zeros_like(val)
        ops.activate_truncate(val.clone(), self.prev_out, None, mask, -1, -1, ops.TRUNC_NONE)
        return ops.activation(self.prev_out.clone(), self.act)

    def reset(self):
        self.prev_out = None


class _ConvMixin:
    def _init_delta(self, delta_threshold, activation, dense_out):
        self.frame_idx = -1
        self.dense_out = dense_out
        self.densify_layer = DCDensify(activation=activation) if dense_out else None
        self.activation_layer = None
        if not dense_out and _act_id(activation) > 0:
            self.activation_layer = DCActivation(delta_threshold=delta_threshold, activation=activation)

    def _finish(self, out, om):
        if self.dense_out:
            return self.densify_layer((out, om))
        if self.activation_layer is not None:
            return self.activation_layer((out, om))
        return out, om

    def reset(self):
        self.frame_idx = -1


class DCConv2d(nn.Conv2d, _ConvMixin, DCModule):
    """sparse_layers.py:261-675 (delta path ``_forward_delta_conv`` :603-640)."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, padding_mode="zeros", delta_threshold=None, name=None,
                 activation=None, dense_out=False, **kwargs):
        self.padding4 = None
        if not isinstance(padding, int) and len(padding) == 4:
            self.padding4, padding = tuple(padding), 0
        nn.Conv2d.__init__(self, in_channels, out_channels, kernel_size, stride, padding, dilation,
                           groups, bias, padding_mode)
        self._init_delta(delta_threshold, activation, dense_out)

    def forward(self, inp):
        self.frame_idx += 1
        x, mask = inp
        bias = self.bias if self.frame_idx <= 0 else None
        pad = self.padding4 if self.padding4 is not None else self.padding
        out, om = ops.conv(x, mask, self.weight.data, None if bias is None else bias.data,
                           self.stride, pad, self.dilation, self.groups)
        return self._finish(out, om)


class DCConvTranspose2d(nn.ConvTranspose2d, _ConvMixin, DCModule):
    """sparse_layers.py:678-1083."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0,
                 output_padding=0, groups=1, bias=True, dilation=1, padding_mode="zeros",
                 delta_threshold=None, name=None, activation=None, dense_out=False, **kwargs):
        nn.ConvTranspose2d.__init__(self, in_channels, out_channels, kernel_size, stride, padding,
                                    output_padding, groups, bias, dilation, padding_mode)
        self._init_delta(delta_threshold, activation, dense_out)

    def forward(self, inp):
        self.frame_idx += 1
        x, mask = inp
        bias = self.bias if self.frame_idx <= 0 else None
        out, om = ops.deconv(x, mask, self.weight.data, None if bias is None else bias.data,
                             self.stride, self.padding, self.dilation, self.groups)
        return self._finish(out, om)


class DCAdd(DCModule):
    """sparse_layers.py:1086-1182."""

    def __init__(self, activation=None, dense_out=False, weight_a=None, weight_b=None, name=""):
        super().__init__()
        self.act = _act_id(activation)
        self.dense_out = dense_out
        self.weight_a = 1.0 if weight_a is None else weight_a
        self.weight_b = 1.0 if weight_b is None else weight_b
        self.prev_out = None

    def forward(self, a, b, weight_a=None, weight_b=None):
        wa = self.weight_a if weight_a is None else weight_a
        wb = self.weight_b if weight_b is None else weight_b
        if isinstance(a, torch.Tensor):
            return ops.activation(wa * a + wb * b, self.act)
        (va, ma), (vb, mb) = a, b
        if self.prev_out is None and (self.dense_out or self.act > 0):
            self.prev_out = torch.zeros_like(va)
        out, mo = ops.add(va, ma, vb, mb, self.prev_out, wa, wb, self.act, self.dense_out)
        return out if self.dense_out else (out, mo)

    def reset(self):
        self.prev_out = None


class DCMaxPooling(DCModule):
    """sparse_layers.py:1428-1474."""

    def __init__(self, kernel_size, stride=(1, 1), padding=(0, 0), dilation=(1, 1)):
        super().__init__()
        self.kernel_size, self.stride, self.dilation = _pair(kernel_size), _pair(stride), _pair(dilation)
        self.padding = _pair(padding)
        self.prev_in = None

    def forward(self, inp):
        if isinstance(inp, torch.Tensor):
            return F.max_pool2d(inp, self.kernel_size, self.stride, self.padding, self.dilation)
        x, mask = inp
        if self.prev_in is None:
            self.prev_in = torch.zeros_like(x)
        out = ops.pool(x, self.prev_in, mask, self.kernel_size, self.stride, self.padding,
                       self.dilation, mode=0)
        ops.add_to_dense(x, self.prev_in, mask)
        return out

    def reset(self):
        self.prev_in = None


class DCAdaptiveAveragePooling(DCModule):
    """sparse_layers.py:1477-1513 (only a 1x1 output is supported, :1489)."""

    def __init__(self, output_size=None):
        super().__init__()
        self.output_size = _pair(output_size)
        assert self.output_size == (1, 1)

    def forward(self, inp):
        if isinstance(inp, torch.Tensor):
            return F.adaptive_avg_pool2d(inp, self.output_size)
        x, mask = inp
        return ops.pool(x, None, mask, x.shape[2:], (1, 1), (0, 0), (1, 1), mode=1)


class DCUpsamplingNearest2d(DCModule):
    """sparse_layers.py:1336-1359."""

    def __init__(self, scale_factor=2, name=""):
        super().__init__()
        self.scale_factor = int(scale_factor)

    def forward(self, inp):
        if isinstance(inp, torch.Tensor):
            return F.interpolate(inp, scale_factor=self.scale_factor, mode="nearest")
        return ops.upsample(inp[0], inp[1], self.scale_factor)


class DCConcatenate(DCModule):
    """sparse_layers.py:1185-1194."""

    def __init__(self, name=""):
        super().__init__()

    def forward(self, a, b):
        if isinstance(a, torch.Tensor):
            return torch.cat((a, b), dim=1)
        return ops.concatenate(a[0], a[1], b[0], b[1])


class DCBatchNorm2d(nn.BatchNorm2d, DCModule):
    """sparse_layers.py:1516-1585: scale on every frame, offset on the first only."""

    def __init__(self, num_features, eps=1e-5, momentum=0.1, affine=True,
                 track_running_stats=True, inplace=True):
        nn.BatchNorm2d.__init__(self, num_features, eps, momentum, affine, track_running_stats)
        self.first_iter = True

    def forward(self, inp):
        scale = self.weight * torch.rsqrt(self.running_var + self.eps)
        offset = -self.running_mean * scale + self.bias
        if isinstance(inp, torch.Tensor):
            return inp * scale[None, :, None, None] + offset[None, :, None, None]
        x, mask = inp
        first, self.first_iter = self.first_iter, False
        return ops.mul_add(x, mask, scale.data, offset.data if first else None)

    def reset(self):
        self.first_iter = True
