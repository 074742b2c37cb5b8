"""Model builders for the benchmark configurations, written against a *layer namespace*.

Every builder takes ``L``: an object with the DeltaCNN layer classes (``DCConv2d``,
``DCActivation``, ``DCAdd``, ...).  ``L=deltacnn_amd.sparse_layers`` (default) gives the HIP
delta model; :class:`DenseLayers` gives the plain torch model with identical parameter names,
used as the dense baseline.  Tests pass their own CPU layer namespace to obtain a checker with
the same topology and the same ``state_dict`` keys.

Topologies
* :class:`ToyCNN`       the README's three-layer example (readme.md:108-124)
* :class:`MobileNetV2`  example/mobilenet_deltacnn.py:75-230, optionally with batch norm folded
                        into the convolutions (bias=True, fused activation)
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import sparse_layers as _hip_layers


class _DenseConv(nn.Conv2d):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, padding_mode="zeros", delta_threshold=None, name=None,
                 activation=None, dense_out=False, **kwargs):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, groups, bias)
        self.act = DenseLayers.activation_module(activation)

    def forward(self, x):
        x = super().forward(x)
        return x if self.act is None else self.act(x)


class _DenseDeconv(nn.ConvTranspose2d):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, output_padding=0,
                 groups=1, bias=True, dilation=1, padding_mode="zeros", delta_threshold=None,
                 name=None, activation=None, dense_out=False, **kwargs):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, 0, groups, bias, dilation)
        self.act = DenseLayers.activation_module(activation)

    def forward(self, x):
        x = super().forward(x)
        return x if self.act is None else self.act(x)


class _DenseAct(nn.Module):
    def __init__(self, name="", inplace=True, delta_threshold=None, activation="relu", truncation_mode=None):
        super().__init__()
        self.act = DenseLayers.activation_module(activation)

    def forward(self, x):
        return self.act(x)


class _DenseAdd(nn.Module):
    def __init__(self, activation=None, dense_out=False, weight_a=None, weight_b=None, name=""):
        super().__init__()
        self.act = DenseLayers.activation_module(activation)
        self.wa = 1.0 if weight_a is None else weight_a
        self.wb = 1.0 if weight_b is None else weight_b

    def forward(self, a, b):
        c = a + b if self.wa == 1.0 and self.wb == 1.0 else self.wa * a + self.wb * b
        return c if self.act is None else self.act(c)


class _Identity(nn.Module):
    def __init__(self, *args, **kwargs):
        super().__init__()

    def forward(self, x):
        return x


class _DenseConcat(nn.Module):
    def __init__(self, name=""):
        super().__init__()

    def forward(self, a, b):
        return torch.cat((a, b), dim=1)


class _DenseMaxPool(nn.MaxPool2d):
    def __init__(self, kernel_size, stride=(1, 1), padding=(0, 0), dilation=(1, 1)):
        super().__init__(kernel_size, stride=stride, padding=padding, dilation=dilation)


class DenseLayers:
    """Plain torch counterparts of the DC layer classes (the dense baseline model)."""
    DCModule = nn.Module
    DCConv2d = _DenseConv
    DCConvTranspose2d = _DenseDeconv
    DCActivation = _DenseAct
    DCAdd = _DenseAdd
    DCSparsify = _Identity
    DCDensify = _Identity
    DCConcatenate = _DenseConcat
    DCMaxPooling = _DenseMaxPool
    DCBatchNorm2d = nn.BatchNorm2d

    @staticmethod
    def DCAdaptiveAveragePooling(output_size=None):
        return nn.AdaptiveAvgPool2d(output_size)

    @staticmethod
    def DCUpsamplingNearest2d(scale_factor=2, name=""):
        return nn.UpsamplingNearest2d(scale_factor=scale_factor)

    @staticmethod
    def activation_module(name):
        if name is None or name == "" or name == "linear":
            return None
        return {"relu": nn.ReLU, "relu6": nn.ReLU6, "sigmoid": nn.Sigmoid,
                "leaky": lambda: nn.LeakyReLU(0.1), "swish": nn.SiLU}[name.lower()]()


class _Net(nn.Module):
    """Model-level ``process_filters`` / ``reset_layers`` that work for any layer namespace
    (counterparts of DCModule.process_filters / reset_layers, sparse_layers.py:224-243)."""

    def process_filters(self):
        for m in self.modules():
            if m is not self and hasattr(m, "process_filters") and isinstance(m, (nn.Conv2d, nn.ConvTranspose2d)):
                m.process_filters()

    def reset_layers(self):
        for m in self.modules():
            if m is not self and hasattr(m, "reset"):
                m.reset()


class ToyCNN(_Net):
    """Conv 3->16->32->32, each 3x3 / stride 1 / padding 1 / ReLU (readme.md:108-124)."""

    def __init__(self, L=_hip_layers):
        super().__init__()
        self.sparsify = L.DCSparsify()
        self.conv1 = L.DCConv2d(3, 16, 3, padding=1, activation="relu")
        self.conv2 = L.DCConv2d(16, 32, 3, padding=1, activation="relu")
        self.conv3 = L.DCConv2d(32, 32, 3, padding=1, activation="relu", dense_out=True)

    def forward(self, x):
        return self.conv3(self.conv2(self.conv1(self.sparsify(x))))


def _make_divisible(v, divisor, min_value=None):
    min_value = divisor if min_value is None else min_value
    new_v = max(min_value, int(v + divisor / 2) // divisor * divisor)
    if new_v < 0.9 * v:
        new_v += divisor
    return new_v


class _ConvBNAct(nn.Sequential):
    """conv + BN + ReLU6 (example/mobilenet_deltacnn.py:75-86); with ``fold_bn`` a single
    biased convolution with fused activation."""

    def __init__(self, L, inp, oup, kernel_size=3, stride=1, groups=1, fold_bn=True, act="relu6"):
        padding = (kernel_size - 1) // 2
        if fold_bn:
            super().__init__(L.DCConv2d(inp, oup, kernel_size, stride, padding, groups=groups,
                                        bias=True, activation=act))
        else:
            layers = [L.DCConv2d(inp, oup, kernel_size, stride, padding, groups=groups, bias=False),
                      L.DCBatchNorm2d(oup)]
            if act is not None:
                layers.append(L.DCActivation(activation=act, inplace=True))
            super().__init__(*layers)


class _InvertedResidual(nn.Module):
    """example/mobilenet_deltacnn.py:89-122."""

    def __init__(self, L, inp, oup, stride, expand_ratio, fold_bn):
        super().__init__()
        hidden = int(round(inp * expand_ratio))
        self.use_res_connect = stride == 1 and inp == oup
        self.sparse_add = L.DCAdd()
        layers = []
        if expand_ratio != 1:
            layers.append(_ConvBNAct(L, inp, hidden, kernel_size=1, fold_bn=fold_bn))
        layers.append(_ConvBNAct(L, hidden, hidden, stride=stride, groups=hidden, fold_bn=fold_bn))
        layers.append(_ConvBNAct(L, hidden, oup, kernel_size=1, fold_bn=fold_bn, act=None))
        self.conv = nn.Sequential(*layers)

    def forward(self, x):
        if not self.use_res_connect:
            return self.conv(x)
        fused = getattr(self.sparse_add, "after_conv", None)
        if fused is None or len(self.conv[-1]) != 1:
            return self.sparse_add(x, self.conv(x))
        # the layer namespace can add the residual inside the last convolution's kernel
        return fused(x, self.conv[-1][0], self.conv[:-1](x))


MOBILENET_V2_SETTING = [  # t, c, n, s  (example/mobilenet_deltacnn.py:160-170)
    [1, 16, 1, 1], [6, 24, 2, 2], [6, 32, 3, 2], [6, 64, 4, 2], [6, 96, 3, 1], [6, 160, 3, 2],
    [6, 320, 1, 1]]


class MobileNetV2(_Net):
    """MobileNetV2 with DeltaCNN layers (example/mobilenet_deltacnn.py:125-230)."""

    def __init__(self, L=_hip_layers, num_classes=1000, width_mult=1.0, round_nearest=8,
                 fold_bn=True, setting=None):
        super().__init__()
        setting = MOBILENET_V2_SETTING if setting is None else setting
        input_channel = _make_divisible(32 * width_mult, round_nearest)
        self.last_channel = _make_divisible(1280 * max(1.0, width_mult), round_nearest)
        features = [_ConvBNAct(L, 3, input_channel, stride=2, fold_bn=fold_bn)]
        for t, c, n, s in setting:
            output_channel = _make_divisible(c * width_mult, round_nearest)
            for i in range(n):
                features.append(_InvertedResidual(L, input_channel, output_channel, s if i == 0 else 1,
                                                  t, fold_bn))
                input_channel = output_channel
        features.append(_ConvBNAct(L, input_channel, self.last_channel, kernel_size=1, fold_bn=fold_bn))
        self.features = nn.Sequential(*features)
        self.sparsify = L.DCSparsify()
        self.densify = L.DCDensify()
        self.adaptive_avg_pooling = L.DCAdaptiveAveragePooling(output_size=(1, 1))
        self.classifier = nn.Sequential(nn.Dropout(0.2), nn.Linear(self.last_channel, num_classes))
        for m in self.modules():
            if isinstance(m, nn.Conv2d):
                nn.init.kaiming_normal_(m.weight, mode="fan_out")
                if m.bias is not None:
                    nn.init.zeros_(m.bias)
            elif isinstance(m, nn.BatchNorm2d):
                nn.init.ones_(m.weight)
                nn.init.zeros_(m.bias)
            elif isinstance(m, nn.Linear):
                nn.init.normal_(m.weight, 0, 0.01)
                nn.init.zeros_(m.bias)

    def forward(self, x):
        x = self.sparsify(x)
        x = self.features(x)
        x = self.adaptive_avg_pooling(x)
        x = self.densify(x)
        x = x.reshape(x.shape[0], -1)
        return self.classifier(x)


@torch.no_grad()
def fold_data_statistics(dense_model: nn.Module, frames: torch.Tensor) -> None:
    """Give a randomly initialised BN-folded model the scale a trained one has.

    A trained network's batch norm makes every convolution output roughly zero-mean /
    unit-variance per channel; folding it leaves that scale in the weights and bias.  With
    random weights there is no batch norm to fold, so this rescales each convolution of the
    *dense* model, in execution order, to zero mean and unit variance per output channel on
    ``frames`` -- the same affine map a batch norm layer with gamma=1, beta=0 would apply.
    Copy the resulting ``state_dict`` into the delta models afterwards.
    """
    convs = [m for m in dense_model.modules() if isinstance(m, nn.Conv2d)]
    captured = {}

    def hook(mod, inp, out):
        captured["x"] = inp[0]

    for conv in convs:
        h = conv.register_forward_hook(hook)
        dense_model(frames)
        h.remove()
        y = nn.functional.conv2d(captured["x"], conv.weight, None, conv.stride, conv.padding,
                                 conv.dilation, conv.groups).float()
        mean = y.mean(dim=(0, 2, 3))
        std = y.std(dim=(0, 2, 3)).clamp_min(1e-3)
        conv.weight.mul_((1.0 / std).to(conv.weight.dtype)[:, None, None, None])
        if conv.bias is not None:
            conv.bias.copy_((-mean / std).to(conv.bias.dtype))
