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
        self.has_expansion = expand_ratio != 1
        self._expand_depthwise = getattr(L, "expand_depthwise", None)
        self._block_wanted = getattr(L, "fused_block_wanted", None) or (lambda *a: False)
        self._project_expand = getattr(L, "project_expand", None)

    def _tail(self, x, hidden):
        """Depthwise convolution and projection (+ residual sum) of the block, layer by layer;
        ``hidden`` is the output of the expansion layer (the block input itself without one)."""
        start = 1 if self.has_expansion else 0
        if not self.use_res_connect:
            return self.conv[start:](hidden)
        fused = getattr(self.sparse_add, "after_conv", None)
        if fused is None or len(self.conv[-1]) != 1:
            return self.sparse_add(x, self.conv[start:](hidden))
        # the layer namespace can add the residual inside the last convolution's kernel
        return fused(x, self.conv[-1][0], self.conv[start:-1](hidden))

    def _project(self, x, hidden):
        """The projection (+ residual sum) behind the depthwise layer's output ``hidden``."""
        last = self.conv[2 if self.has_expansion else 1:]
        if not self.use_res_connect:
            return last(hidden)
        fused = getattr(self.sparse_add, "after_conv", None)
        if fused is None or len(last) != 1 or len(last[0]) != 1:
            return self.sparse_add(x, last(hidden))
        return fused(x, last[0][0], hidden)

    def forward(self, x):
        return self._tail(x, self.conv[0](x) if self.has_expansion else x)

    def single_layers(self):
        """(expansion or None, depthwise, projection) when each is ONE layer (batch norm folded),
        else None."""
        if any(len(seq) != 1 for seq in self.conv):
            return None
        convs = [seq[0] for seq in self.conv]
        return ([None] + convs) if not self.has_expansion else convs

    def forward_ahead(self, x, expanded, fused_block, next_layers):
        """The block when a layer namespace offers fused forms.  ``expanded`` is this block's
        expansion output if the previous block's launch already produced it (an ``OpenExpansion``
        if its activation still has to be finished by this block's depthwise layer);
        ``next_layers`` = (expansion, depthwise) of the next block, or (final 1x1 convolution,
        None), or None.  The block's own last launch runs the next block's expansion ahead in
        turn where a form for that exists.  Returns (block output, expansion output of the next
        block or None)."""
        layers = self.single_layers()
        next_expansion = next_layers[0] if next_layers is not None else None
        opened = expanded is not None and not isinstance(expanded, (tuple, torch.Tensor))
        hidden = None
        if opened:
            hidden = self._expand_depthwise(layers[0], layers[1], x, opened=expanded)
        elif (expanded is None and self.has_expansion and layers is not None and self._expand_depthwise is not None
                and not isinstance(x, torch.Tensor)):
            # where the block launch below would not take the block anyway: expansion and depthwise
            # layer as two launches (the expansion's activation is finished by the depthwise kernel)
            hidden_shape = (x[0].shape[0], layers[0].out_channels) + tuple(x[0].shape[2:])
            if not self._block_wanted(layers[1], layers[2], next_expansion, hidden_shape, x[0].dtype):
                hidden = self._expand_depthwise(layers[0], layers[1], x)
        if hidden is None:
            if expanded is None:
                expanded = self.conv[0](x) if self.has_expansion else x
            if layers is not None:
                add = self.sparse_add if self.use_res_connect else None
                done = fused_block(expanded, layers[1], layers[2], add, x if add is not None else None, next_expansion)
                if done is not None:
                    return done
            hidden = self.conv[1 if self.has_expansion else 0](expanded)
        if (layers is not None and self._project_expand is not None and next_layers is not None
                and next_layers[1] is not None and not isinstance(hidden, torch.Tensor)):
            # projection (+ residual sum) and the next block's expansion in one launch
            add = self.sparse_add if self.use_res_connect else None
            done = self._project_expand(layers[2], add, x if add is not None else None, next_layers[0],
                                        next_layers[1], hidden)
            if done is not None:
                return done
        return self._project(x, hidden), None


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
        self._fused_block = getattr(L, "fused_block", None)
        self.fuse_head = True
        self.sparsify = L.DCSparsify()
        self.densify = L.DCDensify()
        self.adaptive_avg_pooling = L.DCAdaptiveAveragePooling(output_size=(1, 1))
        self._pooled_dense = getattr(L, "pooled_dense", None)
        self.classifier = nn.Sequential(nn.Dropout(0.2), getattr(L, "Linear", nn.Linear)(self.last_channel, num_classes))
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

    def _features(self, x):
        """``self.features(x)``; with a layer namespace that has ``fused_block``, every inverted
        residual block runs as one launch that also carries the next block's expansion (or the
        final 1x1 convolution)."""
        fused_block = self._fused_block
        if fused_block is None or isinstance(x, torch.Tensor):
            return self.features(x)
        stages = list(self.features)
        x = stages[0](x)
        expanded = None
        for i in range(1, len(stages) - 1):
            nxt = stages[i + 1]
            if isinstance(nxt, _InvertedResidual):
                layers = nxt.single_layers()
                ahead = (layers[0], layers[1]) if layers is not None and layers[0] is not None else None
            else:  # the final 1x1 convolution
                ahead = (nxt[0], None) if len(nxt) == 1 and self.fuse_head else None
            x, expanded = stages[i].forward_ahead(x, expanded, fused_block, ahead)
        return expanded if expanded is not None else stages[-1](x)

    def forward(self, x):
        x = self.sparsify(x)
        x = self._features(x)
        dense = None
        if self._pooled_dense is not None:  # pooling and densify as one launch where the namespace has it
            dense = self._pooled_dense(self.adaptive_avg_pooling, self.densify, x)
        x = dense if dense is not None else self.densify(self.adaptive_avg_pooling(x))
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


# ---------------------------------------------------------------------------- HRNet-W32
def _conv_act(L, inp, oup, k=3, stride=1, act="relu"):
    """conv + folded batch norm (+ activation): one biased convolution."""
    return L.DCConv2d(inp, oup, k, stride, (k - 1) // 2, bias=True, activation=act)


def _residual_sum(add, residual, conv, conv_input):
    """``add(residual, conv(conv_input))``; a layer namespace whose DCAdd has ``after_conv`` may
    run the sum inside the convolution's kernel."""
    fused = getattr(add, "after_conv", None)
    if fused is None:
        return add(residual, conv(conv_input))
    return fused(residual, conv, conv_input)


class _BasicBlock(nn.Module):
    """Two 3x3 convolutions and a residual sum followed by ReLU."""
    expansion = 1

    def __init__(self, L, inp, planes, stride=1, project=False):
        super().__init__()
        self.conv1 = _conv_act(L, inp, planes, 3, stride)
        self.conv2 = _conv_act(L, planes, planes, 3, 1, act=None)
        self.project = _conv_act(L, inp, planes, 1, stride, act=None) if project else None
        self.add = L.DCAdd(activation="relu")

    def forward(self, x):
        res = x if self.project is None else self.project(x)
        return _residual_sum(self.add, res, self.conv2, self.conv1(x))


class _Bottleneck(nn.Module):
    """1x1 -> 3x3 -> 1x1 (x4 channels) and a residual sum followed by ReLU."""
    expansion = 4

    def __init__(self, L, inp, planes, stride=1, project=False):
        super().__init__()
        self.conv1 = _conv_act(L, inp, planes, 1)
        self.conv2 = _conv_act(L, planes, planes, 3, stride)
        self.conv3 = _conv_act(L, planes, planes * 4, 1, act=None)
        self.project = _conv_act(L, inp, planes * 4, 1, stride, act=None) if project else None
        self.add = L.DCAdd(activation="relu")

    def forward(self, x):
        res = x if self.project is None else self.project(x)
        return _residual_sum(self.add, res, self.conv3, self.conv2(self.conv1(x)))


class _HRModule(nn.Module):
    """Parallel branches of basic blocks followed by the multi-resolution exchange: every output
    branch i sums all input branches j, brought to its resolution by strided 3x3 convolutions
    (j < i) or a 1x1 convolution + nearest upsampling (j > i), then ReLU."""

    def __init__(self, L, channels, blocks=4, multi_scale_output=True):
        super().__init__()
        n = len(channels)
        self._conv_group = getattr(L, "conv_group", None)
        self._residual_group = getattr(L, "residual_group", None)
        self._add_group = getattr(L, "add_group", None)
        self.branches = nn.ModuleList(
            nn.Sequential(*[_BasicBlock(L, c, c) for _ in range(blocks)]) for c in channels)
        n_out = n if multi_scale_output else 1
        self.fuse = nn.ModuleList()
        self.adds = nn.ModuleList()
        for i in range(n_out):
            row = nn.ModuleList()
            for j in range(n):
                if j == i:
                    row.append(nn.Identity())
                elif j > i:
                    row.append(nn.Sequential(_conv_act(L, channels[j], channels[i], 1, act=None),
                                             L.DCUpsamplingNearest2d(scale_factor=2 ** (j - i))))
                else:
                    steps = [_conv_act(L, channels[j], channels[j], 3, 2) for _ in range(i - j - 1)]
                    steps.append(_conv_act(L, channels[j], channels[i], 3, 2, act=None))
                    row.append(nn.Sequential(*steps))
            self.fuse.append(row)
            # n - 1 sums per output; the last one carries the ReLU
            self.adds.append(nn.ModuleList(L.DCAdd(activation="relu" if k == n - 2 else None)
                                           for k in range(n - 1)))

    def _run_branches(self, xs):
        """The branches side by side: block k of every branch before block k + 1 of any, so that
        a layer namespace with ``conv_group`` / ``residual_group`` can launch the same layer of
        all branches together."""
        for blocks in zip(*self.branches):
            mids = self._conv_group([blk.conv1 for blk in blocks], xs)
            xs = self._residual_group([blk.add for blk in blocks], xs, [blk.conv2 for blk in blocks], mids)
        return xs

    def _run_strided_chains(self, xs):
        """The strided 3x3 convolutions of the exchange, as far as they depend on the branch
        outputs only: chain (i, j) brings branch j down to the resolution of output i in i - j
        steps; all but its last step -- and the last one too for j == 0, where it starts the sum
        of output i instead of joining it -- run level by level, the steps of one level as a group.
        Returns ``{(i, j): tensor}``: the start of output i's sum for j == 0, otherwise the input
        of the chain's last convolution."""
        chains = {(i, j): list(row[j]) for i, row in enumerate(self.fuse) for j in range(min(i, len(xs)))}
        cur = {key: xs[key[1]] for key in chains}
        pos = dict.fromkeys(chains, 0)
        while True:
            ready = [k for k, steps in chains.items() if pos[k] < len(steps) - (1 if k[1] > 0 else 0)]
            if not ready:
                return cur
            done = self._conv_group([chains[k][pos[k]] for k in ready], [cur[k] for k in ready])
            for k, y in zip(ready, done):
                cur[k], pos[k] = y, pos[k] + 1

    def _run_pointwise(self, xs):
        """The 1x1 convolutions of the exchange (branch j up to the resolution of output i < j,
        in front of the upsampling): all of them depend on the branch outputs only and run as one
        group.  Returns ``{(i, j): tensor}``."""
        keys = [(i, j) for i in range(len(self.fuse)) for j in range(i + 1, len(xs))]
        done = self._conv_group([self.fuse[i][j][0] for i, j in keys], [xs[j] for _, j in keys]) if keys else []
        return dict(zip(keys, done))

    def _exchange_by_levels(self, xs):
        """The exchange with everything that is independent launched together: the strided and
        the 1x1 convolutions first (they depend on the branch outputs only), then the sums level
        by level -- term j of every output before term j + 1 of any: the sums of one level belong
        to different outputs and run as one group, each output still adds its terms in order."""
        ahead, narrow = self._run_strided_chains(xs), self._run_pointwise(xs)
        ys = [ahead[(i, 0)] if (i, 0) in ahead else row[0](xs[0]) for i, row in enumerate(self.fuse)]
        for j in range(1, len(xs)):
            sums, carried = [], []
            for i, (row, adds) in enumerate(zip(self.fuse, self.adds)):
                add, branch = adds[j - 1], row[j]
                if j > i:    # 1x1 convolution (done) + upsampling, folded into the sum
                    sums.append((i, add, narrow[(i, j)], branch[1]))
                elif j == i:
                    sums.append((i, add, xs[j], None))
                else:        # the last strided convolution carries the sum
                    carried.append((i, add, branch[-1], ahead[(i, j)]))
            done = self._residual_group([a for _, a, _, _ in carried], [ys[i] for i, _, _, _ in carried],
                                        [c for _, _, c, _ in carried], [m for _, _, _, m in carried])
            done += self._add_group([a for _, a, _, _ in sums], [ys[i] for i, _, _, _ in sums],
                                    [b for _, _, b, _ in sums], [up for _, _, _, up in sums])
            for (i, _, _, _), y in zip(carried + sums, done):
                ys[i] = y
        return ys

    def forward(self, xs):
        # Layers of parallel paths side by side where the layer namespace can launch them together;
        # on a model's first frame -- layers take their numbers in call order -- and for namespaces
        # without those functions: path after path.
        grouped = self._conv_group is not None and len(xs) > 1 and all(
            getattr(m, "frame_idx", 0) >= 0 for m in self.modules())
        xs = self._run_branches(xs) if grouped else [b(x) for b, x in zip(self.branches, xs)]
        if grouped and self._add_group is not None:
            return self._exchange_by_levels(xs)
        ahead = self._run_strided_chains(xs) if grouped else {}
        narrow = self._run_pointwise(xs) if grouped and hasattr(self.adds[0][0], "after_upsample") else {}
        outs = []
        for i, (row, adds) in enumerate(zip(self.fuse, self.adds)):
            y = ahead[(i, 0)] if (i, 0) in ahead else row[0](xs[0])
            for j in range(1, len(xs)):
                add, branch = adds[j - 1], row[j]
                if j > i and hasattr(add, "after_upsample"):
                    # 1x1 convolution + upsampling: the upsampling is folded into the sum
                    y = add.after_upsample(y, narrow[(i, j)] if (i, j) in narrow else branch[0](xs[j]), branch[1])
                elif isinstance(branch, nn.Sequential):
                    # strided 3x3 convolutions: the sum rides in the last one's kernel where it can
                    mid = ahead.get((i, j))
                    if mid is None:
                        mid = xs[j]
                        for step in list(branch)[:-1]:
                            mid = step(mid)
                    y = _residual_sum(add, y, branch[-1], mid)
                else:
                    y = add(y, branch(xs[j]))
            outs.append(y)
        return outs


class HRNet(_Net):
    """HRNet pose network (width 32 by default): stem of two strided 3x3 convolutions, a
    bottleneck stage, then 1 / 4 / 3 exchange modules on 2 / 3 / 4 resolutions, and a 1x1 head
    producing ``num_joints`` heat maps at 1/4 resolution.  Batch norm is folded."""

    def __init__(self, L=_hip_layers, width=32, num_joints=17, modules=(1, 4, 3), blocks=4):
        super().__init__()
        c = [width, width * 2, width * 4, width * 8]
        self.sparsify = L.DCSparsify()
        self.stem = nn.Sequential(_conv_act(L, 3, 64, 3, 2), _conv_act(L, 64, 64, 3, 2))
        self.layer1 = nn.Sequential(_Bottleneck(L, 64, 64, project=True),
                                    *[_Bottleneck(L, 256, 64) for _ in range(3)])
        self.transition1 = nn.ModuleList([_conv_act(L, 256, c[0], 3, 1), _conv_act(L, 256, c[1], 3, 2)])
        self.stage2 = nn.ModuleList(_HRModule(L, c[:2], blocks) for _ in range(modules[0]))
        self.transition2 = _conv_act(L, c[1], c[2], 3, 2)
        self.stage3 = nn.ModuleList(_HRModule(L, c[:3], blocks) for _ in range(modules[1]))
        self.transition3 = _conv_act(L, c[2], c[3], 3, 2)
        self.stage4 = nn.ModuleList(_HRModule(L, c[:4], blocks, multi_scale_output=(k < modules[2] - 1))
                                    for k in range(modules[2]))
        self.final = L.DCConv2d(c[0], num_joints, 1, bias=True, dense_out=True)

    def forward(self, x):
        x = self.layer1(self.stem(self.sparsify(x)))
        xs = [t(x) for t in self.transition1]
        for m in self.stage2:
            xs = m(xs)
        xs.append(self.transition2(xs[-1]))
        for m in self.stage3:
            xs = m(xs)
        xs.append(self.transition3(xs[-1]))
        for m in self.stage4:
            xs = m(xs)
        return self.final(xs[0])


# ------------------------------------------------------------------- DLA-34 + CenterNet head
class _Root(nn.Module):
    """1x1 convolution over the concatenated children of a tree node, + ReLU."""

    def __init__(self, L, in_channels, out_channels, n_inputs):
        super().__init__()
        self.cats = nn.ModuleList(L.DCConcatenate() for _ in range(n_inputs - 1))
        self.conv = _conv_act(L, in_channels, out_channels, 1)
        self._concat_conv = getattr(L, "concat_conv", None)  # the convolution reads the children where they lie

    def forward(self, xs):
        if self._concat_conv is not None:
            y = self._concat_conv(self.conv, xs)
            if y is not None:
                return y
        y = xs[0]
        for cat, x in zip(self.cats, xs[1:]):
            y = cat(y, x)
        return self.conv(y)


class _Tree(nn.Module):
    """Deep layer aggregation tree: two sub-trees (basic blocks at the leaves) whose outputs,
    with the down-sampled input when ``level_root``, are aggregated by a root node."""

    def __init__(self, L, levels, inp, oup, stride=1, level_root=False, root_dim=0, n_children=0):
        super().__init__()
        if root_dim == 0:
            root_dim = 2 * oup
        if level_root:
            root_dim += inp
        self.levels, self.level_root = levels, level_root
        self.downsample = L.DCMaxPooling(stride, stride=stride) if stride > 1 else None
        self.project = _conv_act(L, inp, oup, 1, act=None) if inp != oup else None
        if levels == 1:
            self.tree1 = _BasicBlockExt(L, inp, oup, stride)
            self.tree2 = _BasicBlockExt(L, oup, oup, 1)
            self.root = _Root(L, root_dim, oup, 2 + n_children + (1 if level_root else 0))
        else:
            self.tree1 = _Tree(L, levels - 1, inp, oup, stride, root_dim=0)
            self.tree2 = _Tree(L, levels - 1, oup, oup, root_dim=root_dim + oup,
                               n_children=n_children + (1 if level_root else 0) + 1)
            self.root = None

    def forward(self, x, residual=None, children=None):
        children = [] if children is None else children
        bottom = self.downsample(x) if self.downsample is not None else x
        residual = self.project(bottom) if self.project is not None else bottom
        if self.level_root:
            children.append(bottom)
        x1 = self.tree1(x, residual)
        if self.levels == 1:
            x2 = self.tree2(x1)
            return self.root([x2, x1] + children)
        children.append(x1)
        return self.tree2(x1, children=children)


class _BasicBlockExt(nn.Module):
    """Basic block whose residual operand is handed in (the tree computes it once)."""

    def __init__(self, L, inp, planes, stride=1):
        super().__init__()
        self.conv1 = _conv_act(L, inp, planes, 3, stride)
        self.conv2 = _conv_act(L, planes, planes, 3, 1, act=None)
        self.add = L.DCAdd(activation="relu")

    def forward(self, x, residual=None, children=None):
        residual = x if residual is None else residual
        return _residual_sum(self.add, residual, self.conv2, self.conv1(x))


class _IDAUp(nn.Module):
    """Iterative aggregation: every deeper level is projected (3x3), up-sampled by a transposed
    convolution (kernel 2f, stride f, padding f/2, dense groups) and merged (sum + 3x3 node)."""

    def __init__(self, L, out_dim, channels, factors):
        super().__init__()
        self.proj, self.up, self.add, self.node = (nn.ModuleList() for _ in range(4))
        for c, f in zip(channels[1:], factors[1:]):
            self.proj.append(_conv_act(L, c, out_dim, 3))
            self.up.append(L.DCConvTranspose2d(out_dim, out_dim, f * 2, stride=f, padding=f // 2, bias=False))
            self.add.append(L.DCAdd())
            self.node.append(_conv_act(L, out_dim, out_dim, 3))

    def forward(self, layers, start, end):
        for i in range(start + 1, end):
            k = i - start - 1
            # add(up(proj(x)), previous level): a layer namespace whose DCAdd has ``conv_first`` may
            # run the sum inside the transposed convolution's kernel
            fused = getattr(self.add[k], "conv_first", None)
            if fused is None:
                merged = self.add[k](self.up[k](self.proj[k](layers[i])), layers[i - 1])
            else:
                merged = fused(self.up[k], self.proj[k](layers[i]), layers[i - 1])
            layers[i] = self.node[k](merged)


class DLA34CenterNet(_Net):
    """DLA-34 backbone, DLA-up / IDA-up decoder at output stride 4 and three CenterNet heads
    (heat map, size, offset).  The 7x7 stem has stride 1, tree nodes down-sample with 2x2
    max-pooling, roots concatenate, the decoder up-samples with transposed convolutions
    (kernel 4, stride 2, padding 1, groups 1).  Batch norm is folded."""

    def __init__(self, L=_hip_layers, num_classes=80, head_conv=256,
                 channels=(16, 32, 64, 128, 256, 512)):
        super().__init__()
        c = list(channels)
        self.sparsify = L.DCSparsify()
        self.base_layer = _conv_act(L, 3, c[0], 7)
        self.level0 = _conv_act(L, c[0], c[0], 3)
        self.level1 = _conv_act(L, c[0], c[1], 3, 2)
        self.level2 = _Tree(L, 1, c[1], c[2], 2)
        self.level3 = _Tree(L, 2, c[2], c[3], 2, level_root=True)
        self.level4 = _Tree(L, 2, c[3], c[4], 2, level_root=True)
        self.level5 = _Tree(L, 1, c[4], c[5], 2, level_root=True)
        # DLA-up over levels 2..5 (strides 4..32)
        up_c = c[2:]
        scales = [1, 2, 4, 8]
        self.dla_up = nn.ModuleList()
        in_c = list(up_c)
        sc = list(scales)
        for i in range(len(up_c) - 1):
            j = -i - 2
            self.dla_up.append(_IDAUp(L, up_c[j], in_c[j:], [s // sc[j] for s in sc[j:]]))
            sc[j + 1:] = [sc[j]] * len(sc[j + 1:])
            in_c[j + 1:] = [up_c[j]] * len(in_c[j + 1:])
        self.ida_up = _IDAUp(L, up_c[0], up_c[:3], [1, 2, 4])
        self.heads = nn.ModuleDict({
            name: nn.Sequential(_conv_act(L, up_c[0], head_conv, 3),
                                L.DCConv2d(head_conv, n, 1, bias=True, dense_out=True))
            for name, n in (("hm", num_classes), ("wh", 2), ("reg", 2))})

    def forward(self, x):
        x = self.level0(self.base_layer(self.sparsify(x)))
        x = self.level1(x)
        feats = []
        for lvl in (self.level2, self.level3, self.level4, self.level5):
            x = lvl(x)
            feats.append(x)
        layers = list(feats)
        outs = [layers[-1]]
        for i, ida in enumerate(self.dla_up):
            ida(layers, len(layers) - i - 2, len(layers))
            outs.insert(0, layers[-1])
        y = outs[:3]
        self.ida_up(y, 0, len(y))
        return {name: head(y[-1]) for name, head in self.heads.items()}
