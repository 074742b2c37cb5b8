"""Functional CPU restatement of DeltaCNN's delta-propagation operators.

TEST INFRASTRUCTURE: the checker the HIP kernels are compared against and the
reported CPU baseline.  Never imported by the shipped package.

Conventions
-----------
* feature tensors are logical ``[B, C, H, W]`` (any memory format), fp32 or fp16
* masks are ``int32 [B, 1, H, W]``; a pixel is *active* iff its mask word != 0
* values at inactive pixels are undefined in the reference (``torch.empty``);
  every function here treats them as absent (never lets them reach an output of
  an active pixel) and returns zeros at pixels it does not define
* fp16: the reference performs one IEEE fp16 operation at a time (``__hadd2``,
  ``__hsub2``, ``__hmul2``; ``__hfma2`` single rounding).  PyTorch CPU half ops
  compute in fp32 and round once, which is bit-identical for a single
  add/sub/mul, so every reference operation is kept as a separate tensor op.

Paths are relative to the reference tree (``src/cuda/...``, ``src/deltacnn/...``).

Pinning status (what fixes each function besides re-reading the source; tests are in
tests/test_oracle_pins.py unless another file is named)
----------------------------------------------------------------------
activation          ids 1-3: scalar loops (test_activate_truncate_against_loops); ids 4/5:
                    torch.sigmoid / F.silu (test_sigmoid_and_swish_against_library).  The
                    reference's fp16 ``hexp``/``hrcp`` rounding is source-derived only:
                    parity unpinned for the last fp16 ulp of sigmoid / swish.
sparsify            loops (test_sparsify_against_loops) + cache invariants; the fp16 even-C
                    ``>=`` tie rule (``other_nn_layers.cu:1289``) is source-derived only:
                    parity unpinned for that tie case.
sparsify_dilated    window loops (test_sparsify_dilated_against_window_loops).
activate_truncate   mode max: loops + conservation invariant prev + trunc == running
                    pre-activation; modes norm / rms: loops away from ties
                    (test_norm_rms_truncation_against_loops; at a tie the reference's
                    lane-order sum in the tensor's type decides: parity unpinned there);
                    mode < 0 with an activation: telescoping sum
                    (test_accumulate_with_activation_telescopes).
conv / deconv       brute-force loops on tiny inputs, all 2^9 3x3 mask patterns, frame sums =
                    dense conv.  The fp16 rounding sequence of the reference accumulation
                    (``conv_kernel.cu:1390``) cannot be run: parity unpinned beyond the 2e-2
                    tolerance.  deconv with dilation / groups: library call only (the
                    reference has no such path).
pool                loops incl. dilation (test_pool_against_loops,
                    test_pool_with_dilation_against_loops_and_library) and library pooling;
                    the asymmetric-padding zero quirk is source-derived only: parity
                    unpinned for that quirk.  Global max follows the windowed definition,
                    not the reference's per-block atomicMax.
add                 loops (test_add_against_loops), dense-sum tracking with activation,
                    dense_out by indexing (test_add_dense_out_against_indexing).
add_to_dense        indexing loops (test_add_to_dense_against_indexing).
upsample / concat / mul_add   indexing (test_upsample_concat_mul_add_against_indexing).
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F

ACT_LINEAR, ACT_RELU, ACT_RELU6, ACT_LEAKY, ACT_SIGMOID, ACT_SWISH = 0, 1, 2, 3, 4, 5
TRUNC_NONE, TRUNC_MAX, TRUNC_NORM, TRUNC_RMS = -1, 0, 1, 2


def _scalar(v: float, like: torch.Tensor) -> torch.Tensor:
    """A C ``float`` argument narrowed to the tensor dtype (``__float2half_rn``)."""
    return torch.tensor(float(v), dtype=torch.float32).to(like.dtype)


def activation(x: torch.Tensor, act: int) -> torch.Tensor:
    """``activation_selector`` other_nn_layers.cu:21-121 (fp32) / 46-104 (fp16)."""
    if act <= 0:
        return x
    zero = torch.zeros((), dtype=x.dtype)
    if act == ACT_RELU:
        return torch.where(x < zero, zero, x)
    if act == ACT_RELU6:
        six = _scalar(6.0, x)
        return torch.where(x < zero, zero, torch.where(x > six, six, x))
    if act == ACT_LEAKY:
        return torch.where(x < zero, x * _scalar(0.1, x), x)
    if act == ACT_SIGMOID:
        return (1.0 / (1.0 + torch.exp(-x.float()))).to(x.dtype)
    if act == ACT_SWISH:
        return (x.float() * (1.0 / (1.0 + torch.exp(-x.float())))).to(x.dtype)
    raise ValueError(f"activation id {act}")


def _round_f64(value: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """One rounding from float64 to `dtype`.  torch converts float64 to float16 by way of
    float32, which rounds twice (about one value in 10^5 of a fused multiply-add ends one ulp
    off); numpy converts directly."""
    if dtype == torch.float16:
        return torch.from_numpy(value.contiguous().numpy().astype(np.float16)).view(value.shape)
    return value.to(dtype)


def _active(mask: torch.Tensor) -> torch.Tensor:
    return mask != 0


# --------------------------------------------------------------------------- sparsify
def sparsify(x: torch.Tensor, prev: torch.Tensor, threshold: float
             ) -> Tuple[torch.Tensor, torch.Tensor]:
    """other_nn_layers.cu:820-881 (fp32), :1260-1376 (fp16).

    ``d = x - prev``; a pixel is active if any channel passes the compare; active
    pixels get ``delta = d`` and ``prev = x`` on all channels.  ``prev`` is
    updated in place.  Compare: fp32 ``>``; fp16 with even C ``>=``
    (``!__hblt2``, :1289); fp16 with odd C ``>`` (``__hgt``, :1343).
    """
    d = x - prev
    thr = _scalar(threshold, x)
    if x.dtype == torch.float16 and x.shape[1] % 2 == 0:
        hit = ~(d.abs() < thr)
    else:
        hit = d.abs() > thr
    m = hit.any(dim=1, keepdim=True)
    delta = torch.where(m, d, torch.zeros_like(d))
    prev.copy_(torch.where(m, x, prev))
    return delta, m.to(torch.int32)


def sparsify_dilated(x, prev, threshold: float, dilation: int):
    """Torch-side option of DCSparsify, sparse_layers.py:1233-1244."""
    d = x - prev
    a = d.abs().amax(dim=1, keepdim=True)
    # a tensor compared with a Python number is compared in the tensor's type
    m = F.max_pool2d(a.float(), dilation, stride=1, padding=(dilation - 1) // 2) > float(_scalar(threshold, x))
    prev.copy_(torch.where(m, x, prev))
    return torch.where(m, d, torch.zeros_like(d)), m.to(torch.int32)


# ------------------------------------------------------------- activation + truncation
def activate_truncate(delta: torch.Tensor, prev: torch.Tensor, trunc: Optional[torch.Tensor],
                      mask: torch.Tensor, threshold: float, act: int, mode: int) -> None:
    """other_nn_layers.cu:378-463 (max), :664-719 (norm/rms), :754-817; fp16 :884-1258.

    In place on ``delta``, ``prev``, ``trunc`` and ``mask``.  ``mode < 0`` is the
    densify accumulation (``activate_no_truncation`` :378-394): ``prev += delta``
    and, for a non-linear activation, ``delta = act(prev_new) - act(prev_old)``.

    Deviation kept on purpose: for a *linear* activation with truncation the
    reference leaves part (fp32) or all (fp16) of ``delta`` as the raw incoming
    value (:448-452, :950-952); here ``delta = T + prev - prev`` consistently.
    The public layer API cannot reach that case.
    """
    m = _active(mask)
    if mode < 0:
        s = delta + prev
        if act > 0:
            d = activation(s, act) - activation(prev, act)
            delta.copy_(torch.where(m, d, delta))
        prev.copy_(torch.where(m, s, prev))
        return
    t = trunc + delta
    s = t + prev
    d = activation(s, act) - activation(prev, act)
    thr = _scalar(threshold, delta)
    if mode == TRUNC_MAX:
        keep = (d.abs() > thr).any(dim=1, keepdim=True)
    else:
        sq = (d.float() * d.float()).sum(dim=1, keepdim=True)
        if mode == TRUNC_RMS:
            sq = sq / d.shape[1]
        keep = torch.sqrt(sq) > float(thr)
    keep = keep & m
    drop = m & ~keep
    zero = torch.zeros_like(delta)
    prev.copy_(torch.where(keep, s, prev))
    delta.copy_(torch.where(keep, d, delta))
    trunc.copy_(torch.where(keep, zero, torch.where(drop, t, trunc)))
    mask.copy_(keep.to(mask.dtype))


# ------------------------------------------------------------------------------ conv
def _pad4(padding: Sequence[int]) -> Tuple[int, int, int, int]:
    """(top, bottom, left, right) from a 2- or 4-tuple, cuda_kernels.py:21-26."""
    if len(padding) == 2:
        return padding[0], padding[0], padding[1], padding[1]
    if len(padding) == 4:
        return tuple(padding)
    raise ValueError("Padding must be iterable of size 2 or 4")


def dilate_mask(mask: torch.Tensor, kernel: Sequence[int], stride: Sequence[int],
                padding: Sequence[int], dilation: Sequence[int]) -> torch.Tensor:
    """out_mask[o] = OR over in-bounds taps of mask[o*s - pad + k*d]; conv_kernel.cu:156-213."""
    t, b, l, r = _pad4(padding)
    mf = F.pad((mask != 0).float(), (l, r, t, b))
    ones = torch.ones(1, 1, kernel[0], kernel[1])
    return (F.conv2d(mf, ones, stride=tuple(stride), dilation=tuple(dilation)) > 0).to(torch.int32)


def conv(delta: torch.Tensor, mask: torch.Tensor, weight: torch.Tensor,
         bias: Optional[torch.Tensor] = None, stride=(1, 1), padding=(0, 0),
         dilation=(1, 1), groups: int = 1) -> Tuple[torch.Tensor, torch.Tensor]:
    """Delta convolution, conv_kernel.cu:46-63,156-213,511-630,699-757.

    ``weight`` is in torch layout ``[Cout, Cin/g, Kh, Kw]``.  Inactive inputs count
    as zero, the result is an ordinary cross-correlation; it is defined on pixels
    of the dilated mask and returned as zero elsewhere.  Accumulation is fp32,
    rounded once to the tensor dtype.
    """
    t, b, l, r = _pad4(padding)
    x = torch.where(_active(mask), delta, torch.zeros_like(delta)).float()
    x = F.pad(x, (l, r, t, b))
    out = F.conv2d(x, weight.float(), None if bias is None else bias.float(),
                   stride=tuple(stride), dilation=tuple(dilation), groups=groups)
    om = dilate_mask(mask, weight.shape[2:], stride, padding, dilation)
    out = torch.where(_active(om), out, torch.zeros_like(out)).to(delta.dtype)
    return out, om


def deconv(delta: torch.Tensor, mask: torch.Tensor, weight: torch.Tensor,
           bias: Optional[torch.Tensor] = None, stride=(1, 1), padding=(0, 0),
           dilation=(1, 1), groups: int = 1) -> Tuple[torch.Tensor, torch.Tensor]:
    """Delta transposed convolution, deconv_kernel.cu:296-336,460-481.

    ``weight`` is in torch layout ``[Cin, Cout/g, Kh, Kw]``; output size ignores
    ``output_padding`` (cuda_kernels.py:56-57).  Pinned by scatter loops for dilation 1 and
    one group (all the reference supports, deconv_kernel.cu:857); with dilation or groups this
    is the library call alone, there is no reference behaviour to match.
    """
    x = torch.where(_active(mask), delta, torch.zeros_like(delta)).float()
    out = F.conv_transpose2d(x, weight.float(), None if bias is None else bias.float(),
                             stride=tuple(stride), padding=tuple(padding),
                             dilation=tuple(dilation), groups=groups)
    ones = torch.ones(1, 1, weight.shape[2], weight.shape[3])
    om = (F.conv_transpose2d((mask != 0).float(), ones, stride=tuple(stride),
                             padding=tuple(padding), dilation=tuple(dilation)) > 0).to(torch.int32)
    out = torch.where(_active(om), out, torch.zeros_like(out)).to(delta.dtype)
    return out, om


# --------------------------------------------------------------------------- pooling
def _pool_taps(x: torch.Tensor, kernel, stride, pad4, dilation, fill_tl: float,
               fill_b: float, fill_r: float):
    """Yield one ``[B,C,Ho,Wo]`` view per window tap, row-major, after explicit padding."""
    t, b, l, r = pad4
    B, C, H, W = x.shape
    xp = x.new_full((B, C, H + t + b, W + l + r), fill_tl)
    xp[:, :, t:t + H, l:l + W] = x
    if r > 0:
        xp[:, :, t:t + H, l + W:] = fill_r
    if b > 0:
        xp[:, :, t + H:, :] = fill_b
    ho = (H + t + b - dilation[0] * (kernel[0] - 1) - 1) // stride[0] + 1
    wo = (W + l + r - dilation[1] * (kernel[1] - 1) - 1) // stride[1] + 1
    for ky in range(kernel[0]):
        for kx in range(kernel[1]):
            y0, x0 = ky * dilation[0], kx * dilation[1]
            yield xp[:, :, y0:y0 + (ho - 1) * stride[0] + 1:stride[0],
                     x0:x0 + (wo - 1) * stride[1] + 1:stride[1]]


def pool(delta: torch.Tensor, prev: Optional[torch.Tensor], mask: torch.Tensor, kernel,
         stride=(1, 1), padding=(0, 0), dilation=(1, 1), mode: int = 0
         ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Delta pooling, other_nn_layers.cu:1961-1988, 2261-2461; global :3138-3288.

    mode 0 = max: ``max_w(prev + M*delta) - max_w(prev)`` over in-bounds window
    pixels.  With asymmetric 4-tuple padding a literal 0 joins both maxima for
    bottom (right) padded positions when top != bottom (left != right)
    (:2404-2406, :2418-2420).  mode 1 = avg: ``sum_w M*delta / (Kh*Kw)``.
    The cache update ``prev[active] += delta`` is a separate step
    (``add_to_dense``, sparse_layers.py:1468).

    Arithmetic is fp32 for both dtypes with one rounding on store, like the
    reference's fp16 kernels (:2640-2663) and its fp32 global-pool buffer
    (cuda_kernels.py:101-124).
    """
    kernel, stride, dilation = tuple(kernel), tuple(stride), tuple(dilation)
    pad4 = _pad4(padding)
    t, b, l, r = pad4
    om = dilate_mask(mask, kernel, stride, padding, dilation)
    # the fp16 kernels widen to fp32, pool there and round once on store (:2640-2663)
    x = torch.where(_active(mask), delta, torch.zeros_like(delta)).float()
    if mode == 0:
        ninf = -math.inf
        fb = 0.0 if t != b else ninf
        fr = 0.0 if l != r else ninf
        pf = prev.float()
        acc = x + pf
        hi = hp = None
        for ta, tp in zip(_pool_taps(acc, kernel, stride, pad4, dilation, ninf, fb, fr),
                          _pool_taps(pf, kernel, stride, pad4, dilation, ninf, fb, fr)):
            hi = ta if hi is None else torch.maximum(hi, ta)
            hp = tp if hp is None else torch.maximum(hp, tp)
        out = hi - hp
    else:
        acc = None
        for ta in _pool_taps(x, kernel, stride, pad4, dilation, 0.0, 0.0, 0.0):
            acc = ta.clone() if acc is None else acc + ta
        out = acc / float(kernel[0] * kernel[1])
    out = torch.where(_active(om), out, torch.zeros_like(out)).to(delta.dtype)
    return out, om


def add_to_dense(a: torch.Tensor, b: torch.Tensor, mask_a: torch.Tensor, act: int = 0) -> None:
    """``b[px] += a[px]`` on active pixels, other_nn_layers.cu:1731-1957; with ``act > 0``
    (the USE_ACTIVATION variant) ``a`` additionally becomes ``act(b)`` on every pixel."""
    b.copy_(torch.where(_active(mask_a), b + a, b))
    if act > 0:
        a.copy_(activation(b, act))


# ------------------------------------------------------------------------------- add
def add(a, mask_a, b, mask_b, prev_out: Optional[torch.Tensor], weight_a: float = 1.0,
        weight_b: float = 1.0, act: int = 0, dense_out: bool = False):
    """DCAdd, other_nn_layers.cu:1379-1559 (fp32), :1562-1728 (fp16).

    ``s = wa*a*[Ma]``, then ``s = fma(b, wb, s)*[Mb]``.  Without activation and
    dense_out: ``out = s``.  With activation: ``prev += s; out = act(prev_new) -
    act(prev_old)``.  dense_out: ``prev += s`` on active pixels and
    ``out = act(prev)`` everywhere (returned with mask None).
    """
    ma, mb = _active(mask_a), _active(mask_b)
    mo = ma | mb
    wa, wb = _scalar(weight_a, a), _scalar(weight_b, a)
    zero = torch.zeros_like(a)
    s = torch.where(ma, a * wa, zero)
    # single-rounding fma: the fp64 product and sum are exact for fp16 operands
    sb = _round_f64(torch.where(mb, b, zero).double() * wb.double() + s.double(), a.dtype)
    s = torch.where(mb, sb, s)
    if dense_out:
        new = s + prev_out
        prev_out.copy_(torch.where(mo, new, prev_out))
        return activation(prev_out.clone(), act), None
    if act > 0:
        new = s + prev_out
        d = activation(new, act) - activation(prev_out, act)
        prev_out.copy_(torch.where(mo, new, prev_out))
        s = d
    return torch.where(mo, s, zero), mo.to(torch.int32)


# ------------------------------------------------------------------- next-row operators
def upsample(delta, mask, scale: int):
    """Nearest upsample, other_nn_layers.cu:3450-3523."""
    out = delta.repeat_interleave(scale, dim=2).repeat_interleave(scale, dim=3)
    om = mask.repeat_interleave(scale, dim=2).repeat_interleave(scale, dim=3)
    om = (om != 0).to(torch.int32)
    return torch.where(_active(om), out, torch.zeros_like(out)), om


def concatenate(a, mask_a, b, mask_b):
    """Channel concat, union mask, zero fill of the inactive side; other_nn_layers.cu:3601-3771."""
    za = torch.where(_active(mask_a), a, torch.zeros_like(a))
    zb = torch.where(_active(mask_b), b, torch.zeros_like(b))
    return torch.cat((za, zb), dim=1), (_active(mask_a) | _active(mask_b)).to(torch.int32)


def mul_add(x, mask, scale, bias: Optional[torch.Tensor]):
    """Per-channel ``x*scale (+bias)`` on active pixels, other_nn_layers.cu:3773-3896."""
    sc = scale.reshape(1, -1, 1, 1).to(x.dtype)
    if bias is None:
        y = x * sc
    else:
        # single-rounding fma (``__hfma2``, :3861): exact in fp64 for fp16 operands
        y = _round_f64(x.double() * sc.double() + bias.reshape(1, -1, 1, 1).to(x.dtype).double(), x.dtype)
    return torch.where(_active(mask), y, torch.zeros_like(y)), (mask != 0).to(torch.int32)
