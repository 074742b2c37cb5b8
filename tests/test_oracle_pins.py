"""Pins of the CPU oracle (no GPU needed): every operator of `oracle.delta_ops` is compared
with something that does not share its formula --

  * loop-level per-pixel statements in plain numpy (tests/golden/bruteforce.py) on tiny inputs,
    including all 2^9 mask patterns of a 3x3 neighbourhood,
  * library routines it reduces to in special cases (max_pool2d, avg_pool2d),
  * invariants of the delta scheme: frame sums of a linear operator equal the dense operator
    on the last frame, caches conserve the running pre-activation, threshold 0 reproduces the
    dense network.

A dropped term, a wrong sign, a transposed weight or a shifted index fails at least one of them.
"""
import itertools
import os
import sys

import numpy as np
import pytest
import torch
import torch.nn.functional as F

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import bruteforce as bf  # noqa: E402

from oracle import delta_layers as OL  # noqa: E402
from oracle import delta_ops as O  # noqa: E402


def _np(t):
    return t.detach().cpu().numpy()


def _rand(gen, *shape, dtype=torch.float32):
    return torch.randn(*shape, generator=gen).to(dtype)


CONV_CASES = [
    # cin, cout, k, stride, padding, dilation, groups, H, W
    (3, 4, (3, 3), (1, 1), (1, 1), (1, 1), 1, 6, 7),
    (4, 6, (3, 3), (2, 2), (1, 1), (1, 1), 1, 7, 6),
    (2, 3, (3, 3), (1, 1), (2, 2), (2, 2), 1, 7, 7),
    (4, 4, (3, 3), (1, 1), (1, 1), (1, 1), 4, 5, 6),          # depthwise
    (4, 4, (3, 3), (2, 2), (1, 1), (1, 1), 4, 6, 6),          # depthwise strided
    (5, 3, (1, 1), (1, 1), (0, 0), (1, 1), 1, 4, 5),          # pointwise
    (3, 2, (1, 1), (2, 2), (0, 0), (1, 1), 1, 5, 5),          # strided pointwise samples the mask
    (2, 2, (5, 5), (1, 1), (2, 2), (1, 1), 1, 6, 6),
    (2, 3, (7, 7), (2, 2), (3, 3), (1, 1), 1, 9, 8),
    (3, 2, (3, 3), (1, 1), (0, 1, 2, 0), (1, 1), 1, 6, 6),    # (top, bottom, left, right)
    (4, 6, (3, 2), (1, 2), (1, 0), (1, 1), 2, 6, 6),          # two groups, rectangular kernel
]


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("bias", [False, True])
def test_conv_against_loops(case, bias):
    cin, cout, k, s, p, d, g, H, W = case
    gen = torch.Generator().manual_seed(hash(case) % 1000)
    x = _rand(gen, 2, cin, H, W)
    mask = (torch.rand(2, 1, H, W, generator=gen) < 0.4).to(torch.int32)
    w = _rand(gen, cout, cin // g, *k)
    b = _rand(gen, cout) if bias else None
    xin = torch.where(mask != 0, x, torch.full_like(x, float("nan")))
    got, gm = O.conv(xin, mask, w, b, s, p, d, g)
    want, wm = bf.conv(_np(x), _np(mask), _np(w), None if b is None else _np(b), s, p, d, g)
    assert np.array_equal(_np(gm), wm)
    assert np.allclose(_np(got).astype(np.float64), want, rtol=1e-5, atol=1e-5)


def test_mask_dilation_all_3x3_patterns():
    """All 512 activity patterns of the centre 3x3 block of a 5x5 map, through 3x3 kernels with
    stride 1 / stride 2 / dilation 2, against the tap loop."""
    w = torch.ones(1, 1, 3, 3)
    for bits in range(512):
        mask = torch.zeros(1, 1, 5, 5, dtype=torch.int32)
        for i in range(9):
            if bits >> i & 1:
                mask[0, 0, 1 + i // 3, 1 + i % 3] = 1
        x = torch.ones(1, 1, 5, 5)
        for s, p, d in (((1, 1), (1, 1), (1, 1)), ((2, 2), (1, 1), (1, 1)), ((1, 1), (2, 2), (2, 2))):
            got = O.dilate_mask(mask, (3, 3), s, p, d)
            _, want = bf.conv(_np(x), _np(mask), _np(w), None, s, p, d, 1)
            assert np.array_equal(_np(got), want), (bits, s, p, d)


@pytest.mark.parametrize("k,s,p", [(4, 2, 1), (6, 4, 1), (3, 1, 1), (2, 2, 0)])
def test_deconv_against_scatter_loops(k, s, p):
    gen = torch.Generator().manual_seed(k * 10 + s)
    x = _rand(gen, 2, 3, 4, 5)
    mask = (torch.rand(2, 1, 4, 5, generator=gen) < 0.4).to(torch.int32)
    w = _rand(gen, 3, 4, k, k)
    b = _rand(gen, 4)
    xin = torch.where(mask != 0, x, torch.full_like(x, float("nan")))
    got, gm = O.deconv(xin, mask, w, b, (s, s), (p, p))
    want, wm = bf.deconv(_np(x), _np(mask), _np(w), _np(b), (s, s), (p, p))
    assert got.shape[2] == (4 - 1) * s - 2 * p + k  # no output_padding term
    assert np.array_equal(_np(gm), wm)
    assert np.allclose(_np(got).astype(np.float64), want, rtol=1e-5, atol=1e-5)


def test_conv_frame_sums_equal_dense_conv():
    """Linearity: the dense first frame (with bias) plus the delta outputs of the following
    frames equals the dense convolution of the last frame (bias only once)."""
    gen = torch.Generator().manual_seed(3)
    w, b = _rand(gen, 5, 3, 3, 3), _rand(gen, 5)
    frames = [_rand(gen, 1, 3, 8, 8)]
    for _ in range(4):
        nxt = frames[-1].clone()
        nxt[:, :, 2:5, 3:7] = _rand(gen, 1, 3, 3, 4)
        frames.append(nxt)
    ones = torch.ones(1, 1, 8, 8, dtype=torch.int32)
    acc, _ = O.conv(frames[0], ones, w, b, (1, 1), (1, 1))
    prev = frames[0].clone()
    for f in frames[1:]:
        delta, mask = O.sparsify(f, prev, 0.0)
        out, om = O.conv(delta, mask, w, None, (1, 1), (1, 1))
        assert int(om.sum()) < 64  # really sparse
        acc = acc + out
    want = F.conv2d(frames[-1], w, b, padding=1)
    assert torch.allclose(acc, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_sparsify_against_loops(dtype):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 3, 6, 5)).astype(dtype)
    prev = (x + (rng.standard_normal(x.shape) * (rng.random((2, 1, 6, 5)) < 0.5) * 0.2)).astype(dtype)
    # keep differences away from the threshold: the tie rule is checked on its own below
    thr = 0.1
    d = np.abs((x - prev).astype(dtype))
    prev = np.where((d > 0.09) & (d < 0.11), x, prev).astype(dtype)
    tp = torch.from_numpy(prev.copy())
    delta, mask = O.sparsify(torch.from_numpy(x), tp, thr)
    wd, wm, wp = bf.sparsify(x, prev, thr)
    assert np.array_equal(_np(mask), wm) and 0 < wm.sum() < wm.size
    assert np.array_equal(_np(delta), wd)
    assert np.array_equal(_np(tp), wp)


def test_sparsify_half_tie_rule():
    """A difference exactly equal to the threshold: active for fp16 with an even channel count
    (the half2 compare is `not less`), inactive for fp16 odd C and for fp32 (strict `>`).
    This restates the reference source (other_nn_layers.cu:848, :1289, :1343); only a run of the
    reference could pin it."""
    for dtype, c, want in ((torch.float16, 2, 1), (torch.float16, 3, 0), (torch.float32, 2, 0)):
        x = torch.zeros(1, c, 1, 1, dtype=dtype)
        x[0, 0] = 0.5
        prev = torch.zeros_like(x)
        _, m = O.sparsify(x, prev, 0.5)
        assert int(m) == want, (dtype, c)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("act", [1, 2, 3])
def test_activate_truncate_against_loops(dtype, act):
    rng = np.random.default_rng(act)
    shape = (1, 5, 6, 6)
    scale = (rng.random((1, 1, 6, 6)) < 0.5) * 0.97 + 0.03      # half of the pixels: tiny updates
    delta = (rng.standard_normal(shape) * scale).astype(dtype)
    prev = (rng.standard_normal(shape) * 3).astype(dtype)
    trunc = (rng.standard_normal(shape) * 0.02).astype(dtype)
    mask = (rng.random((1, 1, 6, 6)) < 0.7).astype(np.int32)
    want = bf.activate_truncate(delta, prev, trunc, mask, 0.05, act)
    td, tp, tt, tm = (torch.from_numpy(a.copy()) for a in (delta, prev, trunc, mask))
    O.activate_truncate(td, tp, tt, tm, 0.05, act, O.TRUNC_MAX)
    assert 0 < want[3].sum() < mask.sum()  # some kept, some dropped
    assert np.array_equal(_np(tm), want[3])
    assert np.array_equal(_np(tp), want[1])
    assert np.array_equal(_np(tt), want[2])
    kept = np.broadcast_to(want[3] != 0, shape)
    assert np.array_equal(_np(td)[kept], want[0][kept])


def test_activate_truncate_conserves_preactivation():
    """prev + trunc always equals the running sum of everything that entered the layer, and the
    emitted deltas sum to act(prev) - act(prev_0): nothing is lost, only deferred."""
    gen = torch.Generator().manual_seed(11)
    first = _rand(gen, 1, 4, 5, 5)
    prev, trunc = first.clone(), torch.zeros_like(first)
    total, emitted = first.clone().double(), torch.zeros_like(first).double()
    for _ in range(12):
        mask = (torch.rand(1, 1, 5, 5, generator=gen) < 0.6).to(torch.int32)
        delta = _rand(gen, 1, 4, 5, 5) * 0.04
        total += torch.where(mask != 0, delta, torch.zeros_like(delta)).double()
        O.activate_truncate(delta, prev, trunc, mask, 0.05, O.ACT_RELU, O.TRUNC_MAX)
        emitted += torch.where(mask != 0, delta, torch.zeros_like(delta)).double()
        assert torch.allclose((prev + trunc).double(), total, atol=1e-5)
    assert torch.allclose(emitted, (torch.relu(prev) - torch.relu(first)).double(), atol=1e-5)
    assert float(trunc.abs().max()) > 0  # the test did exercise truncation


def test_densify_accumulates():
    gen = torch.Generator().manual_seed(2)
    prev = _rand(gen, 1, 3, 4, 4)
    start = prev.clone()
    delta = _rand(gen, 1, 3, 4, 4)
    mask = (torch.rand(1, 1, 4, 4, generator=gen) < 0.5).to(torch.int32)
    O.activate_truncate(delta, prev, None, mask, 0.0, 0, O.TRUNC_NONE)
    m = (mask != 0).expand_as(prev)
    assert torch.equal(prev[m], (start + delta)[m]) and torch.equal(prev[~m], start[~m])


POOL_CASES = [((2, 2), (2, 2), (0, 0)), ((3, 3), (2, 2), (1, 1)), ((3, 3), (1, 1), (1, 1)),
              ((2, 2), (2, 2), (0, 1, 0, 1)), ((3, 3), (2, 2), (0, 1, 0, 1)), ((3, 3), (2, 2), (1, 0, 1, 0))]


@pytest.mark.parametrize("kernel,stride,padding", POOL_CASES)
@pytest.mark.parametrize("mode", [0, 1])
def test_pool_against_loops(kernel, stride, padding, mode):
    gen = torch.Generator().manual_seed(len(padding) * 7 + kernel[0])
    delta, prev = _rand(gen, 1, 3, 7, 6), _rand(gen, 1, 3, 7, 6)
    mask = (torch.rand(1, 1, 7, 6, generator=gen) < 0.4).to(torch.int32)
    din = torch.where(mask != 0, delta, torch.full_like(delta, float("nan")))
    got, gm = O.pool(din, prev, mask, kernel, stride, padding, (1, 1), mode)
    want, wm = bf.pool(_np(delta), _np(prev), _np(mask), kernel, stride, padding, mode)
    assert np.array_equal(_np(gm), wm)
    assert np.allclose(_np(got).astype(np.float64), want, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("kernel,stride,pad", [(2, 2, 0), (3, 2, 1), (3, 1, 1)])
def test_pool_reduces_to_library_pooling(kernel, stride, pad):
    """Symmetric padding: max = max_pool2d(prev + M*delta) - max_pool2d(prev); avg =
    avg_pool2d(M*delta) with the padding counted in the divisor."""
    gen = torch.Generator().manual_seed(kernel)
    delta, prev = _rand(gen, 2, 4, 8, 8), _rand(gen, 2, 4, 8, 8)
    mask = (torch.rand(2, 1, 8, 8, generator=gen) < 0.5).to(torch.int32)
    z = torch.where(mask != 0, delta, torch.zeros_like(delta))
    got, om = O.pool(delta, prev, mask, (kernel, kernel), (stride, stride), (pad, pad), (1, 1), 0)
    want = F.max_pool2d(prev + z, kernel, stride, pad) - F.max_pool2d(prev, kernel, stride, pad)
    m = (om != 0).expand_as(want)
    assert torch.allclose(got[m], want[m], atol=1e-6)
    got, om = O.pool(delta, None, mask, (kernel, kernel), (stride, stride), (pad, pad), (1, 1), 1)
    want = F.avg_pool2d(z, kernel, stride, pad, count_include_pad=True)
    m = (om != 0).expand_as(want)
    assert torch.allclose(got[m], want[m], atol=1e-6)
    assert torch.equal(om, (F.max_pool2d((mask != 0).float(), kernel, stride, pad) > 0).to(torch.int32))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_add_against_loops(dtype):
    rng = np.random.default_rng(9)
    a = rng.standard_normal((1, 3, 5, 5)).astype(dtype)
    b = rng.standard_normal((1, 3, 5, 5)).astype(dtype)
    ma = (rng.random((1, 1, 5, 5)) < 0.5).astype(np.int32)
    mb = (rng.random((1, 1, 5, 5)) < 0.5).astype(np.int32)
    want, wm = bf.add(a, ma, b, mb, 0.7, 1.3)
    got, gm = O.add(torch.from_numpy(a), torch.from_numpy(ma), torch.from_numpy(b), torch.from_numpy(mb),
                    None, 0.7, 1.3)
    assert np.array_equal(_np(gm), wm)
    assert np.array_equal(_np(got), want)


def test_add_with_activation_tracks_dense_sum():
    """With an activation the emitted deltas sum to act(a_total + b_total) - act(first)."""
    gen = torch.Generator().manual_seed(4)
    first = _rand(gen, 1, 3, 4, 4)
    prev = first.clone()
    total, emitted = first.clone(), torch.zeros_like(first)
    for _ in range(5):
        a, b = _rand(gen, 1, 3, 4, 4), _rand(gen, 1, 3, 4, 4)
        ma = (torch.rand(1, 1, 4, 4, generator=gen) < 0.5).to(torch.int32)
        mb = (torch.rand(1, 1, 4, 4, generator=gen) < 0.5).to(torch.int32)
        total = total + a * (ma != 0) + b * (mb != 0)
        out, mo = O.add(a, ma, b, mb, prev, 1.0, 1.0, O.ACT_RELU)
        assert torch.equal(mo != 0, (ma != 0) | (mb != 0))
        emitted = emitted + out
    assert torch.allclose(prev, total, atol=1e-5)
    assert torch.allclose(emitted, torch.relu(total) - torch.relu(first), atol=1e-5)


def test_upsample_concat_mul_add_against_indexing():
    gen = torch.Generator().manual_seed(6)
    x, y = _rand(gen, 1, 3, 4, 5), _rand(gen, 1, 2, 4, 5)
    mx = (torch.rand(1, 1, 4, 5, generator=gen) < 0.5).to(torch.int32)
    my = (torch.rand(1, 1, 4, 5, generator=gen) < 0.5).to(torch.int32)
    up, um = O.upsample(x, mx, 2)
    cat, cm = O.concatenate(x, mx, y, my)
    sc, bi = _rand(gen, 3), _rand(gen, 3)
    ma, mm = O.mul_add(x, mx, sc, bi)
    for yy, xx in itertools.product(range(4), range(5)):
        on_x, on_y = bool(mx[0, 0, yy, xx]), bool(my[0, 0, yy, xx])
        for dy, dx in itertools.product(range(2), range(2)):
            assert bool(um[0, 0, 2 * yy + dy, 2 * xx + dx]) == on_x
            if on_x:
                assert torch.equal(up[0, :, 2 * yy + dy, 2 * xx + dx], x[0, :, yy, xx])
        assert bool(cm[0, 0, yy, xx]) == (on_x or on_y)
        if on_x or on_y:
            assert torch.equal(cat[0, :3, yy, xx], x[0, :, yy, xx] if on_x else torch.zeros(3))
            assert torch.equal(cat[0, 3:, yy, xx], y[0, :, yy, xx] if on_y else torch.zeros(2))
        assert bool(mm[0, 0, yy, xx]) == on_x
        if on_x:
            assert torch.allclose(ma[0, :, yy, xx], x[0, :, yy, xx] * sc + bi, atol=1e-6)


# ------------------------------------------------------------------------ layer / network level
def _pair(builder, thr, **kw):
    from deltacnn_amd.networks import DenseLayers
    OL.DCThreshold.t_default = thr
    torch.manual_seed(0)
    dense = builder(DenseLayers, **kw).eval()
    model = builder(OL, **kw).eval()
    model.load_state_dict(dense.state_dict())
    return dense, model


def test_toy_network_threshold_zero_equals_dense():
    from deltacnn_amd.networks import ToyCNN
    from deltacnn_amd.video import noise_block_video
    dense, model = _pair(ToyCNN, 0.0)
    video = noise_block_video(frames=5, size=32, fraction=0.1)
    with torch.no_grad():
        for t in range(video.shape[0]):
            assert torch.allclose(model(video[t:t + 1]), dense(video[t:t + 1]), rtol=1e-4, atol=1e-5), t


def test_mobilenet_threshold_zero_equals_dense():
    """Stride-2 stem, depthwise and pointwise convolutions, residual adds, global pooling and
    the classifier: with threshold 0 the delta model reproduces the dense model on every frame."""
    from deltacnn_amd.networks import MobileNetV2
    from deltacnn_amd.video import moving_rectangles_video

    def mb(L):
        return MobileNetV2(L, num_classes=10)
    dense, model = _pair(mb, 0.0)
    video = moving_rectangles_video(frames=4, height=64, width=64, n_rect=2, min_size=8, max_size=20)
    with torch.no_grad():
        for t in range(video.shape[0]):
            want = dense(video[t:t + 1])
            got = model(video[t:t + 1])
            assert torch.allclose(got, want, rtol=1e-3, atol=1e-4 * float(want.abs().max())), t


def test_truncation_error_stays_bounded():
    """Threshold > 0: the output drifts from the dense model by a bounded amount that does not
    grow with the number of frames (the truncated remainder is carried, never dropped)."""
    from deltacnn_amd.networks import ToyCNN
    from deltacnn_amd.video import noise_block_video
    dense, model = _pair(ToyCNN, 0.05)
    video = noise_block_video(frames=24, size=32, fraction=0.05)
    errs = []
    with torch.no_grad():
        for t in range(video.shape[0]):
            errs.append(float((model(video[t:t + 1]) - dense(video[t:t + 1])).abs().max()))
    assert max(errs[12:]) <= 2.0 * max(errs[:12]) + 1e-3 and max(errs) < 0.5


@pytest.mark.parametrize("which", ["hrnet", "dla34"])
def test_multibranch_networks_threshold_zero_equal_dense(which):
    """HRNet (strided 3x3 exchange convolutions, 1x1 + nearest upsampling, chained adds with
    ReLU) and DLA-34 + CenterNet heads (7x7 stem, 2x2 max-pooling, concatenating roots,
    transposed convolutions): with threshold 0 the delta model reproduces the dense model."""
    from deltacnn_amd.networks import HRNet, DLA34CenterNet
    from deltacnn_amd.video import moving_rectangles_video
    if which == "hrnet":
        def builder(L):
            return HRNet(L, modules=(1, 1, 1), blocks=2)
        size = (64, 64)
    else:
        def builder(L):
            return DLA34CenterNet(L, num_classes=4, head_conv=32)
        size = (64, 96)
    dense, model = _pair(builder, 0.0)
    video = moving_rectangles_video(frames=3, height=size[0], width=size[1], n_rect=2, min_size=8, max_size=20)
    with torch.no_grad():
        for t in range(video.shape[0]):
            want, got = dense(video[t:t + 1]), model(video[t:t + 1])
            if not isinstance(want, dict):
                want, got = {"out": want}, {"out": got}
            for k in want:
                assert torch.allclose(got[k], want[k], rtol=1e-3, atol=1e-4 * max(1.0, float(want[k].abs().max()))), (t, k)


def test_fused_multiply_add_rounds_once_in_half_precision():
    """The fp16 fused multiply-adds of the oracle (DCAdd's second operand, mul_add with a bias)
    must be a nearest representable value of the EXACT a*b+c, checked in rational arithmetic
    -- a conversion from float64 by way of float32 is one ulp off about once in 10^5 values."""
    from fractions import Fraction
    g = torch.Generator().manual_seed(0)
    n = 400_000
    x = torch.randn(1, 1, 1, n, generator=g).half().permute(0, 3, 1, 2)  # [1, n, 1, 1]: a channel each
    scale, shift = torch.randn(n, generator=g).half(), torch.randn(n, generator=g).half()
    mask = torch.ones(1, 1, 1, 1, dtype=torch.int32)
    got, _ = O.mul_add(x, mask, scale, shift)
    got = got.flatten()
    exact64 = x.flatten().double() * scale.double() + shift.double()  # exact: 22 + 11 bits, close exponents
    # candidates: every value where the two-step conversion and the direct one disagree, plus a sample
    two_step = exact64.float().half()
    idx = (two_step != torch.from_numpy(exact64.numpy().astype(np.float16))).nonzero().flatten().tolist()
    assert len(idx) >= 1, "no double-rounding candidate among the inputs: the test pins nothing"
    idx += list(range(0, n, 997))
    for i in idx:
        ex = Fraction(float(x.flatten()[i])) * Fraction(float(scale[i])) + Fraction(float(shift[i]))
        r = np.float16(float(got[i]))
        err = abs(Fraction(float(r)) - ex)
        for nb in (np.nextafter(r, np.float16(np.inf)), np.nextafter(r, np.float16(-np.inf))):
            assert err <= abs(Fraction(float(nb)) - ex), (i, float(r), float(nb))
    # DCAdd: s = a*wa, then fma(b, wb, s)
    a, b = x, torch.randn(1, n, 1, 1, generator=g).half()
    out, _ = O.add(a, mask, b, mask, None, 0.5, -1.25, 0, False)
    out = out.flatten()
    s = (a.flatten() * torch.tensor(0.5).half())
    for i in idx[:200]:
        ex = Fraction(float(b.flatten()[i])) * Fraction(-1.25) + Fraction(float(s[i]))
        r = np.float16(float(out[i]))
        err = abs(Fraction(float(r)) - ex)
        for nb in (np.nextafter(r, np.float16(np.inf)), np.nextafter(r, np.float16(-np.inf))):
            assert err <= abs(Fraction(float(nb)) - ex), (i, float(r), float(nb))


# --------------------------------------------------------------------------------------------
# Branches that the operator-level loops above do not reach
# --------------------------------------------------------------------------------------------
def test_sigmoid_and_swish_against_library():
    """Activation ids 4 / 5 (other_nn_layers.cu:36-44, 106-121) against torch.sigmoid / F.silu:
    fp32 to a few ulp; fp16 = the fp32 value rounded once (at most one fp16 ulp apart from the
    library's own rounding of its fp32 result, and equal almost everywhere)."""
    g = torch.Generator().manual_seed(41)
    x = torch.cat([torch.randn(4000, generator=g) * 4, torch.tensor([0.0, -0.0, 20.0, -20.0, 1e-4, -1e-4])])
    for act, lib in ((O.ACT_SIGMOID, torch.sigmoid), (O.ACT_SWISH, F.silu)):
        got = O.activation(x.clone(), act)
        want = lib(x.double())
        assert torch.allclose(got.double(), want, rtol=3e-7, atol=1e-9), act
        xh = x.half()
        got_h = O.activation(xh.clone(), act)
        assert got_h.dtype == torch.float16
        want_h = lib(xh.double())
        # spacing of fp16 at the result's magnitude: 2^-10 relative (2^-24 absolute floor)
        ulp = torch.maximum(want_h.abs() * 2.0 ** -10, torch.tensor(2.0 ** -24, dtype=torch.float64))
        assert ((got_h.double() - want_h).abs() <= 0.5 * ulp * (1 + 1e-3)).all(), act  # correctly rounded
    # a sign error or a missing "x *" would fail these closed forms
    assert O.activation(torch.tensor([0.0]), O.ACT_SIGMOID).item() == 0.5
    assert O.activation(torch.tensor([2.0]), O.ACT_SWISH).item() == pytest.approx(2.0 / (1.0 + np.exp(-2.0)), rel=1e-6)
    assert O.activation(torch.tensor([-30.0]), O.ACT_SIGMOID).item() < 1e-12


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("mode", [O.TRUNC_NORM, O.TRUNC_RMS])
@pytest.mark.parametrize("act", [1, 3])
def test_norm_rms_truncation_against_loops(dtype, mode, act):
    """other_nn_layers.cu:664-719: keep iff sqrt(sum D^2) (norm) or sqrt(sum D^2 / C) (rms)
    exceeds the threshold.  The loop statement sums in float64; pixels whose statistic lies
    within 2 % of the threshold are left out of the case (there the summation order of the
    tensor's type decides)."""
    rng = np.random.default_rng(77 + mode)
    B, C, H, W = 1, 6, 6, 7
    thr = 0.45 if mode == O.TRUNC_NORM else 0.2
    delta = (rng.standard_normal((B, C, H, W)) * 0.25).astype(dtype)
    prev = rng.standard_normal((B, C, H, W)).astype(dtype)
    trunc = (rng.standard_normal((B, C, H, W)) * 0.05).astype(dtype)
    mask = (rng.random((B, 1, H, W)) < 0.7).astype(np.int32)
    _, _, _, _, stat = bf.activate_truncate_sum(delta, prev, trunc, mask, thr, act, mode)
    near = np.abs(stat - thr) < 0.02 * thr
    mask = np.where(near, 0, mask).astype(np.int32)   # drop near-tie pixels from the case
    wd, wp, wt, wm, stat = bf.activate_truncate_sum(delta, prev, trunc, mask, thr, act, mode)
    kept, dropped = int(wm.sum()), int(mask.sum() - wm.sum())
    assert kept >= 5 and dropped >= 5, (kept, dropped)  # both branches are exercised
    d, p, t, m = (torch.from_numpy(v.copy()) for v in (delta, prev, trunc, mask))
    O.activate_truncate(d, p, t, m, thr, act, mode)
    assert np.array_equal(_np(m), wm)
    assert np.array_equal(_np(p), wp)
    assert np.array_equal(_np(t), wt)
    on = np.broadcast_to(wm != 0, wd.shape)
    assert np.array_equal(_np(d)[on], wd[on])
    # the two modes differ by exactly the factor sqrt(C): the same input under the other mode
    # with the threshold scaled accordingly takes the same decisions
    other = O.TRUNC_RMS if mode == O.TRUNC_NORM else O.TRUNC_NORM
    thr2 = thr / np.sqrt(C) if mode == O.TRUNC_NORM else thr * np.sqrt(C)
    d2, p2, t2, m2 = (torch.from_numpy(v.copy()) for v in (delta, prev, trunc, mask))
    O.activate_truncate(d2, p2, t2, m2, float(thr2), act, other)
    assert np.array_equal(_np(m2), wm)


@pytest.mark.parametrize("act", [1, 2, 3, 5])
def test_accumulate_with_activation_telescopes(act):
    """mode < 0 with an activation (activate_no_truncation, other_nn_layers.cu:378-394):
    prev += delta and delta := act(prev_new) - act(prev_old) on active pixels.  Over T frames
    the emitted deltas of a pixel telescope to act(prev_T) - act(prev_0), the cache is the plain
    sum of the incoming deltas, and an inactive pixel changes nothing."""
    g = torch.Generator().manual_seed(5 + act)
    B, C, H, W, T = 1, 3, 5, 6, 6
    prev0 = torch.randn(B, C, H, W, generator=g, dtype=torch.float64) * 2
    prev = prev0.clone()
    emitted = torch.zeros_like(prev)
    incoming = torch.zeros_like(prev)
    for _ in range(T):
        delta = torch.randn(B, C, H, W, generator=g, dtype=torch.float64)
        mask = (torch.rand(B, 1, H, W, generator=g) < 0.6).to(torch.int32)
        raw = delta.clone()
        before = prev.clone()
        O.activate_truncate(delta, prev, None, mask, 0.0, act, O.TRUNC_NONE)
        on = (mask != 0).expand_as(delta)
        assert torch.equal(delta[~on], raw[~on]) and torch.equal(prev[~on], before[~on])
        emitted += torch.where(on, delta, torch.zeros_like(delta))
        incoming += torch.where(on, raw, torch.zeros_like(raw))
    lib = {1: torch.relu, 2: lambda v: v.clamp(0, 6), 3: lambda v: F.leaky_relu(v, float(np.float32(0.1))),  # the slope is a C float
           5: F.silu}[act]
    assert torch.allclose(prev, prev0 + incoming, rtol=0, atol=1e-12)
    # sigmoid / swish are evaluated in float32 whatever the tensor's type
    assert torch.allclose(emitted, lib(prev) - lib(prev0), rtol=0, atol=1e-12 if act < 4 else 1e-5)


@pytest.mark.parametrize("act", [0, 1, 2])
def test_add_dense_out_against_indexing(act):
    """DCAdd(dense_out=True), sparse_layers.py:1140-1172: the cache takes the weighted sum on
    the union of the masks and act(cache) is returned for EVERY pixel, as a plain tensor."""
    rng = np.random.default_rng(11 + act)
    B, C, H, W = 2, 3, 5, 4
    a, b, prev = (rng.standard_normal((B, C, H, W)).astype(np.float32) * 3 for _ in range(3))
    ma = (rng.random((B, 1, H, W)) < 0.5).astype(np.int32)
    mb = (rng.random((B, 1, H, W)) < 0.5).astype(np.int32)
    a_p = np.where(ma != 0, a, np.nan).astype(np.float32)   # inactive operands must not be read
    b_p = np.where(mb != 0, b, np.nan).astype(np.float32)
    want, want_prev = bf.add_dense_out(a, ma, b, mb, prev, 0.5, -2.0, act)
    p = torch.from_numpy(prev.copy())
    out, mask = O.add(torch.from_numpy(a_p), torch.from_numpy(ma), torch.from_numpy(b_p), torch.from_numpy(mb),
                      p, 0.5, -2.0, act, dense_out=True)
    assert mask is None
    assert np.allclose(_np(p), want_prev, rtol=1e-6, atol=1e-6)
    assert np.allclose(_np(out), want, rtol=1e-6, atol=1e-6)
    assert ((ma | mb) == 0).any() and ((ma & mb) != 0).any()   # all four mask combinations occur


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_add_to_dense_against_indexing(dtype):
    rng = np.random.default_rng(3)
    B, C, H, W = 2, 5, 4, 6
    a = rng.standard_normal((B, C, H, W)).astype(dtype)
    b = rng.standard_normal((B, C, H, W)).astype(dtype)
    m = (rng.random((B, 1, H, W)) < 0.5).astype(np.int32)
    want = bf.add_to_dense(a, b, m)
    a_p = np.where(m != 0, a, np.nan).astype(dtype)
    tb = torch.from_numpy(b.copy())
    O.add_to_dense(torch.from_numpy(a_p), tb, torch.from_numpy(m))
    assert np.array_equal(_np(tb), want)
    # the activation variant also turns `a` into act(b) on every pixel
    ta, tb = torch.from_numpy(a.copy()), torch.from_numpy(b.copy())
    O.add_to_dense(ta, tb, torch.from_numpy(m), act=1)
    assert np.array_equal(_np(tb), want)
    assert np.array_equal(_np(ta), np.maximum(want, 0))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("k", [3, 5])
def test_sparsify_dilated_against_window_loops(dtype, k):
    """DCSparsify(dilation=k), sparse_layers.py:1233-1244."""
    rng = np.random.default_rng(19 + k)
    B, C, H, W = 1, 3, 9, 8
    prev = rng.random((B, C, H, W)).astype(dtype)
    x = prev.copy()
    for _ in range(3):  # a few isolated changed pixels, one of them in a corner
        y0, x0 = rng.integers(0, H), rng.integers(0, W)
        x[0, :, y0, x0] += dtype(0.5)
    x[0, 1, 0, 0] -= dtype(0.4)
    x = (x + (rng.standard_normal(x.shape) * 0.004).astype(dtype)).astype(dtype)  # sub-threshold noise
    thr = 0.1
    wd, wm, wp = bf.sparsify_neighbourhood(x, prev, thr, k)
    assert 0 < wm.sum() < wm.size
    tp = torch.from_numpy(prev.copy())
    d, m = O.sparsify_dilated(torch.from_numpy(x), tp, thr, k)
    assert np.array_equal(_np(m), wm)
    assert np.array_equal(_np(tp), wp)
    on = np.broadcast_to(wm != 0, wd.shape)
    assert np.array_equal(_np(d)[on], wd[on])


@pytest.mark.parametrize("kernel,stride,padding,dilation", [
    ((2, 2), (1, 1), (0, 0), (2, 2)), ((3, 3), (1, 1), (2, 2), (2, 2)), ((3, 2), (2, 1), (2, 1), (2, 3)),
    ((2, 2), (2, 2), (1, 1), (3, 3))])
@pytest.mark.parametrize("mode", [0, 1])
def test_pool_with_dilation_against_loops_and_library(kernel, stride, padding, dilation, mode):
    """Window taps `dilation` pixels apart: against the dilated loop statement on a sparse mask,
    and (max) against F.max_pool2d(..., dilation=) with every pixel active."""
    rng = np.random.default_rng(23)
    B, C, H, W = 1, 3, 10, 10
    delta = rng.standard_normal((B, C, H, W)).astype(np.float32)
    prev = rng.standard_normal((B, C, H, W)).astype(np.float32)
    mask = (rng.random((B, 1, H, W)) < 0.3).astype(np.int32)
    want, wm = bf.pool(delta, prev, mask, kernel, stride, padding, mode, dilation)
    d_p = np.where(mask != 0, delta, np.nan).astype(np.float32)
    out, om = O.pool(torch.from_numpy(d_p), torch.from_numpy(prev), torch.from_numpy(mask), kernel, stride,
                     padding, dilation, mode)
    assert np.array_equal(_np(om), wm)
    on = np.broadcast_to(wm != 0, want.shape)
    assert np.allclose(_np(out)[on], want[on], rtol=1e-6, atol=1e-6)
    # torch's pooling refuses padding beyond half the window
    if mode == 0 and all(2 * p <= k for p, k in zip(padding, kernel)):
        ones = torch.ones(B, 1, H, W, dtype=torch.int32)
        d, p = torch.from_numpy(delta), torch.from_numpy(prev)
        out, om = O.pool(d, p, ones, kernel, stride, padding, dilation, 0)
        lib = (F.max_pool2d(p + d, kernel, stride, padding, dilation) - F.max_pool2d(p, kernel, stride, padding, dilation))
        assert out.shape == lib.shape and bool((om != 0).all())
        assert torch.allclose(out, lib, rtol=1e-6, atol=1e-6)
