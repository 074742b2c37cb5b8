"""Random-shape parity sweep: operators of the HIP library against the CPU oracle on shapes,
strides, paddings, densities and channel counts drawn from a fixed seed per case, so that
corners nobody thought of listing by hand (ragged maps, partial channel tiles, windows larger
than the map's remainder) are visited too.  Masks bit-exact, elementwise operators bit-exact,
contractions within the fp16 tolerance (2e-2 absolute)."""
import os
import random
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from oracle import delta_ops as ops  # noqa: E402
from util import DEV, assert_masked_close, assert_masked_equal, cl, poison, rand_mask  # noqa: E402

pytestmark = pytest.mark.gpu

KINDS = ["stem", "stem_act", "depthwise", "pool", "add_upsampled", "pointwise", "conv", "deconv", "small_conv_act"]


def hk():
    from deltacnn_amd import hip_kernels
    return hip_kernels


def _half_filter(wt, transposed=False, depthwise=False):
    from deltacnn_amd.filter_conversion import convert_half_filter
    return convert_half_filter(wt, pixel_wise=depthwise, transposed=transposed).to(DEV)


def _conv_and_fused_activation(x, mask, wt, filt, pk, stride, pad, cout, rnd, g):
    """dc_conv against the oracle, then dc_conv_act against dc_conv + dc_activate_truncate."""
    want, wm = ops.conv(x, mask, wt, None, stride, pad, (1, 1), 1)
    dx, dm = cl(poison(x, mask)), cl(mask)
    o1, m1 = hk().sparse_conv(dx, filt, dm, None, stride, pad, (1, 1), 1, c_out=cout, create_out_mask=True, packed_filter=pk)
    assert torch.equal(m1.cpu(), wm)
    assert_masked_close(o1, want, wm, 0, 2e-2, "conv")
    act, mode = rnd.choice([(1, 0), (2, 0), (3, 1), (1, 2)])
    prev = torch.randn(want.shape, generator=g).half()
    trunc = (torch.randn(want.shape, generator=g) * 0.01).half()
    p1, t1 = cl(prev), cl(trunc)
    hk().sparse_activation(o1, p1, t1, m1, 0.3, act, mode)
    p2, t2 = cl(prev), cl(trunc)
    o2, m2 = hk().sparse_conv_activation(dx, filt, dm, None, p2, t2, 0.3, act, mode, stride, pad, (1, 1), 1, cout, packed_filter=pk)
    assert torch.equal(m1, m2) and torch.equal(p1, p2) and torch.equal(t1, t2)
    assert_masked_equal(o2, o1.cpu(), m1.cpu(), "fused activation")


@pytest.mark.parametrize("case", range(72))
def test_random_shape(lib, case):
    rnd = random.Random(7000 + case)
    g = torch.Generator().manual_seed(9000 + case)
    kind = KINDS[case % len(KINDS)]
    B = rnd.choice([1, 2])
    density = rnd.choice([0.0, 0.05, 0.5, 1.0])
    if kind in ("stem", "stem_act"):
        cin, cout = rnd.choice([1, 2, 3, 4]), rnd.choice([4, 8, 16, 20, 32, 48, 64])
        k, st = rnd.choice([1, 2, 3, 5, 7, 8]), rnd.choice([1, 2])
        pad = rnd.choice([0, k // 2, max(0, k // 2 - 1)])
        H, W = rnd.randint(k + 1, 70), rnd.randint(k + 1, 70)
        mask = rand_mask(g, B, H, W, max(density, 0.05))
        x = (torch.randn(B, cin, H, W, generator=g) * (0.01 + rand_mask(g, B, H, W, 0.5).float())).half()
        wt = (torch.randn(cout, cin, k, k, generator=g) / (cin * k * k) ** 0.5).half()
        filt = _half_filter(wt)
        pk = hk().pack_filter(filt, cin, cout, 1)
        if kind == "stem":
            want, wm = ops.conv(x, mask, wt, None, (st, st), (pad, pad), (1, 1), 1)
            out, om = hk().sparse_conv(cl(poison(x, mask)), filt, cl(mask), None, (st, st), (pad, pad), (1, 1), 1,
                                       c_out=cout, create_out_mask=True, packed_filter=pk)
            assert torch.equal(om.cpu(), wm)
            assert_masked_close(out, want, wm, 0, 2e-2, "out")
        else:
            _conv_and_fused_activation(x, mask, wt, filt, pk, (st, st), (pad, pad), cout, rnd, g)
    elif kind == "depthwise":
        C, st = rnd.choice([8, 16, 24, 40, 64, 136]), rnd.choice([1, 2])
        H, W = rnd.choice([(rnd.randint(5, 40), rnd.randint(5, 40)), (rnd.randint(380, 420), rnd.randint(380, 420))])
        mask = rand_mask(g, B, H, W, density)
        x = torch.randn(B, C, H, W, generator=g).half()
        wt = (torch.randn(C, 1, 3, 3, generator=g) / 3).half()
        filt = _half_filter(wt, depthwise=True)
        want, wm = ops.conv(x, mask, wt, None, (st, st), (1, 1), (1, 1), C)
        out, om = hk().sparse_conv(cl(poison(x, mask)), filt, cl(mask), None, (st, st), (1, 1), (1, 1), C, c_out=C,
                                   create_out_mask=True)
        assert torch.equal(om.cpu(), wm)
        assert_masked_close(out, want, wm, 0, 2e-2, "out")
    elif kind == "pool":
        C, K, st, mode = rnd.choice([8, 16, 24, 64, 128, 520]), rnd.choice([2, 3]), rnd.choice([1, 2]), rnd.choice([0, 1])
        pad = rnd.choice([0, 1]) if K == 3 else 0
        H, W = rnd.randint(K + 1, 40), rnd.randint(K + 1, 40)
        mask = rand_mask(g, B, H, W, density)
        x, prev = torch.randn(B, C, H, W, generator=g).half(), torch.randn(B, C, H, W, generator=g).half()
        want, wm = ops.pool(x, prev if mode == 0 else None, mask, (K, K), (st, st), (pad, pad), (1, 1), mode)
        out, om = hk().sparse_pooling(cl(poison(x, mask)), cl(prev) if mode == 0 else None, (K, K), cl(mask), (st, st),
                                      (pad, pad), (1, 1), pooling_mode_int=mode)
        assert torch.equal(om.cpu(), wm)
        assert_masked_equal(out, want, wm, "out")
    elif kind == "add_upsampled":
        C, sc, act = rnd.choice([3, 8, 32, 72, 136]), rnd.choice([2, 4, 8]), rnd.choice([-1, 1, 3])
        h, w = rnd.randint(1, 9), rnd.randint(1, 9)
        H, W = h * sc, w * sc
        ma, mb = rand_mask(g, B, H, W, 0.3), rand_mask(g, B, h, w, 0.5)
        a, b = torch.randn(B, C, H, W, generator=g).half(), torch.randn(B, C, h, w, generator=g).half()
        prev = torch.randn(B, C, H, W, generator=g).half() if act > 0 else None
        up, um = ops.upsample(b, mb, sc)
        wp = prev.clone() if act > 0 else None
        want, wm = ops.add(a, ma, up, um, wp, 0.75, -0.5, act, False)
        dp = cl(prev) if act > 0 else None
        out = torch.full((B, C, H, W), float("nan"), dtype=torch.half, device=DEV).contiguous(memory_format=torch.channels_last)
        mo = torch.full((B, 1, H, W), -3, dtype=torch.int32, device=DEV)
        hk().sparse_add_upsampled(cl(poison(a, ma)), cl(poison(b, mb)), dp, out, cl(ma), cl(mb), mo, 0.75, -0.5, act, sc)
        assert torch.equal(mo.cpu(), wm)
        assert_masked_equal(out, want, wm, "out")
        if act > 0:
            assert torch.equal(dp.cpu(), wp)
    elif kind == "pointwise":
        cin, cout = rnd.choice([8, 24, 64, 136, 320, 448]), rnd.choice([4, 20, 64, 80, 128, 256])
        H, W = rnd.randint(5, 70), rnd.randint(5, 70)
        mask = rand_mask(g, B, H, W, density)
        x = torch.randn(B, cin, H, W, generator=g).half()
        wt = (torch.randn(cout, cin, 1, 1, generator=g) / cin ** 0.5).half()
        filt = _half_filter(wt)
        pk = hk().pack_filter(filt, cin, cout, 1)
        want, wm = ops.conv(x, mask, wt, None, (1, 1), (0, 0), (1, 1), 1)
        out, om = hk().sparse_conv(cl(poison(x, mask)), filt, cl(mask), None, (1, 1), (0, 0), (1, 1), 1, c_out=cout,
                                   create_out_mask=True, packed_filter=pk)
        assert torch.equal(om.cpu(), wm)
        assert_masked_close(out, want, wm, 0, 2e-2, "out")
    elif kind == "conv":
        cin, cout = rnd.choice([16, 32, 64, 128, 256, 320]), rnd.choice([16, 24, 64, 128, 256])
        k, st, dil = rnd.choice([3, 3, 5]), rnd.choice([1, 1, 2]), rnd.choice([1, 1, 2])
        H, W = rnd.randint(20, 90), rnd.randint(20, 90)
        pad = dil * (k // 2)
        mask = rand_mask(g, 1, H, W, density)
        x = torch.randn(1, cin, H, W, generator=g).half()
        wt = (torch.randn(cout, cin, k, k, generator=g) / (cin * k * k) ** 0.5).half()
        filt = _half_filter(wt)
        pk = hk().pack_filter(filt, cin, cout, 1)
        want, wm = ops.conv(x, mask, wt, None, (st, st), (pad, pad), (dil, dil), 1)
        out, om = hk().sparse_conv(cl(poison(x, mask)), filt, cl(mask), None, (st, st), (pad, pad), (dil, dil), 1,
                                   c_out=cout, create_out_mask=True, packed_filter=pk)
        assert torch.equal(om.cpu(), wm)
        assert_masked_close(out, want, wm, 0, 2e-2, "out")
    elif kind == "deconv":
        cin, cout = rnd.choice([8, 16, 64, 128, 256]), rnd.choice([8, 16, 64, 128])
        k, st = rnd.choice([(4, 2), (2, 2), (3, 2), (8, 4), (6, 4), (3, 1), (2, 4)])
        H, W = rnd.randint(3, 40), rnd.randint(3, 40)
        pad = rnd.choice([0, max(0, (k - st) // 2)])
        mask = rand_mask(g, B, H, W, density)
        x = torch.randn(B, cin, H, W, generator=g).half()
        wt = (torch.randn(cin, cout, k, k, generator=g) / (cin * k * k / st / st) ** 0.5).half()
        filt = _half_filter(wt, transposed=True)
        pk = hk().pack_filter(filt, cin, cout, 1, transposed=True)
        want, wm = ops.deconv(x, mask, wt, None, (st, st), (pad, pad), (1, 1), 1)
        out, om = hk().sparse_deconv(cl(poison(x, mask)), filt, cl(mask), None, (st, st), (pad, pad), (1, 1), 1,
                                     c_out=cout, create_out_mask=True, packed_filter=pk)
        assert torch.equal(om.cpu(), wm)
        assert_masked_close(out, want, wm, 0, 2e-2, "out")
    else:  # small K x K layers with the activation fused where one wavefront holds all channels
        cin, cout = rnd.choice([8, 16, 32, 64]), rnd.choice([4, 16, 24, 32, 64])
        k, st = rnd.choice([3, 3, 5]), rnd.choice([1, 2])
        H, W = rnd.randint(6, 70), rnd.randint(6, 70)
        mask = rand_mask(g, B, H, W, max(density, 0.05))
        x = (torch.randn(B, cin, H, W, generator=g) * (0.01 + rand_mask(g, B, H, W, 0.5).float())).half()
        wt = (torch.randn(cout, cin, k, k, generator=g) / (cin * k * k) ** 0.5).half()
        filt = _half_filter(wt)
        pk = hk().pack_filter(filt, cin, cout, 1)
        _conv_and_fused_activation(x, mask, wt, filt, pk, (st, st), (k // 2, k // 2), cout, rnd, g)


@pytest.mark.parametrize("case", range(48))
def test_random_rectangular_fp32(lib, case):
    """fp32 with everything unequal in y and x (window, stride, padding, dilation), grouped
    channels and a bias: the generic kernels' index arithmetic.  1e-4 relative."""
    from deltacnn_amd.filter_conversion import convert_filter_out_channels_last
    rnd = random.Random(17000 + case)
    g = torch.Generator().manual_seed(19000 + case)
    kind = ["conv", "deconv", "pool"][case % 3]
    B = rnd.choice([1, 2, 3])
    density = rnd.choice([0.05, 0.3, 1.0])
    K = (rnd.randint(1, 5), rnd.randint(1, 5))
    H, W = rnd.randint(6, 33), rnd.randint(6, 33)
    mask = rand_mask(g, B, H, W, density)
    if kind == "conv":
        groups = rnd.choice([1, 1, 2, 4])
        cin, cout = groups * rnd.choice([1, 3, 4, 9]), groups * rnd.choice([1, 2, 4, 7])
        st, dil = (rnd.randint(1, 3), rnd.randint(1, 3)), (rnd.randint(1, 2), rnd.randint(1, 2))
        pad = (rnd.randint(0, dil[0] * (K[0] - 1)), rnd.randint(0, dil[1] * (K[1] - 1)))
        # a window larger than the padded map has no output: grow the map instead
        H = max(H, dil[0] * (K[0] - 1) + 1 - 2 * pad[0])
        W = max(W, dil[1] * (K[1] - 1) + 1 - 2 * pad[1])
        mask = rand_mask(g, B, H, W, density)
        x = torch.randn(B, cin, H, W, generator=g)
        wt = torch.randn(cout, cin // groups, *K, generator=g) / (cin // groups * K[0] * K[1]) ** 0.5
        bias = torch.randn(cout, generator=g) if rnd.random() < 0.5 else None
        want, wm = ops.conv(x, mask, wt, bias, st, pad, dil, groups)
        out, om = hk().sparse_conv(cl(poison(x, mask)), convert_filter_out_channels_last(wt).to(DEV), cl(mask),
                                   bias.to(DEV) if bias is not None else None, st, pad, dil, groups, c_out=cout,
                                   create_out_mask=True)
        assert out.shape == want.shape and torch.equal(om.cpu(), wm)
        assert_masked_close(out, want, wm, 1e-4, 1e-5, "out")
    elif kind == "deconv":
        cin, cout = rnd.choice([1, 3, 8, 17]), rnd.choice([1, 4, 6, 13])
        st = (rnd.randint(1, 3), rnd.randint(1, 3))
        p = rnd.randint(0, min(K[0], K[1]) - 1)
        x = torch.randn(B, cin, H, W, generator=g)
        wt = torch.randn(cin, cout, *K, generator=g) / (cin * K[0] * K[1]) ** 0.5
        bias = torch.randn(cout, generator=g) if rnd.random() < 0.5 else None
        want, wm = ops.deconv(x, mask, wt, bias, st, (p, p), (1, 1), 1)
        out, om = hk().sparse_deconv(cl(poison(x, mask)), convert_filter_out_channels_last(wt, transposed=True).to(DEV),
                                     cl(mask), bias.to(DEV) if bias is not None else None, st, (p, p), (1, 1), 1,
                                     c_out=cout, create_out_mask=True)
        assert out.shape == want.shape and torch.equal(om.cpu(), wm)
        assert_masked_close(out, want, wm, 1e-4, 1e-5, "out")
    else:
        C, mode = rnd.choice([1, 4, 5, 12, 68]), rnd.choice([0, 1])
        K = (max(K[0], 2), max(K[1], 2))
        st = (rnd.randint(1, K[0]), rnd.randint(1, K[1]))
        pad = (rnd.randint(0, K[0] // 2), rnd.randint(0, K[1] // 2))
        x, prev = torch.randn(B, C, H, W, generator=g), torch.randn(B, C, H, W, generator=g)
        want, wm = ops.pool(x, prev if mode == 0 else None, mask, K, st, pad, (1, 1), mode)
        out, om = hk().sparse_pooling(cl(poison(x, mask)), cl(prev) if mode == 0 else None, K, cl(mask), st, pad, (1, 1),
                                      pooling_mode_int=mode)
        assert out.shape == want.shape and torch.equal(om.cpu(), wm)
        assert_masked_close(out, want, wm, 1e-5, 1e-6, "out")


ELEMENTWISE = ["sparsify", "activate_truncate", "accumulate", "densify", "add", "add_to_dense", "mul_add", "concat",
               "upsample"]


@pytest.mark.parametrize("case", range(108))
def test_random_elementwise(lib, case):
    """The bandwidth operators in both types on any channel count (odd ones included) and on maps
    on either side of 2^18 pixels, where the per-pixel kernels hand over to the scanning ones.
    Bit-exact (fp32 multiply-add with a bias: 1e-6, the oracle fuses in fp64)."""
    rnd = random.Random(27000 + case)
    g = torch.Generator().manual_seed(29000 + case)
    kind = ELEMENTWISE[case % len(ELEMENTWISE)]
    dtype = rnd.choice([torch.float32, torch.float16])
    big = rnd.random() < 0.25
    if big:
        B, H, W = 2, rnd.randint(300, 340), rnd.randint(440, 480)
        C = rnd.choice([3, 8, 12, 24, 33, 40])
    else:
        B, H, W = rnd.choice([1, 2, 3]), rnd.randint(1, 40), rnd.randint(1, 40)
        C = rnd.randint(1, 140)
    density = rnd.choice([0.0, 0.03, 0.3, 1.0])
    mask = rand_mask(g, B, H, W, density)
    x = torch.randn(B, C, H, W, generator=g).to(dtype)
    nan_like = lambda t: torch.full_like(t, float("nan"))  # noqa: E731
    if kind == "sparsify":
        prev = torch.randn(B, C, H, W, generator=g).to(dtype)
        xin = torch.where(mask != 0, (prev.float() + torch.randn(B, C, H, W, generator=g) * 0.5).to(dtype), prev)
        wp = prev.clone()
        want, wm = ops.sparsify(xin, wp, 0.25)
        dp, dx = cl(prev), cl(xin)
        dd, dm = nan_like(dx), torch.full((B, 1, H, W), -7, dtype=torch.int32, device=DEV)
        hk().sparsify(dx, dp, dd, dm, 0.25)
        assert torch.equal(dm.cpu(), wm) and torch.equal(dp.cpu(), wp)
        assert_masked_equal(dd, want, wm, "delta")
    elif kind in ("activate_truncate", "accumulate"):
        act = rnd.choice([1, 2, 3])
        mode = 0 if kind == "activate_truncate" else -1
        prev = (torch.randn(B, C, H, W, generator=g) * 2).to(dtype)
        trunc = (torch.randn(B, C, H, W, generator=g) * 0.005).to(dtype)
        delta = (x.float() * (0.005 + 0.5 * rand_mask(g, B, H, W, 0.5).float())).to(dtype)
        w = [delta.clone(), prev.clone(), trunc.clone(), mask.clone()]
        ops.activate_truncate(*w, 0.1, act, mode)
        d = [cl(poison(delta, mask)), cl(prev), cl(trunc), cl(mask)]
        hk().sparse_activation(*d, 0.1, act, mode)
        assert torch.equal(d[3].cpu(), w[3])
        assert_masked_equal(d[0], w[0], w[3], "delta")
        assert torch.equal(d[1].cpu(), w[1]) and torch.equal(d[2].cpu(), w[2])
    elif kind == "densify":
        prev = torch.randn(B, C, H, W, generator=g).to(dtype)
        wp = prev.clone()
        ops.activate_truncate(x.clone(), wp, None, mask.clone(), 0.0, 0, -1)
        dp = cl(prev)
        out = nan_like(dp)
        hk().densify(cl(poison(x, mask)), dp, out, cl(mask))
        assert torch.equal(dp.cpu(), wp) and torch.equal(out.cpu(), wp)
    elif kind == "add":
        act = rnd.choice([-1, 1, 2])
        wa, wb = rnd.choice([(1.0, 1.0), (0.5, -1.25), (2.0, 0.3)])
        mb = rand_mask(g, B, H, W, rnd.choice([0.0, 0.2, 1.0]))
        b = torch.randn(B, C, H, W, generator=g).to(dtype)
        prev = torch.randn(B, C, H, W, generator=g).to(dtype) if act > 0 else None
        wp = prev.clone() if act > 0 else None
        want, wm = ops.add(x, mask, b, mb, wp, wa, wb, act, False)
        dp = cl(prev) if act > 0 else None
        out = nan_like(cl(x))
        mo = torch.full((B, 1, H, W), -3, dtype=torch.int32, device=DEV)
        hk().sparse_add_tensors(cl(poison(x, mask)), cl(poison(b, mb)), dp, out, cl(mask), cl(mb), mo, wa, wb, act, False)
        assert torch.equal(mo.cpu(), wm)
        assert_masked_equal(out, want, wm, "out")
        if act > 0:
            assert torch.equal(dp.cpu(), wp)
    elif kind == "add_to_dense":
        b = torch.randn(B, C, H, W, generator=g).to(dtype)
        wb = b.clone()
        ops.add_to_dense(x, wb, mask)
        db = cl(b)
        hk().sparse_add_to_dense_tensor(cl(poison(x, mask)), db, cl(mask))
        assert torch.equal(db.cpu(), wb)
    elif kind == "mul_add":
        scale = torch.randn(C, generator=g).to(dtype)
        bias = torch.randn(C, generator=g).to(dtype) if rnd.random() < 0.5 else None
        want, wm = ops.mul_add(x, mask, scale, bias)
        dx, dm = cl(poison(x, mask)), cl(mask)
        out, om = nan_like(dx), torch.zeros_like(dm)
        hk().sparse_mul_add(dx, dm, out, om, scale.to(DEV), None if bias is None else bias.to(DEV))
        assert torch.equal(om.cpu(), wm)
        if dtype == torch.float32 and bias is not None:
            assert_masked_close(out, want, wm, 1e-6, 1e-6, "out")
        else:
            assert_masked_equal(out, want, wm, "out")
    elif kind == "concat":
        Cb = rnd.randint(1, 40) if big else rnd.randint(1, 140)
        mb = rand_mask(g, B, H, W, rnd.choice([0.0, 0.2, 1.0]))
        b = torch.randn(B, Cb, H, W, generator=g).to(dtype)
        want, wm = ops.concatenate(x, mask, b, mb)
        out, om = hk().sparse_concatenate((cl(poison(x, mask)), cl(mask)), (cl(poison(b, mb)), cl(mb)))
        assert torch.equal(om.cpu(), wm)
        assert_masked_equal(out, want, wm, "out")
    else:
        scale = rnd.choice([2, 2, 4]) if big else rnd.choice([2, 3, 4, 8])
        if big:
            x, mask = x[:, :, ::2, ::2].contiguous(), mask[:, :, ::2, ::2].contiguous()
        want, wm = ops.upsample(x, mask, scale)
        out, om = hk().sparse_upsample(cl(poison(x, mask)), cl(mask), scale)
        assert torch.equal(om.cpu(), wm)
        assert_masked_equal(out, want, wm, "out")
