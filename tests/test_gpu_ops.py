"""Operator-level parity: every C-ABI operator against the CPU oracle on identical seeded
inputs.  Masks and pixel sets must match exactly; elementwise operators must match bit for
bit; contractions within 1e-4 relative (fp32) / 2e-2 absolute (fp16).  Inactive pixels of
every delta input are NaN-poisoned, so a kernel that reads them cannot pass.
"""
import pytest
import torch

from oracle import delta_ops as ops
from util import DEV, assert_masked_close, assert_masked_equal, cl, packed_form_exists, poison, rand_mask

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
# tolerance of results that pass through a transcendental or a reordered float sum: a few steps of the type
LOOSE = {torch.float32: 1e-5, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}
CHANNELS = [1, 3, 4, 8, 16, 31, 32, 33, 64, 96, 130, 256, 960, 1280, 2100]


def hk():
    import deltacnn_amd.hip_kernels as m
    return m


def _gen(seed):
    return torch.Generator().manual_seed(seed)


# ------------------------------------------------------------------------------- sparsify
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", CHANNELS)
def test_sparsify(lib, dtype, C):
    g = _gen(100 + C)
    B, H, W = 2, 13, 9
    prev = torch.randn(B, C, H, W, generator=g).to(dtype)
    x = prev.clone()
    upd = rand_mask(g, B, H, W, 0.3) != 0
    x = torch.where(upd, (x.float() + torch.randn(B, C, H, W, generator=g) * 0.5).to(dtype), x)
    # ties: a pixel whose largest |difference| equals the threshold exactly
    thr = 0.25
    x[0, :, 0, 0] = prev[0, :, 0, 0]
    x[0, 0, 0, 0] = 1.0
    prev[0, 0, 0, 0] = 0.75
    want_prev = prev.clone()
    want_delta, want_mask = ops.sparsify(x, want_prev, thr)

    d_prev, d_x = cl(prev), cl(x)
    d_delta = torch.full_like(d_x, float("nan"))
    d_mask = torch.full((B, 1, H, W), -7, dtype=torch.int32, device=DEV)
    hk().sparsify(d_x, d_prev, d_delta, d_mask, thr)
    assert torch.equal(d_mask.cpu(), want_mask)
    assert_masked_equal(d_delta, want_delta, want_mask, "delta")
    assert torch.equal(d_prev.cpu(), want_prev)
    # inactive pixels of delta are not written
    assert bool(d_delta.cpu()[(want_mask == 0).expand_as(want_delta)].isnan().all())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,H,W", [(24, 192, 192), (96, 96, 96), (3, 224, 224)])
def test_sparsify_large_map(lib, dtype, C, H, W):
    """Big enough that a lane holds several vectors of its pixel."""
    g = _gen(150 + C)
    B = 2
    prev = torch.randn(B, C, H, W, generator=g).to(dtype)
    upd = rand_mask(g, B, H, W, 0.2) != 0
    x = torch.where(upd, (prev.float() + torch.randn(B, C, H, W, generator=g) * 0.5).to(dtype), prev)
    want_prev = prev.clone()
    want_delta, want_mask = ops.sparsify(x, want_prev, 0.25)
    d_prev, d_x = cl(prev), cl(x)
    d_delta = torch.full_like(d_x, float("nan"))
    d_mask = torch.full((B, 1, H, W), -7, dtype=torch.int32, device=DEV)
    hk().sparsify(d_x, d_prev, d_delta, d_mask, 0.25)
    assert torch.equal(d_mask.cpu(), want_mask)
    assert_masked_equal(d_delta, want_delta, want_mask, "delta")
    assert torch.equal(d_prev.cpu(), want_prev)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,H,W", [(24, 192, 192), (96, 96, 96)])
def test_activate_truncate_large_map(lib, dtype, C, H, W):
    g = _gen(250 + C)
    B = 2
    mask = rand_mask(g, B, H, W, 0.3)
    prev = (torch.randn(B, C, H, W, generator=g) * 3).to(dtype)
    trunc = (torch.randn(B, C, H, W, generator=g) * 0.005).to(dtype)
    big = rand_mask(g, B, H, W, 0.5).float()
    delta = (torch.randn(B, C, H, W, generator=g) * (0.005 + 0.5 * big)).to(dtype)
    w = [delta.clone(), prev.clone(), trunc.clone(), mask.clone()]
    ops.activate_truncate(*w, 0.1, 2, 0)
    d = [cl(poison(delta, mask)), cl(prev), cl(trunc), cl(mask)]
    hk().sparse_activation(*d, 0.1, 2, 0)
    assert torch.equal(d[3].cpu(), w[3])
    assert_masked_equal(d[0], w[0], w[3], "delta")
    assert torch.equal(d[1].cpu(), w[1]) and torch.equal(d[2].cpu(), w[2])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,act,mode", [(40, 1, 0), (64, 3, 1), (8, 2, 2), (136, 1, 0)])
@pytest.mark.parametrize("density", [0.02, 0.6])
def test_activate_truncate_scanned_map(lib, dtype, C, act, mode, density):
    """Maps of 262144 pixels and more: mask scan and compaction per wavefront (uneven tail)."""
    g = _gen(260 + C)
    B, H, W = 2, 401, 331
    mask = rand_mask(g, B, H, W, density)
    prev = (torch.randn(B, C, H, W, generator=g) * 3).to(dtype)
    trunc = (torch.randn(B, C, H, W, generator=g) * 0.005).to(dtype)
    big = rand_mask(g, B, H, W, 0.5).float()
    delta = (torch.randn(B, C, H, W, generator=g) * (0.005 + 0.5 * big)).to(dtype)
    w = [delta.clone(), prev.clone(), trunc.clone(), mask.clone()]
    ops.activate_truncate(*w, 0.1, act, mode)
    d = [cl(poison(delta, mask)), cl(prev), cl(trunc), cl(mask)]
    hk().sparse_activation(*d, 0.1, act, mode)
    if mode == 0:
        assert torch.equal(d[3].cpu(), w[3])
        assert_masked_equal(d[0], w[0], w[3], "delta")
        assert torch.equal(d[1].cpu(), w[1]) and torch.equal(d[2].cpu(), w[2])
    else:  # norm / rms: the sum order differs from the oracle's, decisions may differ at ties
        agree = (d[3].cpu() == w[3])
        assert float(agree.float().mean()) > 0.999
        both = (agree & (w[3] != 0)).to(torch.int32)
        assert_masked_equal(d[0], w[0], both, "delta")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [24, 64, 136])
@pytest.mark.parametrize("act", [-1, 1])
def test_add_scanned_map(lib, dtype, C, act):
    g = _gen(640 + C)
    B, H, W = 2, 401, 331
    ma, mb = rand_mask(g, B, H, W, 0.05), rand_mask(g, B, H, W, 0.3)
    a = torch.randn(B, C, H, W, generator=g).to(dtype)
    b = torch.randn(B, C, H, W, generator=g).to(dtype)
    prev = torch.randn(B, C, H, W, generator=g).to(dtype) if act > 0 else None
    w_prev = prev.clone() if act > 0 else None
    w_out, w_mask = ops.add(a, ma, b, mb, w_prev, 0.5, -1.25, act, False)
    d_prev = cl(prev) if act > 0 else None
    d_out = torch.full((B, C, H, W), float("nan"), dtype=dtype, device=DEV).contiguous(
        memory_format=torch.channels_last)
    d_mo = torch.full((B, 1, H, W), -3, dtype=torch.int32, device=DEV)
    hk().sparse_add_tensors(cl(poison(a, ma)), cl(poison(b, mb)), d_prev, d_out, cl(ma), cl(mb), d_mo,
                            0.5, -1.25, act, False)
    assert torch.equal(d_mo.cpu(), w_mask)
    assert_masked_equal(d_out, w_out, w_mask, "out")
    if act > 0:
        assert torch.equal(d_prev.cpu(), w_prev)


# ------------------------------------------------------------------ activation + truncation
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", CHANNELS)
@pytest.mark.parametrize("act", [1, 2, 3])
def test_activate_truncate_max(lib, dtype, C, act):
    g = _gen(200 + C + act)
    B, H, W = 2, 11, 7
    mask = rand_mask(g, B, H, W, 0.5)
    scale = 3.0 if act == 2 else 1.0
    prev = (torch.randn(B, C, H, W, generator=g) * scale).to(dtype)
    trunc = (torch.randn(B, C, H, W, generator=g) * 0.005).to(dtype)
    big = rand_mask(g, B, H, W, 0.5).float()
    delta = (torch.randn(B, C, H, W, generator=g) * (0.005 + 0.5 * big)).to(dtype)
    thr = 0.1
    w_delta, w_prev, w_trunc, w_mask = delta.clone(), prev.clone(), trunc.clone(), mask.clone()
    ops.activate_truncate(w_delta, w_prev, w_trunc, w_mask, thr, act, 0)
    assert 0 < int(w_mask.sum()) < int(mask.sum())

    d_delta, d_prev, d_trunc, d_mask = cl(poison(delta, mask)), cl(prev), cl(trunc), cl(mask)
    hk().sparse_activation(d_delta, d_prev, d_trunc, d_mask, thr, act, 0)
    assert torch.equal(d_mask.cpu(), w_mask)
    assert_masked_equal(d_delta, w_delta, w_mask, "delta")
    assert torch.equal(d_prev.cpu(), w_prev)
    assert torch.equal(d_trunc.cpu(), w_trunc)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("act", [4, 5])
def test_activate_truncate_transcendental(lib, dtype, act):
    """sigmoid / swish go through exp: tolerance instead of bit equality, ties excluded."""
    g = _gen(300 + act)
    B, C, H, W = 1, 24, 9, 9
    mask = rand_mask(g, B, H, W, 0.6)
    prev = torch.randn(B, C, H, W, generator=g).to(dtype)
    trunc = torch.zeros(B, C, H, W).to(dtype)
    big = rand_mask(g, B, H, W, 0.5).float()
    delta = (torch.randn(B, C, H, W, generator=g) * (0.001 + 2.0 * big)).to(dtype)
    thr = 0.05
    w_delta, w_prev, w_trunc, w_mask = delta.clone(), prev.clone(), trunc.clone(), mask.clone()
    ops.activate_truncate(w_delta, w_prev, w_trunc, w_mask, thr, act, 0)
    d_delta, d_prev, d_trunc, d_mask = cl(poison(delta, mask)), cl(prev), cl(trunc), cl(mask)
    hk().sparse_activation(d_delta, d_prev, d_trunc, d_mask, thr, act, 0)
    assert torch.equal(d_mask.cpu(), w_mask)
    tol = LOOSE[dtype]
    assert_masked_close(d_delta, w_delta, w_mask, tol, tol, "delta")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mode", [1, 2])
@pytest.mark.parametrize("C", [8, 33, 96])
def test_activate_truncate_norm_modes(lib, dtype, mode, C):
    """norm / rms: pixels are either far above or far below the threshold."""
    g = _gen(400 + mode + C)
    B, H, W = 1, 10, 10
    mask = rand_mask(g, B, H, W, 0.7)
    prev = (torch.rand(B, C, H, W, generator=g) + 0.5).to(dtype)
    trunc = torch.zeros(B, C, H, W).to(dtype)
    big = rand_mask(g, B, H, W, 0.5).float()
    delta = ((torch.rand(B, C, H, W, generator=g) + 0.5) * (1e-4 + 0.5 * big)).to(dtype)
    thr = 0.2
    w = [delta.clone(), prev.clone(), trunc.clone(), mask.clone()]
    ops.activate_truncate(*w, thr, 1, mode)
    d = [cl(poison(delta, mask)), cl(prev), cl(trunc), cl(mask)]
    hk().sparse_activation(*d, thr, 1, mode)
    assert torch.equal(d[3].cpu(), w[3])
    assert_masked_equal(d[0], w[0], w[3], "delta")
    assert torch.equal(d[1].cpu(), w[1])
    assert torch.equal(d[2].cpu(), w[2])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [3, 17, 80, 84, 1280])
@pytest.mark.parametrize("act", [-1, 1])
def test_densify_accumulate(lib, dtype, C, act):
    g = _gen(500 + C)
    B, H, W = 2, 8, 12
    mask = rand_mask(g, B, H, W, 0.4)
    prev = torch.randn(B, C, H, W, generator=g).to(dtype)
    delta = torch.randn(B, C, H, W, generator=g).to(dtype)
    w_delta, w_prev = delta.clone(), prev.clone()
    ops.activate_truncate(w_delta, w_prev, None, mask, -1, act, -1)
    d_delta, d_prev, d_mask = cl(poison(delta, mask)), cl(prev), cl(mask)
    hk().sparse_activation(d_delta, d_prev, None, d_mask, -1, act, -1)
    assert torch.equal(d_prev.cpu(), w_prev)
    assert_masked_equal(d_delta, w_delta, mask, "delta")
    assert torch.equal(d_mask.cpu(), mask)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,H,W", [(3, 8, 12), (17, 8, 12), (64, 16, 9), (1280, 1, 1), (2100, 3, 3)])
def test_densify_fused(lib, dtype, C, H, W):
    """Accumulate + dense copy in one launch == accumulate, then clone."""
    g = _gen(550 + C)
    B = 2
    mask = rand_mask(g, B, H, W, 0.4)
    prev = torch.randn(B, C, H, W, generator=g).to(dtype)
    delta = torch.randn(B, C, H, W, generator=g).to(dtype)
    w_delta, w_prev = delta.clone(), prev.clone()
    ops.activate_truncate(w_delta, w_prev, None, mask, -1, -1, -1)
    d_prev = cl(prev)
    out = torch.full_like(d_prev, float("nan"))
    hk().densify(cl(poison(delta, mask)), d_prev, out, cl(mask))
    assert torch.equal(d_prev.cpu(), w_prev)
    assert torch.equal(out.cpu(), w_prev)


# ------------------------------------------------------------------------------------ add
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [3, 16, 24, 33, 160, 2100])
@pytest.mark.parametrize("act,dense_out", [(-1, False), (1, False), (-1, True), (2, True)])
@pytest.mark.parametrize("weights", [(1.0, 1.0), (0.5, -1.25)])
def test_add(lib, dtype, C, act, dense_out, weights):
    g = _gen(600 + C)
    B, H, W = 2, 9, 10
    ma, mb = rand_mask(g, B, H, W, 0.4), rand_mask(g, B, H, W, 0.3)
    a = torch.randn(B, C, H, W, generator=g).to(dtype)
    b = torch.randn(B, C, H, W, generator=g).to(dtype)
    need_prev = dense_out or act > 0
    prev = torch.randn(B, C, H, W, generator=g).to(dtype) if need_prev else None
    w_prev = prev.clone() if need_prev else None
    w_out, w_mask = ops.add(a, ma, b, mb, w_prev, weights[0], weights[1], act, dense_out)

    d_prev = cl(prev) if need_prev else None
    d_out = torch.full((B, C, H, W), float("nan"), dtype=dtype, device=DEV).contiguous(
        memory_format=torch.channels_last)
    d_mo = torch.full((B, 1, H, W), -3, dtype=torch.int32, device=DEV)
    hk().sparse_add_tensors(cl(poison(a, ma)), cl(poison(b, mb)), d_prev, d_out, cl(ma), cl(mb), d_mo,
                            weights[0], weights[1], act, dense_out)
    if dense_out:
        assert torch.equal(d_out.cpu(), w_out)
    else:
        assert torch.equal(d_mo.cpu(), w_mask)
        assert_masked_equal(d_out, w_out, w_mask, "out")
    if need_prev:
        assert torch.equal(d_prev.cpu(), w_prev)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [5, 64])
@pytest.mark.parametrize("act", [0, 1])
def test_add_to_dense(lib, dtype, C, act):
    g = _gen(700 + C)
    B, H, W = 1, 7, 9
    ma = rand_mask(g, B, H, W, 0.4)
    a = torch.randn(B, C, H, W, generator=g).to(dtype)
    b = torch.randn(B, C, H, W, generator=g).to(dtype)
    w_b = b.clone()
    ops.add_to_dense(a, w_b, ma)
    d_a, d_b = cl(poison(a, ma)), cl(b)
    hk().sparse_add_to_dense_tensor(d_a, d_b, cl(ma), act)
    assert torch.equal(d_b.cpu(), w_b)
    if act:
        assert torch.equal(d_a.cpu(), ops.activation(w_b, act))


# ------------------------------------------------------------------------------------ conv
CONVS = [
    # Cin, Cout, K, stride, padding, dilation, groups, H, W
    (3, 16, 3, 1, 1, 1, 1, 17, 13),
    (16, 32, 3, 1, 1, 1, 1, 16, 16),
    (3, 32, 3, 2, 1, 1, 1, 33, 31),
    (32, 32, 3, 1, 1, 1, 32, 15, 18),       # depthwise
    (96, 96, 3, 2, 1, 1, 96, 19, 17),       # depthwise stride 2
    (24, 24, 5, 1, 2, 1, 24, 12, 12),       # depthwise 5x5
    (16, 96, 1, 1, 0, 1, 1, 14, 14),
    (96, 24, 1, 1, 0, 1, 1, 9, 20),
    (144, 32, 1, 1, 0, 1, 1, 7, 7),
    (64, 64, 1, 2, 0, 1, 1, 11, 11),        # 1x1 stride 2 samples the mask
    (32, 48, 3, 1, 2, 2, 1, 14, 15),        # dilation 2
    (8, 8, 5, 2, 2, 1, 1, 13, 13),
    (8, 16, 7, 1, 3, 1, 1, 12, 10),         # 7x7 stride 1 (not dispatched by the reference)
    (3, 8, 7, 2, 3, 1, 1, 20, 22),
    (16, 16, 3, 1, (0, 1, 1, 0), 1, 1, 9, 9),   # (top, bottom, left, right)
    (40, 24, (1, 3), (1, 2), (0, 1), 1, 1, 8, 16),
    (12, 18, 3, 1, 1, 1, 3, 8, 8),          # general groups (fp32 only)
    (5, 7, 3, 1, 1, 1, 1, 9, 9),            # odd channels: fp16 padding rows/cols of the swizzle
    # stems on the matrix cores (fp16 packed): window rows as reduction steps
    (3, 16, 7, 1, 3, 1, 1, 37, 45),
    (3, 64, 3, 2, 1, 1, 1, 40, 41),
    (4, 24, 5, 1, 2, 1, 1, 19, 23),
    (1, 8, 3, 1, 1, 1, 1, 16, 16),
    (3, 48, 7, 2, 3, 1, 1, 33, 35),
    (2, 64, 8, 2, 3, 1, 1, 30, 30),
    (3, 32, 3, 2, 1, 1, 1, 400, 380),       # ... on a map of 2^18 pixels and more: only updated pixels are staged
    # layers large enough for the LDS-halo MFMA kernel (fp16 packed), one per arrangement / corner
    (64, 64, 3, 1, 1, 1, 1, 72, 70),        # two channel tiles per wave, steps split over two waves
    (64, 32, 3, 1, 1, 1, 1, 100, 100),      # ... over four waves (one channel group)
    (16, 64, 3, 1, 1, 1, 1, 120, 120),      # short reduction: one tile per wave, four channel groups
    (32, 256, 3, 1, 1, 1, 1, 90, 90),       # wide output on many tiles: two tiles per wave, no split
    (320, 32, 3, 1, 1, 1, 1, 40, 40),       # input channels staged in two chunks
    (128, 128, 3, 1, 1, 1, 1, 40, 40),      # few tiles, long reduction: eight waves, steps split four ways
    (64, 80, 3, 2, 1, 1, 1, 120, 121),      # stride 2
    (64, 48, 3, 1, 2, 2, 1, 80, 81),        # dilation 2
    (32, 64, 5, 1, 2, 1, 1, 64, 66),        # 5x5
    (24, 40, 3, 1, 1, 1, 1, 128, 130),      # partial reduction step and partial channel tile
    # thin layers (8 or 16 input channels) on large maps: several taps per reduction step
    (16, 16, 3, 1, 1, 1, 1, 200, 190),      # five steps, one channel tile
    (16, 32, 3, 2, 1, 1, 1, 520, 500),      # stride 2 on a map of 2^18 pixels and more: only updated pixels are staged
    (8, 24, 3, 1, 1, 1, 1, 130, 131),       # three steps, a partial channel tile
    (16, 64, 3, 1, 1, 1, 1, 160, 170),      # four channel tiles per wavefront
    (8, 8, 3, 2, 1, 1, 1, 400, 401),        # half a channel tile
    (16, 40, 2, 2, 0, 1, 1, 300, 300),      # 2 x 2 window
    (8, 48, (1, 3), 1, (0, 1), 1, 1, 150, 160),  # one window row
    (16, 16, 3, 1, 1, 1, 16, 726, 727),     # depthwise on a very large map: mask scan and compaction per wavefront
    (24, 24, 3, 1, 1, 1, 24, 600, 601),     # ... with idle lanes in the group
    (16, 16, 3, 2, 1, 1, 16, 600, 521),     # ... with a stride
    (16, 16, 3, 1, 1, 1, 16, 300, 301),     # ... narrow rows take the scan from 2^16 outputs on
    (64, 64, 3, 1, 1, 1, 64, 180, 181),     # depthwise on a large map: strips of four pixels per lane group
    (40, 40, 3, 1, 1, 1, 40, 180, 181),     # ... with idle lanes in the group
    (144, 144, 3, 1, 1, 1, 144, 130, 131),  # ... wide rows on 8 MB and more: filter through LDS
]


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


def _conv_case(dtype, cfg, seed, density, transposed=False):
    from deltacnn_amd.filter_conversion import convert_filter_out_channels_last, convert_half_filter
    Cin, Cout, K, s, p, d, groups, H, W = cfg
    K, s, d = _pair(K), _pair(s), _pair(d)
    p = _pair(p)
    g = _gen(seed)
    B = 2
    mask = rand_mask(g, B, H, W, density)
    x = torch.randn(B, Cin, H, W, generator=g).to(dtype)
    if transposed:
        wt = (torch.randn(Cin, Cout // groups, *K, generator=g) / (Cin * K[0] * K[1]) ** 0.5).to(dtype)
    else:
        wt = (torch.randn(Cout, Cin // groups, *K, generator=g) / (Cin // groups * K[0] * K[1]) ** 0.5).to(dtype)
    bias = torch.randn(Cout, generator=g).to(dtype)
    dw = groups == Cin == Cout and groups > 1
    if dtype == torch.float16:
        filt = convert_half_filter(wt, pixel_wise=dw, transposed=transposed)
    else:
        filt = convert_filter_out_channels_last(wt, transposed=transposed)
    return x, mask, wt, bias, filt, (K, s, p, d, groups)


def _check_conv(dtype, got, want, want_mask):
    if dtype == torch.float32:
        assert_masked_close(got, want, want_mask, 1e-4, 1e-5, "out")
    elif dtype == torch.bfloat16:  # one bfloat16 step is 2^-8 of the value: 2e-2 absolute or two steps
        assert_masked_close(got, want, want_mask, 2.0 ** -7, 2e-2, "out")
    else:
        assert_masked_close(got, want, want_mask, 0, 2e-2, "out")


def _conv_params(cfgs, transposed=False):
    """(dtype, cfg, packed) for every combination that exists: fp16 filters are defined for one
    group and depthwise only, and `packed` needs a packed form of the filter."""
    out = []
    for cfg in cfgs:
        cin, cout, k, groups = cfg[0], cfg[1], cfg[2], cfg[6]
        for dtype in DTYPES:
            if dtype == torch.float16 and groups > 1 and not (groups == cin == cout):
                continue
            out.append(pytest.param(dtype, cfg, False, id=f"{str(dtype)[6:]}-{'-'.join(str(v).replace(' ', '') for v in cfg)}"))
            if packed_form_exists(dtype, cin, cout, k, groups, transposed):
                out.append(pytest.param(dtype, cfg, True, id=f"{str(dtype)[6:]}-{'-'.join(str(v).replace(' ', '') for v in cfg)}-packed"))
    return out


@pytest.mark.parametrize("dtype,cfg,packed", _conv_params(CONVS))
@pytest.mark.parametrize("density", [0.05, 0.5, 1.0])
@pytest.mark.parametrize("use_bias", [False, True])
def test_conv(lib, dtype, cfg, density, use_bias, packed):
    groups, Cin, Cout = cfg[6], cfg[0], cfg[1]
    x, mask, wt, bias, filt, (K, s, p, d, groups) = _conv_case(dtype, cfg, 800 + Cin + Cout, density)
    want, want_mask = ops.conv(x, mask, wt, bias if use_bias else None, s, p, d, groups)
    d_filt = filt.to(DEV)
    pk = hk().pack_filter(d_filt, Cin, Cout, groups) if packed else None
    assert (pk is not None) == packed
    out, om = hk().sparse_conv(cl(poison(x, mask)), d_filt, cl(mask), bias.to(DEV) if use_bias else None,
                               s, p, d, groups, c_out=Cout, create_out_mask=True, packed_filter=pk)
    assert out.shape == want.shape
    assert torch.equal(om.cpu(), want_mask)
    _check_conv(dtype, out, want, want_mask)


RESIDENT = [  # Cin, Cout, K, stride, padding, dilation, groups, H, W (batch 2): at least 1024 output tiles
    (64, 64, 3, 1, 1, 1, 1, 256, 250),   # two channel tiles per wavefront, two reduction slices
    (64, 96, 3, 1, 1, 1, 1, 256, 256),   # two channel blocks
    (40, 64, 3, 1, 1, 1, 1, 250, 256),   # input channels that do not fill the second reduction step
    (56, 80, 3, 1, 1, 1, 1, 256, 250),   # a last channel block with one tile
    (64, 64, 3, 1, 1, 1, 1, 192, 184),   # 1104 tiles: just above the threshold
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["float16", "bfloat16"])
@pytest.mark.parametrize("cfg", RESIDENT, ids=lambda c: "-".join(str(v) for v in c))
@pytest.mark.parametrize("density", [0.02, 0.3, 1.0])
def test_conv_resident_filter(lib, dtype, cfg, density):
    """The resident-filter form of the K x K MFMA kernel (a workgroup walks over many tiles with
    the filter fragments in registers) against the oracle, with a bias on the dense case."""
    from deltacnn_amd import _lib
    groups, Cin, Cout = cfg[6], cfg[0], cfg[1]
    x, mask, wt, bias, filt, (K, s, p, d, groups) = _conv_case(dtype, cfg, 900 + Cin + Cout, density)
    use_bias = density == 1.0
    want, want_mask = ops.conv(x, mask, wt, bias if use_bias else None, s, p, d, groups)
    d_filt = filt.to(DEV)
    pk = hk().pack_filter(d_filt, Cin, Cout, groups)
    out, om = hk().sparse_conv(cl(poison(x, mask)), d_filt, cl(mask), bias.to(DEV) if use_bias else None,
                               s, p, d, groups, c_out=Cout, create_out_mask=True, packed_filter=pk)
    assert _lib.load().dc_last_kernels().decode() == "conv_res_mfma_kernel"
    assert torch.equal(om.cpu(), want_mask)
    _check_conv(dtype, out, want, want_mask)


@pytest.mark.parametrize("cfg,kernel", [
    ((32, 32, 3, 1, 1, 1, 1, 16, 16), "conv_patch_mfma_kernel"),
    ((64, 64, 3, 1, 1, 1, 1, 72, 70), "conv_lds_mfma_kernel"),
    ((16, 64, 3, 1, 1, 1, 1, 120, 120), "conv_lds_mfma_kernel"),
    ((320, 32, 3, 1, 1, 1, 1, 40, 40), "conv_lds_mfma_kernel"),
    ((64, 64, 3, 1, 1, 1, 1, 256, 250), "conv_res_mfma_kernel"),   # thin layers on >= 1024 tiles: resident filter
    ((32, 32, 3, 2, 1, 1, 1, 520, 500), "conv_lds_mfma_kernel"),   # one channel step: the per-tile kernel stays
    ((16, 32, 3, 2, 1, 1, 1, 520, 500), "conv_thin_mfma_kernel"),  # 8 / 16 input channels on a large map
    ((8, 24, 3, 1, 1, 1, 1, 130, 131), "conv_thin_mfma_kernel"),
    ((64, 256, 1, 1, 0, 1, 1, 20, 20), "pw_mfma_kernel"),
    ((32, 32, 3, 1, 1, 1, 32, 15, 18), "conv_dw_kernel"),
    ((16, 16, 3, 1, 1, 1, 16, 726, 727), "conv_dw_scan_kernel"),
    ((16, 16, 3, 1, 1, 1, 16, 300, 301), "conv_dw_scan_kernel"),
    ((64, 64, 3, 1, 1, 1, 64, 180, 181), "conv_dw_strip_kernel"),
    ((40, 40, 3, 1, 1, 1, 40, 180, 181), "conv_dw_strip_kernel"),
    ((144, 144, 3, 1, 1, 1, 144, 130, 131), "conv_dw_strip_kernel"),
    ((16, 16, 3, 2, 1, 1, 16, 600, 521), "conv_dw_scan_kernel"),
    ((3, 32, 3, 2, 1, 1, 1, 33, 31), "conv_stem_mfma_kernel"),
    ((3, 32, 3, 2, 1, 1, 1, 400, 380), "conv_stem_mfma_kernel"),
    ((3, 64, 3, 2, 1, 1, 1, 600, 520), "conv_fewcin_kernel"),     # many channel tiles on a large map
    ((3, 32, 3, 2, 1, 2, 1, 33, 31), "conv_fewcin_kernel"),       # dilation: no matrix-core form
    ((12, 64, 3, 1, 1, 1, 1, 40, 40), "conv_direct_kernel"),      # Cin not a multiple of 8: the generic kernel
], ids=lambda v: v if isinstance(v, str) else "-".join(str(x) for x in v))
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["float16", "bfloat16"])
def test_conv_dispatch(lib, cfg, kernel, dtype):
    """The shapes the parity cases above are chosen for reach the kernel they are meant to cover
    (the library names the kernels of the last call), in both 16-bit types."""
    from deltacnn_amd import _lib
    Cin, Cout, groups = cfg[0], cfg[1], cfg[6]
    x, mask, wt, bias, filt, (K, s, p, d, groups) = _conv_case(dtype, cfg, 5, 0.5)
    d_filt = filt.to(DEV)
    pk = hk().pack_filter(d_filt, Cin, Cout, groups)
    hk().sparse_conv(cl(x), d_filt, cl(mask), None, s, p, d, groups, c_out=Cout, create_out_mask=True, packed_filter=pk)
    assert _lib.load().dc_last_kernels().decode() == kernel


@pytest.mark.parametrize("cfg,kernel", [
    ((16, 8, 4, 2, 1, 1, 1, 9, 11), "conv_patch_mfma_kernel"),
    ((64, 48, 4, 2, 1, 1, 1, 37, 41), "conv_lds_mfma_kernel"),
    ((64, 64, 3, 2, 1, 2, 1, 40, 41), "conv_mfma_kernel"),
], ids=lambda v: v if isinstance(v, str) else "-".join(str(x) for x in v))
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["float16", "bfloat16"])
def test_deconv_dispatch(lib, cfg, kernel, dtype):
    from deltacnn_amd import _lib
    Cin, Cout = cfg[0], cfg[1]
    x, mask, wt, bias, filt, (K, s, p, d, groups) = _conv_case(dtype, cfg, 6, 0.5, True)
    d_filt = filt.to(DEV)
    pk = hk().pack_filter(d_filt, Cin, Cout, groups, transposed=True)
    hk().sparse_deconv(cl(x), d_filt, cl(mask), None, s, p, d, groups, c_out=Cout, create_out_mask=True, packed_filter=pk)
    assert _lib.load().dc_last_kernels().decode() == kernel


DECONVS = [
    (16, 8, 4, 2, 1, 1, 1, 9, 11),     # k4 s2 p1 (reference config)
    (8, 8, 6, 4, 1, 1, 1, 6, 7),       # k6 s4 p1 (reference config)
    (24, 16, 2, 2, 0, 1, 1, 7, 7),
    (8, 12, 3, 1, 1, 1, 1, 8, 9),
    (5, 3, 4, 2, 1, 1, 1, 6, 6),
    (64, 48, 4, 2, 1, 1, 1, 37, 41),   # large enough for the tiled MFMA kernel: stride-phase tiles
    (32, 32, 8, 4, 2, 1, 1, 20, 23),   # k8 s4: 64 taps, four per phase
    (40, 24, 3, 2, 1, 1, 1, 33, 30),   # kernel not a multiple of the stride: phases differ in tap count
    (64, 64, 3, 2, 1, 2, 1, 40, 41),   # dilation 2: compacted-tile kernel on stride-phase tiles
    (16, 16, 2, 3, 0, 1, 1, 30, 31),   # kernel smaller than the stride: phases without any tap
]


@pytest.mark.parametrize("dtype,cfg,packed", _conv_params(DECONVS, transposed=True))
@pytest.mark.parametrize("density", [0.1, 1.0])
def test_deconv(lib, dtype, cfg, density, packed):
    Cin, Cout = cfg[0], cfg[1]
    x, mask, wt, bias, filt, (K, s, p, d, groups) = _conv_case(dtype, cfg, 900 + Cin, density, True)
    want, want_mask = ops.deconv(x, mask, wt, bias, s, p, d, groups)
    d_filt = filt.to(DEV)
    pk = hk().pack_filter(d_filt, Cin, Cout, groups, transposed=True) if packed else None
    assert (pk is not None) == packed
    out, om = hk().sparse_deconv(cl(poison(x, mask)), d_filt, cl(mask), bias.to(DEV), s, p, d, groups,
                                 c_out=Cout, create_out_mask=True, packed_filter=pk)
    assert out.shape == want.shape
    assert torch.equal(om.cpu(), want_mask)
    _check_conv(dtype, out, want, want_mask)


FUSED = [
    (32, 64, 1, 1, 0, 1, 1, 12, 12),        # pointwise, few pixels (separate epilogue launch)
    (16, 96, 1, 1, 0, 1, 1, 40, 40),        # pointwise, epilogue in the kernel: 2 tiles/wave, 1 step
    (64, 192, 1, 1, 0, 1, 1, 40, 40),       # 3 tiles/wave, 2 steps
    (32, 384, 1, 1, 0, 1, 1, 40, 40),       # 6 tiles/wave, 1 step
    (64, 512, 1, 1, 0, 1, 1, 40, 40),       # a filter too large for the fused kernel: two launches
    (32, 512, 1, 1, 0, 1, 1, 40, 40),       # 2 tiles/wave on 16 wavefronts
    (24, 40, 1, 1, 0, 1, 1, 40, 40),        # partial channel tile and partial reduction step
    (64, 384, 1, 1, 0, 1, 1, 14, 14),       # small maps: two launches
    (96, 576, 1, 1, 0, 1, 1, 14, 14),
    (160, 960, 1, 1, 0, 1, 1, 7, 7),
    (128, 256, 1, 1, 0, 1, 1, 7, 7),
    (128, 64, 1, 1, 0, 1, 1, 40, 40),       # epilogue in the kernel: 4 reduction steps
    (320, 1280, 1, 1, 0, 1, 1, 7, 7),       # too long a reduction: two launches
    (32, 32, 3, 1, 1, 1, 32, 12, 12),       # depthwise 3x3, epilogue in the kernel
    (64, 64, 3, 2, 1, 1, 64, 13, 13),       # depthwise stride 2
    (24, 24, 5, 1, 2, 1, 24, 12, 12),       # depthwise 5x5 (generic tap loop)
    (32, 32, 3, 1, 1, 1, 1, 64, 64),        # small 3x3 layer: epilogue in the patch kernel, two tiles per wavefront
    (32, 24, 3, 1, 1, 1, 1, 64, 62),        # ... partial channel tile, ragged map
    (16, 16, 3, 1, 1, 1, 1, 24, 24),        # ... one tile per wavefront
    (32, 32, 3, 2, 1, 1, 1, 64, 64),        # two channel blocks: separate epilogue launch
    (3, 32, 3, 2, 1, 1, 1, 24, 24),         # RGB stem
    (3, 16, 7, 1, 3, 1, 1, 37, 45),         # 7x7 RGB stem
    (3, 64, 3, 2, 1, 1, 1, 40, 41),         # four channel tiles per wavefront
    (4, 24, 5, 1, 2, 1, 1, 19, 23),         # partial channel tile
    (96, 96, 3, 1, 1, 1, 96, 96, 96),       # large map: two vectors per lane
    (24, 24, 3, 1, 1, 1, 24, 192, 192),     # large map: three vectors per lane
    (16, 16, 3, 1, 1, 1, 16, 726, 727),     # very large map: mask scan and compaction per wavefront
    (24, 24, 3, 2, 1, 1, 24, 600, 521),     # the same with a stride
    (64, 64, 3, 1, 1, 1, 64, 180, 181),     # large map: strips of four pixels per lane group
    (144, 144, 3, 1, 1, 1, 144, 130, 131),  # ... wide rows, filter through LDS
    (16, 96, 1, 1, 0, 1, 1, 110, 111),      # pointwise on a large map: convolution and activation as two launches
    (16, 16, 3, 1, 1, 1, 1, 200, 190),      # thin layer on a large map: epilogue on pixel rows in the kernel
    (16, 32, 3, 2, 1, 1, 1, 520, 500),      # ... stride 2, only updated pixels staged
    (8, 24, 3, 1, 1, 1, 1, 130, 131),       # ... 8 input channels, a partial channel tile
    (16, 64, 3, 1, 1, 1, 1, 160, 170),      # ... four channel tiles: two passes over the row pieces
    (64, 64, 3, 1, 1, 1, 1, 70, 66),        # halo kernel, one workgroup holds all channels: it finishes the activation
    (128, 64, 3, 1, 1, 1, 1, 72, 61),       # ... four reduction slices
    (32, 64, 3, 2, 1, 1, 1, 176, 175),      # ... stride 2
    (64, 56, 3, 1, 1, 1, 1, 70, 66),        # ... a partial channel tile
    (32, 24, 5, 1, 2, 1, 1, 90, 77),        # ... 5x5
    (64, 64, 3, 1, 1, 1, 1, 136, 120),      # ... more workgroups than compute units: two launches
]
HALO_FINISHED = FUSED[-6:-1]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cfg", FUSED, ids=lambda c: "-".join(str(v) for v in c))
@pytest.mark.parametrize("act,mode", [(2, 0), (1, 0), (3, 1), (5, 0)])
def test_conv_activation_fused(lib, dtype, cfg, act, mode):
    """dc_conv_act == dc_conv followed by dc_activate_truncate, also against the oracle."""
    Cin, Cout, H, W = cfg[0], cfg[1], cfg[7], cfg[8]
    x, mask, wt, bias, filt, (K, s, p, d, groups) = _conv_case(dtype, cfg, 77, 0.4)
    g = _gen(78)
    x = (x.float() * (0.01 + rand_mask(g, 2, H, W, 0.5).float())).to(dtype)  # small and large updates
    want_conv, want_mask = ops.conv(x, mask, wt, None, s, p, d, groups)
    prev = torch.randn_like(want_conv.float(), ).to(dtype)
    trunc = (torch.randn_like(prev.float()) * 0.01).to(dtype)
    d_filt = filt.to(DEV)
    pk = hk().pack_filter(d_filt, Cin, Cout, groups)
    dx, dm = cl(poison(x, mask)), cl(mask)
    out1, om1 = hk().sparse_conv(dx, d_filt, dm, None, s, p, d, groups, c_out=Cout, create_out_mask=True,
                                 packed_filter=pk)
    assert torch.equal(om1.cpu(), want_mask)
    p1, t1 = cl(prev), cl(trunc)
    hk().sparse_activation(out1, p1, t1, om1, 0.3, act, mode)
    p2, t2 = cl(prev), cl(trunc)
    out2, om2 = hk().sparse_conv_activation(dx, d_filt, dm, None, p2, t2, 0.3, act, mode, s, p, d, groups, Cout,
                                            packed_filter=pk)
    if cfg in HALO_FINISHED and dtype != torch.float32 and act != 5:
        assert _last_kernel() == "conv_lds_mfma_kernel"   # one launch
    assert torch.equal(om1, om2)
    assert 0 < int(om1.sum()) and (mode != 0 or int(om1.sum()) < int(want_mask.sum()))
    assert torch.equal(p1, p2) and torch.equal(t1, t2)
    assert_masked_equal(out2, out1.cpu(), om1.cpu(), "out")


# ------------------------------------------- pointwise convolutions of large maps: active-pixel gather
GATHER_SHAPES = [(16, 96), (24, 144), (144, 24), (32, 16), (96, 24), (32, 192), (192, 32), (64, 128), (256, 40),
                 (8, 8)]


def _gather_case(dtype, cin, cout, density, seed):
    """Two 192 x 192 maps (73 728 pixels: the gather kernel's range), masks in runs as a video's."""
    g = _gen(seed)
    B, H, W = 2, 192, 192
    mask = (torch.nn.functional.interpolate((torch.rand(B, 1, H // 4, W // 8, generator=g) < density).float(),
                                            size=(H, W)) > 0).to(torch.int32)
    mask[0, 0, 5, 7] = 1                      # a lone pixel, and a map border
    mask[1, 0, H - 1, W - 3:] = 1
    x = torch.randn(B, cin, H, W, generator=g).to(dtype)
    wt = (torch.randn(cout, cin, 1, 1, generator=g) / cin ** 0.5).to(dtype)
    from deltacnn_amd.filter_conversion import convert_filter_out_channels_last, convert_half_filter
    filt = convert_half_filter(wt) if dtype == torch.float16 else convert_filter_out_channels_last(wt)
    return x, mask, wt, filt


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["float16", "bfloat16"])
@pytest.mark.parametrize("cin,cout", GATHER_SHAPES, ids=lambda v: str(v))
@pytest.mark.parametrize("density", [0.0, 0.02, 0.4, 1.0])
def test_pointwise_gather(lib, dtype, cin, cout, density):
    """1x1 convolutions of maps from 2^16 pixels on run on pw_gather_kernel: masks equal to the
    oracle's, values within the convolution tolerance, and bit-identical to the same pixels
    convolved as two smaller maps (which take pw_mfma_kernel): one summation order per layer."""
    x, mask, wt, filt = _gather_case(dtype, cin, cout, density, 1400 + cin + cout)
    want, want_mask = ops.conv(x, mask, wt, None, (1, 1), (0, 0), (1, 1), 1)
    d_filt = filt.to(DEV)
    pk = hk().pack_filter(d_filt, cin, cout, 1)
    dx, dm = cl(poison(x, mask)), cl(mask)
    out, om = hk().sparse_conv(dx, d_filt, dm, None, (1, 1), (0, 0), (1, 1), 1, c_out=cout, create_out_mask=True,
                               packed_filter=pk)
    assert _last_kernel() == "pw_gather_kernel"
    assert torch.equal(om.cpu(), want_mask)
    _check_conv(dtype, out, want, want_mask)
    for b in range(2):
        part, pm = hk().sparse_conv(cl(dx[b:b + 1]), d_filt, cl(dm[b:b + 1]), None, (1, 1), (0, 0), (1, 1), 1,
                                    c_out=cout, create_out_mask=True, packed_filter=pk)
        assert _last_kernel() == "pw_mfma_kernel"
        assert_masked_equal(out[b:b + 1], part.cpu(), want_mask[b:b + 1], f"map {b}: gather vs 64-pixel runs")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["float16", "bfloat16"])
@pytest.mark.parametrize("cin,cout", GATHER_SHAPES, ids=lambda v: str(v))
@pytest.mark.parametrize("act", [1, 2, 5])
@pytest.mark.parametrize("density", [0.02, 0.4, 1.0])
def test_pointwise_gather_with_activation(lib, dtype, cin, cout, act, density):
    """dc_conv_act on a large map (gather kernel with the activation / truncation as its
    epilogue) == dc_conv (gather kernel) followed by dc_activate_truncate: output, both cached
    tensors and the mask bit for bit; some pixels kept, some dropped."""
    x, mask, wt, filt = _gather_case(dtype, cin, cout, density, 1500 + cin + cout)
    g = _gen(1501 + cin)
    # half of the pixels carry a change far below the threshold: their updates are truncated
    x = (x.float() * torch.where(torch.rand(2, 1, 192, 192, generator=g) < 0.5, 1.0, 1e-3)).to(dtype)
    prev = torch.randn(2, cout, 192, 192, generator=g).to(dtype)
    trunc = (torch.randn(2, cout, 192, 192, generator=g) * 0.05).to(dtype)
    d_filt = filt.to(DEV)
    pk = hk().pack_filter(d_filt, cin, cout, 1)
    dx, dm = cl(poison(x, mask)), cl(mask)
    thr = 0.9 if act != 5 else 0.6
    p1, t1 = cl(prev), cl(trunc)
    out1, om1 = hk().sparse_conv(dx, d_filt, dm, None, (1, 1), (0, 0), (1, 1), 1, c_out=cout, create_out_mask=True,
                                 packed_filter=pk)
    hk().sparse_activation(out1, p1, t1, om1, thr, act, 0)
    p2, t2 = cl(prev), cl(trunc)
    out2, om2 = hk().sparse_conv_activation(dx, d_filt, dm, None, p2, t2, thr, act, 0, (1, 1), (0, 0), (1, 1), 1, cout,
                                            packed_filter=pk)
    assert _last_kernel() == "pw_gather_kernel"
    assert torch.equal(om1, om2)
    kept, reached = int(om1.sum()), int(mask.sum())
    assert 0 < kept < reached, (kept, reached)
    assert torch.equal(p1, p2) and torch.equal(t1, t2)
    assert_masked_equal(out2, out1.cpu(), om1.cpu(), "out")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["float16", "bfloat16"])
@pytest.mark.parametrize("cfg", [(64, 384, 56, 56), (96, 576, 56, 56), (32, 192, 112, 112), (64, 1024, 48, 48),
                                 (24, 40, 170, 170), (96, 264, 64, 64)], ids=lambda c: "-".join(str(v) for v in c))
@pytest.mark.parametrize("act", [1, 2, 4])
@pytest.mark.parametrize("density", [0.03, 0.6, 1.0])
def test_pointwise_rows_epilogue(lib, dtype, cfg, act, density):
    """dc_conv_act on layers whose output map exceeds 4 MB (as with many streams in a batch) and
    whose filter stays below 128 KB: one launch (pw_rows_act_kernel), bit-identical -- output,
    both cached tensors, mask -- to dc_conv followed by dc_activate_truncate, and the convolution
    within tolerance of the oracle's."""
    cin, cout, H, W = cfg
    g = _gen(1600 + cin + cout)
    B = 2
    mask = rand_mask(g, B, H, W, density)
    x = torch.randn(B, cin, H, W, generator=g)
    x = (x * torch.where(torch.rand(B, 1, H, W, generator=g) < 0.5, 1.0, 1e-3)).to(dtype)  # half of the updates get truncated
    wt = (torch.randn(cout, cin, 1, 1, generator=g) / cin ** 0.5).to(dtype)
    prev = torch.randn(B, cout, H, W, generator=g).to(dtype)
    trunc = (torch.randn(B, cout, H, W, generator=g) * 0.05).to(dtype)
    from deltacnn_amd.filter_conversion import convert_filter_out_channels_last, convert_half_filter
    d_filt = (convert_half_filter(wt) if dtype == torch.float16 else convert_filter_out_channels_last(wt)).to(DEV)
    pk = hk().pack_filter(d_filt, cin, cout, 1)
    dx, dm = cl(poison(x, mask)), cl(mask)
    thr = 0.9 if act != 4 else 0.2
    p1, t1 = cl(prev), cl(trunc)
    out1, om1 = hk().sparse_conv(dx, d_filt, dm, None, (1, 1), (0, 0), (1, 1), 1, c_out=cout, create_out_mask=True,
                                 packed_filter=pk)
    assert _last_kernel() == "pw_mfma_kernel"
    want, want_mask = ops.conv(x, mask, wt, None, (1, 1), (0, 0), (1, 1), 1)
    _check_conv(dtype, out1, want, want_mask)
    hk().sparse_activation(out1, p1, t1, om1, thr, act, 0)
    p2, t2 = cl(prev), cl(trunc)
    out2, om2 = hk().sparse_conv_activation(dx, d_filt, dm, None, p2, t2, thr, act, 0, (1, 1), (0, 0), (1, 1), 1, cout,
                                            packed_filter=pk)
    assert _last_kernel() == "pw_rows_act_kernel"
    assert torch.equal(om1, om2)
    assert 0 < int(om1.sum()) < int(mask.sum())
    assert torch.equal(p1, p2) and torch.equal(t1, t2)
    assert_masked_equal(out2, out1.cpu(), om1.cpu(), "out")


@pytest.mark.parametrize("cfg", [(96, 24, 56, 56), (144, 32, 28, 28), (384, 64, 14, 14), (960, 160, 7, 7),
                                 (32, 20, 9, 9)], ids=lambda c: "-".join(str(v) for v in c))
@pytest.mark.parametrize("weights", [(1.0, 1.0), (0.5, -1.5)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_conv_add_fused(lib, cfg, weights, dtype):
    """dc_conv_add == DCAdd(residual, conv(x)) of the oracle, and bit-identical to the two
    separate library calls."""
    from deltacnn_amd.hip_kernels import conv_geometry
    Cin, Cout, H, W = cfg
    x, mask, wt, bias, filt, (K, s, p, d, groups) = _conv_case(dtype, (Cin, Cout, 1, 1, 0, 1, 1, H, W), 91, 0.3)
    g = _gen(92)
    mres = rand_mask(g, 2, H, W, 0.3)
    res = torch.randn(2, Cout, H, W, generator=g).to(dtype)
    want_conv, want_cm = ops.conv(x, mask, wt, None, s, p, d, groups)
    want, want_mask = ops.add(res, mres, want_conv, want_cm, None, weights[0], weights[1], 0, False)
    d_filt = filt.to(DEV)
    pk = hk().pack_filter(d_filt, Cin, Cout, 1)
    dx, dm, dres, dmres = cl(poison(x, mask)), cl(mask), cl(poison(res, mres)), cl(mres)
    geo = conv_geometry(x.shape, K, Cout, s, p, d, 1)
    out = torch.full((2, Cout, H, W), float("nan"), dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
    om = torch.full((2, 1, H, W), -5, dtype=torch.int32, device=DEV)
    got = hk().sparse_conv_add(dx, pk, dm, None, dres, dmres, geo, out, om, weights[0], weights[1])
    assert got is not None
    assert torch.equal(om.cpu(), want_mask)
    _check_conv(dtype, out, want, want_mask)
    c_out, c_mask = hk().sparse_conv(dx, d_filt, dm, None, s, p, d, 1, c_out=Cout, create_out_mask=True, packed_filter=pk)
    two = torch.empty_like(out)
    two_mask = torch.empty_like(om)
    hk().sparse_add_tensors(dres, c_out, None, two, dmres, c_mask, two_mask, weights[0], weights[1], 0, False)
    assert torch.equal(two_mask, om)
    assert_masked_equal(out, two.cpu(), want_mask, "fused vs two calls")


@pytest.mark.parametrize("cfg", [(32, 32, 3, 1, 1, 1, 1, 16, 16), (64, 64, 3, 1, 1, 1, 1, 12, 13),
                                 (128, 128, 3, 1, 1, 1, 1, 8, 8), (24, 20, 3, 2, 1, 1, 1, 17, 19),
                                 (16, 18, 5, 1, 2, 1, 1, 9, 9), (48, 32, 1, 1, 0, 1, 1, 10, 10),
                                 # pointwise arrangements: 64x64 tiles, reduction split over 4 and 8 wavefronts
                                 (64, 256, 1, 1, 0, 1, 1, 64, 64), (576, 96, 1, 1, 0, 1, 1, 14, 14),
                                 (960, 160, 1, 1, 0, 1, 1, 7, 7),
                                 # larger K x K layers: the LDS-halo kernel, one case per arrangement / corner
                                 (64, 64, 3, 1, 1, 1, 1, 72, 70), (64, 32, 3, 1, 1, 1, 1, 100, 100),
                                 (16, 64, 3, 1, 1, 1, 1, 120, 120), (32, 256, 3, 1, 1, 1, 1, 90, 90),
                                 (128, 128, 3, 1, 1, 1, 1, 40, 40), (64, 80, 3, 2, 1, 1, 1, 120, 121),
                                 (32, 42, 3, 1, 1, 1, 1, 80, 80), (320, 32, 3, 1, 1, 1, 1, 40, 40)],
                         ids=lambda c: "-".join(str(v) for v in c))
@pytest.mark.parametrize("act", [0, 1, 3])
@pytest.mark.parametrize("weights", [(1.0, 1.0), (0.5, -1.5)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["float16", "bfloat16"])
def test_conv_add_fused_small_layers(lib, cfg, act, weights, dtype):
    """dc_conv_add on KxK layers (4x4-patch and LDS-halo kernels) and on the pointwise
    arrangements, with the DCAdd's activation and accumulated sum: equal to
    the oracle's conv + add, bit-identical to dc_conv followed by dc_add (outputs and state)."""
    from deltacnn_amd.hip_kernels import conv_geometry
    Cin, Cout = cfg[0], cfg[1]
    tol = 2e-2 if dtype == torch.float16 else 8e-2  # one bfloat16 step at |x| <= 8 is 3e-2
    x, mask, wt, bias, filt, (K, s, p, d, groups) = _conv_case(dtype, cfg, 93, 0.05)
    want_conv, want_cm = ops.conv(x, mask, wt, None, s, p, d, groups)
    B, _, Ho, Wo = want_conv.shape
    g = _gen(94)
    mres = rand_mask(g, B, Ho, Wo, 0.3)
    res = torch.randn(B, Cout, Ho, Wo, generator=g).to(dtype)
    prev = torch.randn(B, Cout, Ho, Wo, generator=g).to(dtype)
    want_prev = prev.clone()
    want, want_mask = ops.add(res, mres, want_conv, want_cm, want_prev if act else None, weights[0], weights[1], act, False)
    assert 0 < int((want_cm & (1 - mres)).sum()) and 0 < int(((1 - want_cm) & mres).sum())  # both one-sided cases
    d_filt = filt.to(DEV)
    pk = hk().pack_filter(d_filt, Cin, Cout, 1)
    dx, dm, dres, dmres = cl(poison(x, mask)), cl(mask), cl(poison(res, mres)), cl(mres)
    geo = conv_geometry(x.shape, K, Cout, s, p, d, 1)
    out = torch.full((B, Cout, Ho, Wo), float("nan"), dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
    om = torch.full((B, 1, Ho, Wo), -5, dtype=torch.int32, device=DEV)
    p1 = cl(prev)
    got = hk().sparse_conv_add(dx, pk, dm, None, dres, dmres, geo, out, om, weights[0], weights[1],
                               p1 if act else None, act)
    # small layers run on the 4x4-patch kernel (any activation): patches x channel tiles x steps <= 32768
    patch_work = B * -(-Ho // 4) * -(-Wo // 4) * -(-Cout // 16) * K[0] * K[1] * -(-Cin // 32)
    if K != (1, 1) and patch_work > 32768 and act != 0:
        assert got is None  # the LDS-halo kernel carries the sum of a DCAdd without activation only
        return
    assert got is not None
    assert torch.equal(om.cpu(), want_mask)
    assert_masked_close(out, want, want_mask, 0, tol, "out")
    c_out, c_mask = hk().sparse_conv(dx, d_filt, dm, None, s, p, d, 1, c_out=Cout, create_out_mask=True, packed_filter=pk)
    two, two_mask, p2 = torch.empty_like(out), torch.empty_like(om), cl(prev)
    hk().sparse_add_tensors(dres, c_out, p2 if act else None, two, dmres, c_mask, two_mask, weights[0], weights[1], act, False)
    assert torch.equal(two_mask, om)
    assert_masked_equal(out, two.cpu(), want_mask, "fused vs two calls")
    assert torch.equal(p1, p2)
    if act:
        assert_masked_close(p1, want_prev, torch.ones_like(want_mask), 0, tol, "prev_out")


@pytest.mark.parametrize("cfg", [(64, 48, 4, 2, 1, 1, 1, 37, 41), (64, 64, 4, 2, 1, 1, 1, 34, 60),
                                 (128, 128, 4, 2, 1, 1, 1, 17, 30), (32, 32, 8, 4, 2, 1, 1, 20, 23),
                                 (40, 24, 3, 2, 1, 1, 1, 66, 60)], ids=lambda c: "-".join(str(v) for v in c))
@pytest.mark.parametrize("density", [0.05, 0.6])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["float16", "bfloat16"])
def test_deconv_add_fused(lib, cfg, density, dtype):
    """dc_deconv_add == DCAdd(deconv(x), residual) of the oracle, and bit-identical to dc_deconv
    followed by dc_add with the transposed convolution as FIRST operand (unit weights: the sum is
    commutative), on pixels reached by one operand only and by both."""
    from deltacnn_amd import _lib
    from deltacnn_amd.hip_kernels import conv_geometry
    Cin, Cout = cfg[0], cfg[1]
    tol = 2e-2 if dtype == torch.float16 else 8e-2
    x, mask, wt, bias, filt, (K, s, p, d, groups) = _conv_case(dtype, cfg, 95, density, True)
    want_conv, want_cm = ops.deconv(x, mask, wt, None, s, p, d, groups)
    B, _, Ho, Wo = want_conv.shape
    g = _gen(96)
    mres = rand_mask(g, B, Ho, Wo, 0.3)
    res = torch.randn(B, Cout, Ho, Wo, generator=g).to(dtype)
    want, want_mask = ops.add(want_conv, want_cm, res, mres, None, 1.0, 1.0, 0, False)
    if density < 0.5:
        assert 0 < int((want_cm & (1 - mres)).sum()) and 0 < int(((1 - want_cm) & mres).sum())
    d_filt = filt.to(DEV)
    pk = hk().pack_filter(d_filt, Cin, Cout, 1, transposed=True)
    dx, dm, dres, dmres = cl(poison(x, mask)), cl(mask), cl(poison(res, mres)), cl(mres)
    geo = conv_geometry(x.shape, K, Cout, s, p, d, 1, transposed=True)
    out = torch.full((B, Cout, Ho, Wo), float("nan"), dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
    om = torch.full((B, 1, Ho, Wo), -5, dtype=torch.int32, device=DEV)
    got = hk().sparse_deconv_add(dx, pk, dm, dres, dmres, geo, out, om)
    assert got is not None and _lib.load().dc_last_kernels().decode() == "conv_lds_mfma_kernel"
    assert torch.equal(om.cpu(), want_mask)
    assert_masked_close(out, want, want_mask, 0, tol, "out")
    c_out, c_mask = hk().sparse_deconv(dx, d_filt, dm, None, s, p, d, 1, c_out=Cout, create_out_mask=True, packed_filter=pk)
    two, two_mask = torch.empty_like(out), torch.empty_like(om)
    hk().sparse_add_tensors(c_out, dres, None, two, c_mask, dmres, two_mask, 1.0, 1.0, 0, False)
    assert torch.equal(two_mask, om)
    assert_masked_equal(out, two.cpu(), want_mask, "fused vs two calls")


def test_deconv_add_declines_what_it_cannot_do(lib):
    """Small transposed layers (the 4x4-patch kernel's), windows smaller than the stride and fp32:
    None, nothing launched."""
    from deltacnn_amd.hip_kernels import conv_geometry
    for cfg, dtype in (((16, 8, 4, 2, 1, 1, 1, 9, 11), torch.float16), ((16, 16, 2, 3, 0, 1, 1, 30, 31), torch.float16),
                       ((64, 48, 4, 2, 1, 1, 1, 37, 41), torch.float32)):
        Cin, Cout = cfg[0], cfg[1]
        x, mask, wt, bias, filt, (K, s, p, d, groups) = _conv_case(torch.float16, cfg, 97, 0.5, True)
        want_conv, _ = ops.deconv(x, mask, wt, None, s, p, d, groups)
        B, _, Ho, Wo = want_conv.shape
        pk = hk().pack_filter(filt.to(DEV), Cin, Cout, 1, transposed=True)
        geo = conv_geometry(x.shape, K, Cout, s, p, d, 1, transposed=True)
        out = torch.zeros((B, Cout, Ho, Wo), dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
        om = torch.zeros((B, 1, Ho, Wo), dtype=torch.int32, device=DEV)
        res = torch.ones_like(out)
        assert hk().sparse_deconv_add(cl(x).to(dtype), pk, cl(mask), res, torch.ones_like(om), geo, out, om) is None
        assert not bool(out.any()) and not bool(om.any())


@pytest.mark.parametrize("cfg", [((64, 64), 64, 37, 41, 2), ((64, 64), 64, 136, 240, 1), ((128, 128, 64, 128), 128, 20, 23, 1),
                                 ((256, 256), 256, 17, 30, 1), ((512, 256, 128), 256, 9, 11, 1),
                                 ((512, 512, 256), 512, 6, 7, 1), ((32, 96), 40, 50, 50, 1), ((64, 32, 32, 64), 256, 64, 64, 1)],
                         ids=lambda c: "-".join(str(v).replace(" ", "") for v in c))
@pytest.mark.parametrize("density", [0.1, 0.7])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["float16", "bfloat16"])
def test_concat_conv_fused(lib, cfg, density, dtype):
    """dc_concat_conv == the oracle's chained concatenation + 1x1 convolution, and bit-identical
    to dc_concat (chained) followed by dc_conv, with every tensor active on its own pixels."""
    from deltacnn_amd import _lib
    from deltacnn_amd.filter_conversion import convert_filter_out_channels_last, convert_half_filter
    from deltacnn_amd.hip_kernels import conv_geometry
    chans, Cout, H, W, B = cfg
    g = _gen(1300 + sum(chans) + Cout)
    xs = [torch.randn(B, c, H, W, generator=g).to(dtype) for c in chans]
    ms = [rand_mask(g, B, H, W, density * (0.5 + 0.5 * i / len(chans))) for i in range(len(chans))]
    wt = (torch.randn(Cout, sum(chans), 1, 1, generator=g) / sum(chans) ** 0.5).to(dtype)
    cat, cm = xs[0], ms[0]
    for x, m in zip(xs[1:], ms[1:]):
        cat, cm = ops.concatenate(cat, cm, x, m)
    want, want_mask = ops.conv(cat, cm, wt, None, (1, 1), (0, 0), (1, 1), 1)
    filt = (convert_half_filter(wt) if dtype == torch.float16 else convert_filter_out_channels_last(wt)).to(DEV)
    pk = hk().pack_filter(filt, sum(chans), Cout, 1)
    dxs = [(cl(poison(x, m)), cl(m)) for x, m in zip(xs, ms)]
    geo = conv_geometry((B, sum(chans), H, W), (1, 1), Cout, (1, 1), (0, 0), (1, 1), 1)
    out = torch.full((B, Cout, H, W), float("nan"), dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
    om = torch.full((B, 1, H, W), -5, dtype=torch.int32, device=DEV)
    got = hk().sparse_concat_conv(dxs, pk, geo, out, om)
    assert got is not None and _lib.load().dc_last_kernels().decode() == "pw_mfma_kernel"
    assert torch.equal(om.cpu(), want_mask)
    _check_conv(dtype, out, want, want_mask)
    dcat = dxs[0]
    for d in dxs[1:]:
        dcat = hk().sparse_concatenate(dcat, d)
    two, two_mask = hk().sparse_conv(dcat[0], filt, dcat[1], None, (1, 1), (0, 0), (1, 1), 1, c_out=Cout, create_out_mask=True,
                                     packed_filter=pk)
    assert _lib.load().dc_last_kernels().decode() in ("pw_mfma_kernel", "pw_gather_kernel")
    assert torch.equal(two_mask, om)
    assert_masked_equal(out, two.cpu(), want_mask, "fused vs separate calls")


# ------------------------------------------------------------------ nothing active / all active
@pytest.mark.parametrize("fill", [0, 1], ids=["all-inactive", "all-active"])
@pytest.mark.parametrize("cfg", [
    (32, 32, 3, 1, 1, 1, 1, 16, 16),        # patch kernel
    (64, 64, 3, 1, 1, 1, 1, 72, 70),        # LDS-halo kernel
    (64, 256, 1, 1, 0, 1, 1, 20, 20),       # pointwise
    (32, 32, 3, 1, 1, 1, 32, 15, 18),       # depthwise
    (16, 16, 3, 1, 1, 1, 16, 726, 727),     # depthwise, mask scan
    (64, 64, 3, 1, 1, 1, 64, 180, 181),     # depthwise strips
    (3, 32, 3, 2, 1, 1, 1, 33, 31),         # stem
], ids=lambda c: "-".join(str(v) for v in c))
def test_conv_uniform_masks(lib, cfg, fill):
    """A map without a single active pixel writes an all-zero output mask and touches no output
    value (the output buffer keeps its NaN fill); a fully active map is the dense convolution."""
    Cin, Cout = cfg[0], cfg[1]
    dtype = torch.float16
    x, mask, wt, bias, filt, (K, s, p, d, groups) = _conv_case(dtype, cfg, 31, 0.5)
    mask = torch.full_like(mask, fill)
    want, want_mask = ops.conv(x, mask, wt, None, s, p, d, groups)
    d_filt = filt.to(DEV)
    pk = hk().pack_filter(d_filt, Cin, Cout, groups)
    out = torch.full(tuple(want.shape), float("nan"), dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
    om = torch.full(tuple(want_mask.shape), -7, dtype=torch.int32, device=DEV)
    hk().sparse_conv(cl(poison(x, mask)), d_filt, cl(mask), None, s, p, d, groups, c_out=Cout,
                     create_out_mask=True, packed_filter=pk, out=out, out_mask=om)
    assert torch.equal(om.cpu(), want_mask)
    if fill == 0:
        assert int(om.abs().sum()) == 0 and bool(out.isnan().all())
    else:
        _check_conv(dtype, out, want, want_mask)


@pytest.mark.parametrize("fill", [0, 1], ids=["all-inactive", "all-active"])
def test_scanned_kernels_uniform_masks(lib, fill):
    """The mask-scanning activation and add kernels on a map with no / only active pixels."""
    g = _gen(77)
    B, C, H, W = 1, 16, 520, 511
    dtype = torch.float16
    mask = torch.full((B, 1, H, W), fill, dtype=torch.int32)
    prev = torch.randn(B, C, H, W, generator=g).to(dtype)
    trunc = (torch.randn(B, C, H, W, generator=g) * 0.01).to(dtype)
    delta = torch.randn(B, C, H, W, generator=g).to(dtype)
    w = [delta.clone(), prev.clone(), trunc.clone(), mask.clone()]
    ops.activate_truncate(*w, 0.1, 1, 0)
    d = [cl(poison(delta, mask)), cl(prev), cl(trunc), cl(mask)]
    hk().sparse_activation(*d, 0.1, 1, 0)
    assert torch.equal(d[3].cpu(), w[3])
    assert_masked_equal(d[0], w[0], w[3], "delta")
    assert torch.equal(d[1].cpu(), w[1]) and torch.equal(d[2].cpu(), w[2])
    b = torch.randn(B, C, H, W, generator=g).to(dtype)
    w_out, w_mask = ops.add(delta, mask, b, mask, None, 1.0, 1.0, 0, False)
    d_out = torch.full((B, C, H, W), float("nan"), dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
    d_mo = torch.full((B, 1, H, W), -3, dtype=torch.int32, device=DEV)
    hk().sparse_add_tensors(cl(poison(delta, mask)), cl(poison(b, mask)), None, d_out, cl(mask), cl(mask), d_mo,
                            1.0, 1.0, 0, False)
    assert torch.equal(d_mo.cpu(), w_mask)
    assert_masked_equal(d_out, w_out, w_mask, "out")
    if fill == 0:
        assert bool(d_out.isnan().all())


# --------------------------------------------------------------------------------- pooling
POOLS = [
    # C, K, stride, padding, dilation, H, W
    (16, 2, 2, 0, 1, 12, 14),
    (32, 3, 2, 1, 1, 13, 13),
    (5, 3, 1, 1, 1, 9, 8),
    (8, 2, 2, (0, 1, 0, 1), 1, 9, 9),     # asymmetric: zero joins the maximum
    (24, 3, 1, 2, 2, 10, 10),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cfg", POOLS, ids=lambda c: "-".join(str(v).replace(" ", "") for v in c))
@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("density", [0.1, 0.6])
def test_pool(lib, dtype, cfg, mode, density):
    C, K, s, p, d, H, W = cfg
    K, s, d, p = _pair(K), _pair(s), _pair(d), _pair(p)
    g = _gen(1000 + C)
    B = 2
    mask = rand_mask(g, B, H, W, density)
    x = torch.randn(B, C, H, W, generator=g).to(dtype)
    prev = torch.randn(B, C, H, W, generator=g).to(dtype)
    want, want_mask = ops.pool(x, prev if mode == 0 else None, mask, K, s, p, d, mode)
    out, om = hk().sparse_pooling(cl(poison(x, mask)), cl(prev) if mode == 0 else None, K, cl(mask), s, p, d,
                                  pooling_mode_int=mode)
    assert torch.equal(om.cpu(), want_mask)
    assert_masked_equal(out, want, want_mask, "out")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cfg", [(32, 2, 12, 14, 2), (64, 2, 34, 60, 1), (128, 2, 68, 120, 1), (24, 3, 12, 15, 2),
                                 (512, 2, 6, 8, 1), (1024, 2, 4, 4, 1)], ids=lambda c: "-".join(str(v) for v in c))
@pytest.mark.parametrize("density", [0.0, 0.1, 0.7])
def test_pool_update_fused(lib, dtype, cfg, density):
    """dc_pool_update == the oracle's maximum pooling followed by its cache update, and
    bit-identical (pooled delta, mask and the cached input) to dc_pool + dc_add_to_dense."""
    from deltacnn_amd import _lib
    C, K, H, W, B = cfg
    g = _gen(1100 + C)
    mask = rand_mask(g, B, H, W, density)
    x = torch.randn(B, C, H, W, generator=g).to(dtype)
    prev = torch.randn(B, C, H, W, generator=g).to(dtype)
    want, want_mask = ops.pool(x, prev, mask, (K, K), (K, K), (0, 0), (1, 1), 0)
    want_prev = prev.clone()
    ops.add_to_dense(torch.where(mask != 0, x, torch.zeros_like(x)), want_prev, mask)
    dx, dm = cl(poison(x, mask)), cl(mask)
    p1 = cl(prev)
    got = hk().sparse_max_pooling_update(dx, p1, (K, K), dm, (K, K))
    if C * x.element_size() > 64 * 16:  # more than 64 vectors of 16 bytes per pixel: the two calls
        assert got is None
        return
    assert got is not None and _lib.load().dc_last_kernels().decode() == "pool_pixel_kernel"
    out, om = got
    assert torch.equal(om.cpu(), want_mask)
    assert_masked_equal(out, want, want_mask, "out")
    assert torch.equal(p1.cpu(), want_prev), "cached input"
    p2 = cl(prev)
    out2, om2 = hk().sparse_pooling(dx, p2, (K, K), dm, (K, K), (0, 0), (1, 1), pooling_mode_int=0)
    hk().sparse_add_to_dense_tensor(dx, p2, dm)
    assert torch.equal(om2, om) and torch.equal(p1, p2)
    assert_masked_equal(out, out2.cpu(), want_mask, "fused vs two calls")


def test_pool_update_declines_other_shapes(lib):
    """Windows that overlap, leave pixels over or are padded, channel counts off the vector size:
    None, nothing launched, nothing touched."""
    for C, K, s, H, W in ((32, 3, 2, 13, 13), (32, 2, 2, 13, 14), (20, 2, 2, 12, 12), (32, 2, 1, 12, 12)):
        x = torch.randn(1, C, H, W).half().to(DEV).contiguous(memory_format=torch.channels_last)
        prev = torch.zeros_like(x)
        mask = torch.ones(1, 1, H, W, dtype=torch.int32, device=DEV)
        assert hk().sparse_max_pooling_update(x, prev, (K, K), mask, (s, s)) is None
        assert not bool(prev.any())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("C,H,W", [(1280, 7, 7), (17, 5, 9), (64, 16, 16)])
@pytest.mark.parametrize("density", [0.0, 0.2, 1.0])
def test_pool_global(lib, dtype, mode, C, H, W, density):
    g = _gen(1100 + C)
    B = 2
    mask = rand_mask(g, B, H, W, density)
    x = torch.randn(B, C, H, W, generator=g).to(dtype)
    prev = torch.randn(B, C, H, W, generator=g).to(dtype)
    want, want_mask = ops.pool(x, prev if mode == 0 else None, mask, (H, W), (1, 1), (0, 0), (1, 1), mode)
    out, om = hk().sparse_pooling(cl(poison(x, mask)), cl(prev) if mode == 0 else None, (H, W), cl(mask),
                                  pooling_mode_int=mode)
    assert out.dtype == dtype and out.shape == (B, C, 1, 1)
    assert torch.equal(om.cpu(), want_mask)
    # the average is a float sum over up to H*W values in a different order than the oracle's
    tol = LOOSE[dtype]
    assert_masked_close(out, want, want_mask, tol, tol, "out")
    # the reference's protocol: float32 accumulator handed in by the caller, cast afterwards
    acc = torch.full((B, C, 1, 1), float("nan"), dtype=torch.float32, device=DEV).contiguous(
        memory_format=torch.channels_last)
    out2, om2 = hk().sparse_pooling(cl(poison(x, mask)), cl(prev) if mode == 0 else None, (H, W), cl(mask),
                                    pooling_mode_int=mode, out=acc)
    assert out2.dtype == dtype and torch.equal(om2.cpu(), want_mask)
    assert_masked_close(out2, want, want_mask, tol, tol, "out (float32 accumulator)")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,H,W", [(1280, 7, 7), (64, 16, 16), (24, 3, 5), (2048, 1, 1)])
@pytest.mark.parametrize("density", [0.0, 0.2, 1.0])
def test_pool_densify_fused(lib, dtype, C, H, W, density):
    """dc_pool_densify == global average pooling followed by densify: bit-identical to the two
    library calls (dense result and accumulator), within the pooling tolerance of the oracle's;
    one stream of the batch without any update keeps its accumulator bit for bit."""
    g = _gen(1150 + C)
    B = 3
    mask = rand_mask(g, B, H, W, density)
    mask[2] = 0  # a stream whose frame did not change
    x = torch.randn(B, C, H, W, generator=g).to(dtype)
    acc0 = torch.randn(B, C, 1, 1, generator=g).to(dtype)
    dx, dm = cl(poison(x, mask)), cl(mask)
    acc, dense = cl(acc0), torch.full((B, C, 1, 1), float("nan"), dtype=dtype, device=DEV).contiguous(
        memory_format=torch.channels_last)
    assert hk().pooled_densify(dx, dm, acc, dense)
    assert _last_kernel() == "pool_global_vec_kernel"
    pooled, pm = hk().sparse_pooling(dx, None, (H, W), dm, pooling_mode_int=1)
    acc2, dense2 = cl(acc0), torch.empty_like(dense)
    hk().densify(pooled, acc2, dense2, pm)
    assert torch.equal(acc, acc2) and torch.equal(dense, dense2) and torch.equal(dense, acc)
    assert torch.equal(acc[2].cpu(), acc0[2])
    want, want_mask = ops.pool(x, None, mask, (H, W), (1, 1), (0, 0), (1, 1), 1)
    w_acc = acc0.clone()
    ops.activate_truncate(want.clone(), w_acc, None, want_mask, -1, -1, -1)
    tol = LOOSE[dtype]
    assert float((dense.cpu().float() - w_acc.float()).abs().max()) <= tol * max(1.0, float(w_acc.float().abs().max()))


def test_pool_densify_declines_other_shapes(lib):
    """Channel counts that do not fill 16-byte vectors have no one-launch form: False, nothing
    launched, operands untouched."""
    g = _gen(1199)
    mask = rand_mask(g, 1, 4, 4, 0.5)
    x = torch.randn(1, 20, 4, 4, generator=g).half()
    acc = cl(torch.randn(1, 20, 1, 1, generator=g).half())
    before, dense = acc.clone(), torch.zeros_like(acc)
    assert not hk().pooled_densify(cl(x), cl(mask), acc, dense)
    assert torch.equal(acc, before) and not bool(dense.any())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 3, 8, 9, 32])
@pytest.mark.parametrize("fi,fo", [(1280, 1000), (64, 10), (520, 7), (4104, 33)])
@pytest.mark.parametrize("use_bias", [True, False])
def test_linear(lib, dtype, rows, fi, fo, use_bias):
    """dc_linear against torch's linear evaluated in fp64 on the same (rounded) operands: fp32
    accumulation and one rounding, so the error is half a unit of the output type plus the
    accumulation error of fi fp32 products."""
    g = _gen(1300 + fi + rows)
    x = torch.randn(rows, fi, generator=g).to(dtype)
    w = (torch.randn(fo, fi, generator=g) / fi ** 0.5).to(dtype)
    b = torch.randn(fo, generator=g).to(dtype) if use_bias else None
    want = torch.nn.functional.linear(x.double(), w.double(), None if b is None else b.double())
    got = hk().linear(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV))
    assert _last_kernel() == "linear_kernel"
    assert got.dtype == dtype and got.shape == (rows, fo)
    step = {torch.float32: 2.0 ** -23, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    err = (got.cpu().double() - want).abs()
    bound = step * want.abs().clamp(min=1.0) + 1e-5
    assert bool((err <= bound).all()), float((err / bound).max())


# ------------------------------------------------ the scanning forms of the simple operators
def _last_kernel():
    from deltacnn_amd import _lib
    return _lib.load().dc_last_kernels().decode()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("density", [0.0, 0.03, 0.5, 1.0])
def test_scanned_simple_operators(lib, dtype, density):
    """mul_add, add_to_dense, concat and upsample on maps large enough for their mask-scanning
    kernels (channel counts that fill, underfill and split a lane group)."""
    g = _gen(int(1500 + 100 * density))
    B, H, W = 2, 397, 333
    for C in (24, 64) if dtype != torch.float32 else (12, 40):
        mask = rand_mask(g, B, H, W, density)
        x = torch.randn(B, C, H, W, generator=g).to(dtype)
        scale, bias = torch.randn(C, generator=g).to(dtype), torch.randn(C, generator=g).to(dtype)
        for bi in (None, bias):
            want, want_mask = ops.mul_add(x, mask, scale, bi)
            d_x, d_m = cl(poison(x, mask)), cl(mask)
            out, om = torch.full_like(d_x, float("nan")), torch.full_like(d_m, -3)
            hk().sparse_mul_add(d_x, d_m, out, om, scale.to(DEV), None if bi is None else bi.to(DEV))
            assert _last_kernel() == "mul_add_scan_kernel"
            assert torch.equal(om.cpu(), want_mask)
            if dtype == torch.float32 and bi is not None:
                assert_masked_close(out, want, want_mask, 1e-6, 1e-6, "mul_add")
            else:
                assert_masked_equal(out, want, want_mask, "mul_add")
            if density == 0.0:
                assert bool(out.isnan().all())
            # in place, as the batch-norm layer calls it
            hk().sparse_mul_add(d_x, d_m, d_x, d_m, scale.to(DEV), None if bi is None else bi.to(DEV))
            if not (dtype == torch.float32 and bi is not None):
                assert_masked_equal(d_x, want, want_mask, "mul_add in place")
            assert torch.equal(d_m.cpu(), mask)

        b = torch.randn(B, C, H, W, generator=g).to(dtype)
        w_b = b.clone()
        ops.add_to_dense(x, w_b, mask)
        d_b = cl(b)
        hk().sparse_add_to_dense_tensor(cl(poison(x, mask)), d_b, cl(mask), 0)
        assert _last_kernel() == "add_to_dense_scan_kernel"
        assert torch.equal(d_b.cpu(), w_b)

        Cb = C - (4 if dtype == torch.float32 else 8)
        mb = rand_mask(g, B, H, W, density / 2)
        y = torch.randn(B, Cb, H, W, generator=g).to(dtype)
        want, want_mask = ops.concatenate(x, mask, y, mb)
        d_out = torch.full((B, C + Cb, H, W), float("nan"), dtype=dtype, device=DEV).contiguous(
            memory_format=torch.channels_last)
        d_om = torch.full((B, 1, H, W), -3, dtype=torch.int32, device=DEV)
        hk().sparse_concatenate((cl(poison(x, mask)), cl(mask)), (cl(poison(y, mb)), cl(mb)), out=(d_out, d_om))
        assert _last_kernel() == "concat_scan_kernel"
        assert torch.equal(d_om.cpu(), want_mask)
        assert_masked_equal(d_out, want, want_mask, "concat")

        for s in (2, 3):
            want, want_mask = ops.upsample(x, mask, s)
            d_out = torch.full((B, C, H * s, W * s), float("nan"), dtype=dtype, device=DEV).contiguous(
                memory_format=torch.channels_last)
            d_om = torch.full((B, 1, H * s, W * s), -3, dtype=torch.int32, device=DEV)
            hk().sparse_upsample(cl(poison(x, mask)), cl(mask), s, out=(d_out, d_om))
            assert _last_kernel() == "upsample_scan_kernel"
            assert torch.equal(d_om.cpu(), want_mask)
            assert_masked_equal(d_out, want, want_mask, "upsample")
            if density == 0.0:
                assert bool(d_out.isnan().all())


SCANNED_POOLS = [
    # C, K, stride, padding, H, W
    (16, 2, 2, 0, 1023, 1031),
    (24, 3, 2, 1, 1021, 1035),
    (8, 3, 1, 1, 515, 513),
    (32, 2, 2, (0, 1, 0, 1), 1023, 1031),   # asymmetric: zero joins the maximum
    (16, 2, 1, 0, 520, 511),               # overlapping 2x2 windows
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cfg", SCANNED_POOLS, ids=lambda c: "-".join(str(v).replace(" ", "") for v in c))
@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("density", [0.0, 0.02, 0.6])
def test_pool_scanned_map(lib, dtype, cfg, mode, density):
    C, K, s, p, H, W = cfg
    K, s, p = _pair(K), _pair(s), _pair(p)
    g = _gen(1600 + C)
    B = 1
    mask = rand_mask(g, B, H, W, density)
    x = torch.randn(B, C, H, W, generator=g).to(dtype)
    prev = torch.randn(B, C, H, W, generator=g).to(dtype)
    want, want_mask = ops.pool(x, prev if mode == 0 else None, mask, K, s, p, (1, 1), mode)
    out, om = hk().sparse_pooling(cl(poison(x, mask)), cl(prev) if mode == 0 else None, K, cl(mask), s, p, (1, 1),
                                  pooling_mode_int=mode)
    assert _last_kernel() == "pool_scan_kernel"
    assert torch.equal(om.cpu(), want_mask)
    assert_masked_equal(out, want, want_mask, "out")


# ------------------------------------------------------------- upsample / concat / mul_add
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [3, 32, 72])
@pytest.mark.parametrize("scale", [2, 4, 8])
def test_upsample(lib, dtype, C, scale):
    g = _gen(1200 + C)
    B, H, W = 2, 6, 5
    mask = rand_mask(g, B, H, W, 0.4)
    x = torch.randn(B, C, H, W, generator=g).to(dtype)
    want, want_mask = ops.upsample(x, mask, scale)
    out, om = hk().sparse_upsample(cl(poison(x, mask)), cl(mask), scale)
    assert torch.equal(om.cpu(), want_mask)
    assert_masked_equal(out, want, want_mask, "out")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [5, 32, 72])
@pytest.mark.parametrize("scale", [2, 4])
@pytest.mark.parametrize("act", [-1, 1])
def test_add_upsampled(lib, dtype, C, scale, act):
    """dc_add_upsampled == DCAdd(a, DCUpsamplingNearest2d(b)) of the oracle, bit for bit."""
    g = _gen(1250 + C + scale)
    B, h, w = 2, 5, 7
    H, W = h * scale, w * scale
    ma, mb = rand_mask(g, B, H, W, 0.3), rand_mask(g, B, h, w, 0.4)
    a = torch.randn(B, C, H, W, generator=g).to(dtype)
    b = torch.randn(B, C, h, w, generator=g).to(dtype)
    prev = torch.randn(B, C, H, W, generator=g).to(dtype) if act > 0 else None
    up, up_mask = ops.upsample(b, mb, scale)
    w_prev = prev.clone() if act > 0 else None
    want, want_mask = ops.add(a, ma, up, up_mask, w_prev, 0.75, -0.5, act, False)
    d_prev = cl(prev) if act > 0 else None
    d_out = torch.full((B, C, H, W), float("nan"), dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
    d_mo = torch.full((B, 1, H, W), -3, dtype=torch.int32, device=DEV)
    hk().sparse_add_upsampled(cl(poison(a, ma)), cl(poison(b, mb)), d_prev, d_out, cl(ma), cl(mb), d_mo,
                              0.75, -0.5, act, scale)
    assert torch.equal(d_mo.cpu(), want_mask)
    assert_masked_equal(d_out, want, want_mask, "out")
    if act > 0:
        assert torch.equal(d_prev.cpu(), w_prev)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Ca,Cb", [(3, 5), (16, 32), (64, 24), (8, 3)])
def test_concat(lib, dtype, Ca, Cb):
    g = _gen(1300 + Ca)
    B, H, W = 2, 7, 6
    ma, mb = rand_mask(g, B, H, W, 0.4), rand_mask(g, B, H, W, 0.4)
    a = torch.randn(B, Ca, H, W, generator=g).to(dtype)
    b = torch.randn(B, Cb, H, W, generator=g).to(dtype)
    want, want_mask = ops.concatenate(a, ma, b, mb)
    out, om = hk().sparse_concatenate((cl(poison(a, ma)), cl(ma)), (cl(poison(b, mb)), cl(mb)))
    assert torch.equal(om.cpu(), want_mask)
    assert_masked_equal(out, want, want_mask, "out")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [3, 32, 100])
@pytest.mark.parametrize("with_bias", [False, True])
def test_mul_add(lib, dtype, C, with_bias):
    g = _gen(1400 + C)
    B, H, W = 2, 7, 6
    mask = rand_mask(g, B, H, W, 0.5)
    x = torch.randn(B, C, H, W, generator=g).to(dtype)
    scale = torch.randn(C, generator=g).to(dtype)
    bias = torch.randn(C, generator=g).to(dtype) if with_bias else None
    want, want_mask = ops.mul_add(x, mask, scale, bias)
    d_x, d_m = cl(poison(x, mask)), cl(mask)
    out = torch.full_like(d_x, float("nan"))
    om = torch.zeros_like(d_m)
    hk().sparse_mul_add(d_x, d_m, out, om, scale.to(DEV), None if bias is None else bias.to(DEV))
    assert torch.equal(om.cpu(), want_mask)
    if dtype == torch.float32 and with_bias:
        assert_masked_close(out, want, want_mask, 1e-6, 1e-6, "out")  # fma vs mul+add in fp64
    else:
        assert_masked_equal(out, want, want_mask, "out")
