"""Host-side checks of the C-ABI library that need no GPU: it loads, exports every entry point
the public header declares, rejects bad arguments with the documented codes before touching
the device, and the Python shim refuses to run without it (there is no CPU fallback)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "deltacnn_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return sorted(set(re.findall(r"\b(dc_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_the_operator_set():
    names = declared_symbols()
    for op in ("sparsify", "activate_truncate", "conv", "deconv", "pool", "add", "add_to_dense", "densify",
               "upsample", "concat", "mul_add", "version", "last_error"):
        assert f"dc_{op}" in names


def test_library_exports_every_declared_symbol(lib):
    raw = ctypes.CDLL(lib._name)
    for name in declared_symbols():
        assert hasattr(raw, name), f"{name} is declared in the header but not exported"


def test_python_bindings_cover_the_header(lib):
    from deltacnn_amd import _lib
    assert sorted(_lib._SIGNATURES) == declared_symbols()


def test_version_and_error_string(lib):
    assert b"gfx950" in lib.dc_version()
    assert isinstance(lib.dc_last_error(), bytes)


def _geom(**kw):
    from deltacnn_amd._lib import Geometry
    base = dict(batch=1, in_h=8, in_w=8, in_c=16, out_h=8, out_w=8, out_c=16, kernel_h=3, kernel_w=3,
                stride_h=1, stride_w=1, dilation_h=1, dilation_w=1, pad_top=1, pad_left=1, pad_bottom=1,
                pad_right=1, groups=1)
    base.update(kw)
    return Geometry(**base)


def test_bad_arguments_are_rejected_before_any_launch(lib):
    """Error codes: -1 dtype, -2 shape, -3 unsupported, -4 null, -5 alignment."""
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    assert lib.dc_sparsify(p, p, p, p, 0.1, 16, 4, 7, None) == -1
    assert b"dtype" in lib.dc_last_error()
    assert lib.dc_sparsify(None, p, p, p, 0.1, 16, 4, 0, None) == -4
    assert lib.dc_sparsify(p, p, p, p, 0.1, 0, 4, 0, None) == -2
    assert lib.dc_sparsify(p, p, p, p, 0.1, 16, -1, 0, None) == -2
    assert lib.dc_activate_truncate(p, p, None, p, 0.1, 1, 0, 16, 4, 0, None) == -4   # truncation needs its cache
    assert lib.dc_activate_truncate(p, p, p, p, 0.1, 9, 0, 16, 4, 0, None) == -3      # unknown activation
    # geometry: output size that does not follow from the input size
    g = _geom(out_h=7)
    assert lib.dc_conv(ctypes.byref(g), p, p, None, None, p, p, p, 0, None) == -2
    assert b"expected 8x8" in lib.dc_last_error()
    g = _geom(groups=3)
    assert lib.dc_conv(ctypes.byref(g), p, p, None, None, p, p, p, 0, None) == -2
    g = _geom()
    assert lib.dc_conv(ctypes.byref(g), None, p, None, None, p, p, p, 0, None) == -4
    assert lib.dc_conv(None, p, p, None, None, p, p, p, 0, None) == -4
    # transposed convolution with asymmetric padding is not defined
    g = _geom(kernel_h=4, kernel_w=4, stride_h=2, stride_w=2, pad_bottom=2, out_h=15, out_w=16)
    assert lib.dc_deconv(ctypes.byref(g), p, p, None, None, p, p, p, 0, None) == -3
    # pooling keeps the channel count
    g = _geom(out_c=8)
    assert lib.dc_pool(ctypes.byref(g), p, p, p, p, p, 0, 0, 0, None) == -2
    # a 1x1 output in the tensor's own type needs window == whole unpadded map
    g = _geom(in_h=8, in_w=8, out_h=1, out_w=1, kernel_h=8, kernel_w=8, pad_top=0, pad_left=0, pad_bottom=0, pad_right=0)
    assert lib.dc_pool(ctypes.byref(g), p, p, p, p, p, 1, 1, 2, None) == -1
    g = _geom(in_h=6, in_w=6, out_h=1, out_w=1, kernel_h=8, kernel_w=8)
    assert lib.dc_pool(ctypes.byref(g), p, p, p, p, p, 1, 1, 1, None) == -3
    assert lib.dc_densify(p, p, None, p, 16, 4, 0, None) == -4
    # the sum with an upsampled operand: sizes must be multiples of the scale
    assert lib.dc_add_upsampled(p, p, None, p, p, p, p, 1.0, 1.0, 0, 1, 6, 8, 4, 4, 0, None) == -2
    assert b"multiple of scale" in lib.dc_last_error()
    assert lib.dc_add_upsampled(p, p, None, p, p, p, p, 1.0, 1.0, 0, 1, 8, 8, 4, 0, 0, None) == -2
    assert lib.dc_add_upsampled(p, p, None, p, p, p, p, 1.0, 1.0, 1, 1, 8, 8, 4, 2, 0, None) == -4   # activation needs prev_out
    assert lib.dc_add_upsampled(p, p, None, p, p, p, None, 1.0, 1.0, 0, 1, 8, 8, 4, 2, 0, None) == -4


def test_packed_filter_size_is_host_arithmetic(lib):
    """fp16, groups 1: round_up(Cout, 16) * taps * round_up(Cin, 32) halves; no packed form for
    fp32 or grouped convolutions (0)."""
    g = _geom(in_c=24, out_c=40)
    assert lib.dc_packed_filter_bytes(ctypes.byref(g), 1, 0) == 48 * 9 * 32 * 2
    assert lib.dc_packed_filter_bytes(ctypes.byref(g), 0, 0) == 0
    g = _geom(groups=16)
    assert lib.dc_packed_filter_bytes(ctypes.byref(g), 1, 0) == 0
    # stems (Cin <= 4, window <= 8 x 8, Cout <= 64 and a multiple of 4): one KB per (channel tile, row)
    g = _geom(in_c=3, out_c=24, kernel_h=7, kernel_w=7)
    assert lib.dc_packed_filter_bytes(ctypes.byref(g), 1, 0) == 2 * 7 * 1024
    assert lib.dc_packed_filter_bytes(ctypes.byref(g), 1, 1) == 0      # not for transposed convolutions
    assert lib.dc_packed_filter_bytes(ctypes.byref(g), 0, 0) == 0      # fp32
    for bad in (dict(in_c=5), dict(out_c=22), dict(out_c=80), dict(kernel_h=9, kernel_w=9)):
        g = _geom(**{**dict(in_c=3, out_c=24, kernel_h=7, kernel_w=7), **bad})
        assert lib.dc_packed_filter_bytes(ctypes.byref(g), 1, 0) == 0, bad


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from deltacnn_amd import _lib
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libdeltacnn_hip.so"))
    monkeypatch.setattr(_lib, "_lib", None)
    with pytest.raises(ImportError):
        _lib.load()


def test_package_does_not_import_the_oracle():
    """The oracle is test infrastructure: nothing under deltacnn_amd/ may import it."""
    pkg = os.path.join(ROOT, "deltacnn_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith(".py"):
                src = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", src, flags=re.M), f


@pytest.mark.parametrize("k,s,p,d", [(3, 1, 1, 1), (3, 2, 1, 1), (1, 1, 0, 1), (5, 2, 2, 1), (3, 1, 2, 2), (7, 2, 3, 1)])
def test_conv_geometry_matches_torch(k, s, p, d):
    from deltacnn_amd.hip_kernels import conv_geometry
    x = torch.zeros(2, 4, 23, 17)
    want = torch.nn.functional.conv2d(x, torch.zeros(6, 4, k, k), stride=s, padding=p, dilation=d).shape
    g = conv_geometry(x.shape, (k, k), 6, (s, s), (p, p), (d, d), 1)
    assert (g.batch, g.out_c, g.out_h, g.out_w) == tuple(want)
    # transposed: the reference formula has no output_padding term
    gt = conv_geometry(x.shape, (4, 4), 6, (2, 2), (1, 1), (1, 1), 1, True)
    want = torch.nn.functional.conv_transpose2d(x, torch.zeros(4, 6, 4, 4), stride=2, padding=1).shape
    assert (gt.out_h, gt.out_w) == tuple(want[2:])


def test_filter_layouts():
    """fp32: W_dc[ci,ky,kx,co] = W[co,ci,ky,kx] (transposed: W[ci,co,ky,kx]).  fp16: channels
    padded to even, W[ci,co] stored at row ci ^ (co & 1) -- written out as the four cases of the
    2x2 pair swizzle of filter_conversion.py:34-37."""
    from deltacnn_amd.filter_conversion import (convert_filter_out_channels_last, convert_half_filter,
                                                 restore_half_filter)
    g = torch.Generator().manual_seed(1)
    w = torch.randn(5, 7, 3, 3, generator=g)   # Cout=5, Cin=7
    f = convert_filter_out_channels_last(w)
    assert f.shape == (7, 3, 3, 5) and f.is_contiguous()
    assert float(f[2, 1, 0, 4]) == float(w[4, 2, 1, 0])
    ft = convert_filter_out_channels_last(w, transposed=True)
    assert ft.shape == (5, 3, 3, 7) and float(ft[4, 1, 0, 2]) == float(w[4, 2, 1, 0])
    h = convert_half_filter(w)
    assert h.shape == (8, 3, 3, 6) and h.dtype == torch.float16
    wh = w.half()
    W = torch.zeros(8, 3, 3, 6, dtype=torch.float16)
    W[:7, :, :, :5] = wh.permute(1, 2, 3, 0)
    for i in range(4):
        for j in range(3):
            assert torch.equal(h[2 * i, :, :, 2 * j], W[2 * i, :, :, 2 * j])
            assert torch.equal(h[2 * i, :, :, 2 * j + 1], W[2 * i + 1, :, :, 2 * j + 1])
            assert torch.equal(h[2 * i + 1, :, :, 2 * j], W[2 * i + 1, :, :, 2 * j])
            assert torch.equal(h[2 * i + 1, :, :, 2 * j + 1], W[2 * i, :, :, 2 * j + 1])
    assert torch.equal(restore_half_filter(h, 7, 5), wh.permute(1, 2, 3, 0))
    dw = torch.randn(6, 1, 3, 3, generator=g)
    assert convert_half_filter(dw, pixel_wise=True).shape == (1, 3, 3, 6)


def test_packed_form_rule_matches_the_library(lib):
    """tests/util.packed_form_exists (used to build GPU parametrisations) states the same rule
    as dc_packed_filter_bytes."""
    import sys
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from util import packed_form_exists
    from deltacnn_amd._lib import DC_BF16, DC_F16, DC_F32, Geometry
    for cin in (1, 3, 4, 5, 8, 12, 16, 24, 40, 320):
        for cout in (2, 4, 16, 30, 64, 68, 256):
            for k in (1, 3, 7, 8, 9):
                for groups in (1, 2):
                    if cin % groups or cout % groups:
                        continue
                    for transposed in (False, True):
                        for dtype, code in ((torch.float16, DC_F16), (torch.float32, DC_F32), (torch.bfloat16, DC_BF16)):
                            g = Geometry(1, 1, 1, cin, 1, 1, cout, k, k, 1, 1, 1, 1, 0, 0, 0, 0, groups)
                            have = lib.dc_packed_filter_bytes(g, code, int(transposed)) != 0
                            assert have == packed_form_exists(dtype, cin, cout, k, groups, transposed), \
                                (cin, cout, k, groups, transposed, dtype)


def test_block_arguments_are_checked_before_any_launch(lib):
    """dc_block: shape rules -> -3 (the caller then issues the separate calls), missing operands
    -> -4, misaligned feature pointers -> -5; all without touching a device."""
    from deltacnn_amd._lib import BlockArgs
    buf = (ctypes.c_char * 8192)()
    p = (ctypes.addressof(buf) + 255) // 256 * 256
    g = _geom(in_c=64, out_c=64, groups=64)   # depthwise 3x3, stride 1, padding 1

    def args(**kw):
        a = BlockArgs()
        for name in ("input", "mask", "dw_filter", "dw_prev_out", "dw_truncated", "project_packed_filter", "out",
                     "out_mask"):
            setattr(a, name, p)
        a.dw_threshold, a.dw_activation, a.dw_truncation_mode = 0.05, 2, 0
        a.project_channels, a.weight_residual, a.weight_conv = 24, 1.0, 1.0
        for k, v in kw.items():
            setattr(a, k, v)
        return a

    def call(geom, a, dtype=1):
        return lib.dc_block(ctypes.byref(geom), ctypes.byref(a), dtype, None)

    assert call(g, args(), dtype=0) == -3 and b"fp16 only" in lib.dc_last_error()
    assert call(g, args(), dtype=7) == -1
    assert call(_geom(in_c=64, out_c=64, groups=1), args()) == -3          # not depthwise
    assert call(_geom(in_c=60, out_c=60, groups=60), args()) == -3         # hidden channels not a multiple of 8
    assert call(g, args(project_channels=20)) == -3                       # projection channels not a multiple of 8
    assert call(g, args(dw_activation=4)) == -3                           # sigmoid
    assert call(g, args(dw_truncation_mode=1)) == -3                      # norm truncation
    assert call(g, args(expand_channels=96, expand_activation=1, expand_truncation_mode=0)) == -3  # activations differ
    assert call(_geom(in_c=64, out_c=64, groups=64, out_h=7), args()) == -2
    assert lib.dc_block(None, ctypes.byref(args()), 1, None) == -4
    assert lib.dc_block(ctypes.byref(g), None, 1, None) == -4
    assert call(g, args(out=None)) == -4
    assert call(g, args(residual=p)) == -4                                # a residual needs its mask
    assert call(g, args(expand_channels=96, expand_activation=2)) == -4   # expansion operands missing
    assert call(g, args(input=p + 2)) == -5
    assert call(g, args(out=p + 4)) == -5


def test_head_entry_points_check_their_arguments(lib):
    """dc_pool_densify and dc_linear: shapes without the one-launch form -> -3 (the caller issues
    the separate calls / torch's linear), bad sizes -> -2, missing operands -> -4, alignment -> -5."""
    buf = (ctypes.c_char * 8192)()
    p = (ctypes.addressof(buf) + 255) // 256 * 256
    whole = _geom(in_h=7, in_w=7, in_c=64, out_h=1, out_w=1, out_c=64, kernel_h=7, kernel_w=7, pad_top=0,
                  pad_left=0, pad_bottom=0, pad_right=0)

    def pool(g, x=p, m=p, acc=p, out=p, dtype=1):
        return lib.dc_pool_densify(ctypes.byref(g), x, m, acc, out, dtype, None)

    assert pool(whole, dtype=9) == -1
    assert pool(whole, x=None) == -4 and pool(whole, acc=None) == -4 and pool(whole, out=None) == -4
    assert pool(whole, acc=p + 1) == -5
    assert pool(whole, x=p + 2) == -3                                    # input not 16-byte aligned
    window = _geom(in_h=8, in_w=8, in_c=64, out_h=4, out_w=4, out_c=64, kernel_h=2, kernel_w=2, stride_h=2,
                   stride_w=2, pad_top=0, pad_left=0, pad_bottom=0, pad_right=0)
    assert pool(window) == -3                                            # not a global pooling
    odd = _geom(in_h=7, in_w=7, in_c=60, out_h=1, out_w=1, out_c=60, kernel_h=7, kernel_w=7, pad_top=0,
                pad_left=0, pad_bottom=0, pad_right=0)
    assert pool(odd) == -3                                               # 60 halves do not fill 16-byte vectors
    assert lib.dc_pool_densify(None, p, p, p, p, 1, None) == -4

    def linear(x=p, w=p, b=p, out=p, rows=1, fi=64, fo=10, dtype=1):
        return lib.dc_linear(x, w, b, out, rows, fi, fo, dtype, None)

    assert linear(dtype=5) == -1
    assert linear(rows=0) == -2 and linear(fi=0) == -2 and linear(fo=-3) == -2
    assert linear(fi=36) == -3 and b"16-byte" in lib.dc_last_error()     # 36 halves
    assert linear(x=None) == -4 and linear(w=None) == -4 and linear(out=None) == -4
    assert linear(x=p + 8) == -5 and linear(w=p + 2) == -5 and linear(out=p + 1) == -5


def test_expand_depthwise_arguments_are_checked_before_any_launch(lib):
    """dc_expand_depthwise: shapes without the two-launch form -> -3 (the caller issues the
    separate calls), missing operands -> -4, misaligned pointers -> -5; nothing touches a device."""
    from deltacnn_amd._lib import ExpandDwArgs
    buf = (ctypes.c_char * 8192)()
    p = (ctypes.addressof(buf) + 255) // 256 * 256
    g = _geom(in_h=14, in_w=14, out_h=14, out_w=14, in_c=384, out_c=384, groups=384)

    def args(**kw):
        a = ExpandDwArgs()
        for name in ("input", "mask", "expand_packed_filter", "expand_prev_out", "expand_truncated", "expand_out",
                     "expand_out_mask", "dw_filter", "dw_prev_out", "dw_truncated", "out", "out_mask"):
            setattr(a, name, p)
        a.expand_in_channels, a.expand_threshold, a.expand_activation, a.expand_truncation_mode = 64, 0.05, 2, 0
        a.dw_threshold, a.dw_activation, a.dw_truncation_mode = 0.05, 2, 0
        for k, v in kw.items():
            setattr(a, k, v)
        return a

    def call(geom, a, dtype=1):
        return lib.dc_expand_depthwise(ctypes.byref(geom), ctypes.byref(a), dtype, None)

    assert call(g, args(), dtype=0) == -3 and b"16-bit" in lib.dc_last_error()
    assert call(g, args(), dtype=9) == -1
    assert call(g, args(expand_in_channels=0)) == -2
    assert call(g, args(expand_in_channels=20)) == -3                      # not a multiple of 8
    assert call(g, args(expand_truncation_mode=1)) == -3                   # norm truncation of the expansion
    assert call(g, args(dw_truncation_mode=-1)) == -3                      # a depthwise layer without truncation
    assert call(_geom(in_h=14, in_w=14, out_h=5, out_w=5, in_c=384, out_c=384, groups=384, stride_h=3, stride_w=3),
                args()) == -3                                              # a stride beyond 2
    assert call(_geom(in_h=14, in_w=14, out_h=14, out_w=14, in_c=384, out_c=384, groups=1), args()) == -3  # not depthwise
    assert call(_geom(in_h=224, in_w=224, out_h=224, out_w=224, in_c=96, out_c=96, groups=96), args()) == -3  # too large
    assert lib.dc_expand_depthwise(None, ctypes.byref(args()), 1, None) == -4
    assert lib.dc_expand_depthwise(ctypes.byref(g), None, 1, None) == -4
    assert call(g, args(out=None)) == -4 and call(g, args(expand_truncated=None)) == -4
    assert call(g, args(input=p + 2)) == -5 and call(g, args(dw_prev_out=p + 8)) == -5


def test_project_expand_arguments_are_checked_before_any_launch(lib):
    """dc_project_expand: shapes without the one-launch form, or whose expansion the depthwise
    layer behind it could not finish -> -3 (the caller issues the separate calls), missing
    operands -> -4, misaligned pointers -> -5; nothing touches a device.  dc_expand_depthwise
    accepts a missing expansion filter (the convolution has run already) but no missing state."""
    from deltacnn_amd._lib import ExpandDwArgs, ProjectExpandArgs
    buf = (ctypes.c_char * 8192)()
    p = (ctypes.addressof(buf) + 255) // 256 * 256
    one = dict(kernel_h=1, kernel_w=1, pad_top=0, pad_left=0, pad_bottom=0, pad_right=0)
    g = _geom(in_h=14, in_w=14, out_h=14, out_w=14, in_c=384, out_c=64, **one)
    gd = _geom(in_h=14, in_w=14, out_h=14, out_w=14, in_c=384, out_c=384, groups=384)

    def args(dw=gd, **kw):
        a = ProjectExpandArgs()
        for name in ("input", "mask", "project_packed_filter", "residual", "residual_mask", "out", "out_mask",
                     "expand_packed_filter", "expand_prev_out", "expand_truncated", "expand_out", "expand_out_mask"):
            setattr(a, name, p)
        a.weight_residual = a.weight_conv = 1.0
        a.expand_channels, a.expand_activation, a.dw_activation, a.dw_truncation_mode = 384, 2, 2, 0
        a.dw_geometry = ctypes.pointer(dw) if dw is not None else None
        for k, v in kw.items():
            setattr(a, k, v)
        return a

    def call(geom, a, dtype=1):
        return lib.dc_project_expand(ctypes.byref(geom), ctypes.byref(a), dtype, None)

    assert call(g, args(), dtype=0) == -3 and b"16-bit" in lib.dc_last_error()
    assert call(g, args(), dtype=9) == -1
    assert call(g, args(expand_channels=0)) == -2
    assert call(g, args(expand_activation=3)) == -3                        # leaky ReLU has no open form
    assert call(_geom(in_h=14, in_w=14, out_h=14, out_w=14, in_c=384, out_c=48, **one), args()) == -3   # 48 channels
    assert call(_geom(in_h=14, in_w=14, out_h=14, out_w=14, in_c=960, out_c=160, **one), args()) == -3  # too wide
    assert call(_geom(in_h=14, in_w=14, out_h=14, out_w=14, in_c=384, out_c=64), args()) == -3          # 3x3
    strided = _geom(in_h=14, in_w=14, out_h=5, out_w=5, in_c=384, out_c=384, groups=384, stride_h=3, stride_w=3)
    assert call(g, args(dw=strided)) == -3 and b"depthwise" in lib.dc_last_error()
    other = _geom(in_h=7, in_w=7, out_h=7, out_w=7, in_c=384, out_c=384, groups=384)
    assert call(g, args(dw=other)) == -2                                   # not on the expansion's output map
    assert call(g, args(dw=None)) == -4
    assert lib.dc_project_expand(None, ctypes.byref(args()), 1, None) == -4
    assert lib.dc_project_expand(ctypes.byref(g), None, 1, None) == -4
    assert call(g, args(out=None)) == -4 and call(g, args(expand_truncated=None)) == -4
    assert call(g, args(residual_mask=None)) == -4                         # a residual needs its mask
    assert call(g, args(input=p + 2)) == -5 and call(g, args(expand_prev_out=p + 8)) == -5

    # nothing is summed in place: several workgroups read every input while one stores the outputs
    big = (ctypes.c_char * (4 << 20))()
    q = (ctypes.addressof(big) + 255) // 256 * 256
    names = ("input", "mask", "project_packed_filter", "residual", "residual_mask", "out", "out_mask",
             "expand_packed_filter", "expand_prev_out", "expand_truncated", "expand_out", "expand_out_mask")
    apart = {n: q + i * (256 << 10) for i, n in enumerate(names)}      # 256 KB each: larger than any operand
    for written, read in (("out", "residual"), ("out", "input"), ("out_mask", "mask"), ("expand_out_mask", "residual_mask"),
                          ("out_mask", "residual_mask"), ("expand_out", "out"), ("expand_truncated", "expand_prev_out"),
                          ("expand_out", "expand_truncated"), ("out_mask", "expand_out_mask")):
        alias = dict(apart)
        alias[written] = apart[read]
        assert call(g, args(**alias)) == -3 and b"overlap" in lib.dc_last_error(), (written, read)
    partly = dict(apart)
    partly["out"] = apart["residual"] + 1024                               # a view into the same allocation
    assert call(g, args(**partly)) == -3 and b"overlap" in lib.dc_last_error()

    # the second call of the pair: no expansion filter, no input, but every state tensor
    b = ExpandDwArgs()
    for name in ("expand_prev_out", "expand_truncated", "expand_out", "expand_out_mask", "dw_filter", "dw_prev_out",
                 "dw_truncated", "out", "out_mask"):
        setattr(b, name, p)
    b.expand_in_channels, b.expand_threshold, b.expand_activation, b.expand_truncation_mode = 64, 0.05, 2, 0
    b.dw_threshold, b.dw_activation, b.dw_truncation_mode = 0.05, 2, 0
    b.expand_truncated = None
    assert lib.dc_expand_depthwise(ctypes.byref(gd), ctypes.byref(b), 1, None) == -4
    b.expand_truncated, b.dw_truncated = p, p + 8
    assert lib.dc_expand_depthwise(ctypes.byref(gd), ctypes.byref(b), 1, None) == -5


def test_deconv_add_arguments_are_checked_before_any_launch(lib):
    """dc_deconv_add: layers without the fused form -> -3 (the caller issues the two calls), a
    sum taken in place -> -3, missing operands -> -4, misaligned pointers -> -5; nothing touches
    a device."""
    big = (ctypes.c_char * (8 << 20))()
    q = (ctypes.addressof(big) + 255) // 256 * 256
    names = ("input", "packed_filter", "mask", "residual", "mask_residual", "out", "out_mask")
    g = _geom(in_h=34, in_w=60, out_h=68, out_w=120, in_c=64, out_c=64, kernel_h=4, kernel_w=4, stride_h=2, stride_w=2)

    def call(geom=g, dtype=1, **kw):
        a = {n: q + i * (1 << 20) for i, n in enumerate(names)}  # 1 MB apart: 68 * 120 * 64 * 2 = 1.04e6 bytes fit
        a.update(kw)
        return lib.dc_deconv_add(ctypes.byref(geom), *[a[n] for n in names], 1.0, 1.0, dtype, None)

    assert call(dtype=9) == -1
    assert call(dtype=0) == -3 and b"16-bit" in lib.dc_last_error()
    small = _geom(in_h=9, in_w=11, out_h=18, out_w=22, in_c=16, out_c=8, kernel_h=4, kernel_w=4, stride_h=2, stride_w=2)
    assert call(geom=small) == -3                                           # the 4x4-patch kernel's layer
    gap = _geom(in_h=30, in_w=31, out_h=89, out_w=92, in_c=64, out_c=64, kernel_h=2, kernel_w=2, stride_h=3, stride_w=3,
                pad_top=0, pad_left=0, pad_bottom=0, pad_right=0)
    assert call(geom=gap) == -3                                             # stride phases without a tap
    assert call(geom=_geom(in_h=34, in_w=60, out_h=70, out_w=120, in_c=64, out_c=64, kernel_h=4, kernel_w=4,
                           stride_h=2, stride_w=2)) == -2                   # output size does not match
    assert lib.dc_deconv_add(None, q, q, q, q, q, q, q, 1.0, 1.0, 1, None) == -4
    assert call(residual=None) == -4 and call(out_mask=None) == -4
    assert call(input=q + 2) == -5 and call(out=q + 5 * (1 << 20) + 4) == -5
    assert call(out=q + 3 * (1 << 20)) == -3 and b"overlap" in lib.dc_last_error()          # summed in place
    assert call(out_mask=q + 2 * (1 << 20) + 64) == -3 and b"overlap" in lib.dc_last_error()


def test_pool_update_arguments_are_checked_before_any_launch(lib):
    """dc_pool_update: windows that do not tile the map, channels off the vector size -> -3 (the
    caller issues dc_pool and dc_add_to_dense), outputs that overlap the operands -> -3, missing
    operands -> -4; nothing touches a device."""
    big = (ctypes.c_char * (4 << 20))()
    q = (ctypes.addressof(big) + 255) // 256 * 256
    names = ("input", "prev_input", "out", "mask", "out_mask")
    two = dict(kernel_h=2, kernel_w=2, stride_h=2, stride_w=2, pad_top=0, pad_left=0, pad_bottom=0, pad_right=0)
    g = _geom(in_h=34, in_w=60, out_h=17, out_w=30, in_c=64, out_c=64, **two)

    def call(geom=g, dtype=1, **kw):
        a = {n: q + i * (512 << 10) for i, n in enumerate(names)}  # 34 * 60 * 64 * 2 = 261 120 bytes fit
        a.update(kw)
        return lib.dc_pool_update(ctypes.byref(geom), *[a[n] for n in names], dtype, None)

    assert call(dtype=9) == -1
    assert call(geom=_geom(in_h=35, in_w=60, out_h=17, out_w=30, in_c=64, out_c=64, **two)) == -3   # a row left over
    assert call(geom=_geom(in_h=34, in_w=60, out_h=17, out_w=30, in_c=20, out_c=20, **two)) == -3   # 20 channels
    over = dict(two, kernel_h=3, kernel_w=3, pad_top=1, pad_left=1, pad_bottom=1, pad_right=1)
    assert call(geom=_geom(in_h=34, in_w=60, out_h=17, out_w=30, in_c=64, out_c=64, **over)) == -3  # overlapping windows
    assert call(prev_input=None) == -4 and call(out_mask=None) == -4
    assert call(out=q + (512 << 10) + 4096) == -3 and b"overlap" in lib.dc_last_error()
    assert call(prev_input=q) == -3 and b"overlap" in lib.dc_last_error()


def test_conv_group_arguments_are_checked_before_any_launch(lib):
    """dc_conv_group: a count outside 2..8 -> -2; an item the 4x4-patch kernel does not take, an
    item with both a residual sum and an activation, activations of two kinds for the second
    launch, items that share a buffer one of them writes -> -3 (the caller issues the separate
    calls); missing operands -> -4; misaligned pointers -> -5; nothing touches a device."""
    from deltacnn_amd._lib import ConvItem
    buf = (ctypes.c_char * 65536)()
    base = (ctypes.addressof(buf) + 255) // 256 * 256

    def item(k, geom=None, **kw):
        it = ConvItem()
        it.geometry = geom if geom is not None else _geom(in_h=16, in_w=16, out_h=16, out_w=16, in_c=64, out_c=64)
        p = base + k * 4096  # every item its own buffers
        for j, name in enumerate(("input", "mask", "packed_filter", "out", "out_mask")):
            setattr(it, name, p + j * 256)
        it.weight_residual = it.weight_conv = 1.0
        for name, v in kw.items():
            setattr(it, name, v)
        return it

    def call(items, dtype=1, count=None):
        arr = (ConvItem * len(items))(*items)
        return lib.dc_conv_group(arr, len(items) if count is None else count, dtype, None)

    def act(k, a=1):
        p = base + k * 4096
        return dict(prev_out=p + 2048, truncated=p + 2304, threshold=0.05, activation=a, truncation_mode=0)

    assert call([item(0), item(1)], dtype=9) == -1
    assert call([item(0), item(1)], dtype=0) == -3                          # fp32
    assert call([item(0)]) == -2 and call([item(k) for k in range(9)]) == -2
    assert lib.dc_conv_group(None, 2, 1, None) == -4
    assert call([item(0), item(1, out=None)]) == -4
    assert call([item(0), item(1, input=base + 4096 + 2)]) == -5
    big = _geom(in_h=136, in_w=240, out_h=136, out_w=240, in_c=64, out_c=64)
    assert call([item(0), item(1, geom=big)]) == -3 and b"item 1" in lib.dc_last_error()
    one = _geom(in_h=16, in_w=16, out_h=16, out_w=16, in_c=64, out_c=64, kernel_h=1, kernel_w=1, pad_top=0, pad_left=0,
                pad_bottom=0, pad_right=0)
    assert call([item(0, geom=one), item(1)]) == -3                          # the pointwise kernels' layer
    both = dict(act(1), residual=base + 4096 + 1024, residual_mask=base + 4096 + 1280)
    assert call([item(0), item(1, **both)]) == -3 and b"residual sum and an activation" in lib.dc_last_error()
    assert call([item(0, **act(0)), item(1, **dict(act(1), truncation_mode=1))]) == -3   # norm truncation
    assert call([item(0, **act(0)), item(1, **dict(act(1), truncated=None))]) == -4
    assert call([item(0, **act(0, 1)), item(1, **act(1, 3))]) == -3 and b"activations" in lib.dc_last_error()
    assert call([item(0), item(1, out=base + 3 * 256)]) == -3 and b"share" in lib.dc_last_error()
    assert call([item(0), item(1, input=base + 3 * 256)]) == -3            # item 1 reads what item 0 writes
    # byte ranges, not pointers: views into one allocation, and every buffer an item writes
    wide = (ctypes.c_char * (4 << 20))()
    w0 = (ctypes.addressof(wide) + 255) // 256 * 256

    def roomy(k, **kw):  # 16 x 16 x 64 channels = 32 KB per tensor, 64 KB apart
        names = ("input", "mask", "packed_filter", "out", "out_mask", "prev_out", "truncated")
        d = {n: w0 + (k * 8 + j) * (64 << 10) for j, n in enumerate(names)}
        d.update(threshold=0.05, activation=1, truncation_mode=0)
        d.update(kw)
        return item(k, **d)

    for kw in (dict(out=w0 + 3 * (64 << 10) + 512), dict(input=w0 + 5 * (64 << 10) + 64),
               dict(prev_out=w0 + 3 * (64 << 10)), dict(truncated=w0 + 0 * (64 << 10) + 4096),
               dict(out_mask=w0 + 1 * (64 << 10) + 16)):
        assert call([roomy(0), roomy(1, **kw)]) == -3 and b"share" in lib.dc_last_error(), kw
    assert call([item(0, residual=base + 1024)]) == -2                       # still one item
    assert call([item(0), item(1, residual=base + 4096 + 1024)]) == -4       # a residual needs its mask


def test_add_group_arguments_are_checked_before_any_launch(lib):
    """dc_add_group: a count outside 2..8 or a map that is no multiple of the scale -> -2; channel
    counts off the vector size, fp32, sums that share a buffer one of them writes -> -3; missing
    operands -> -4; nothing touches a device."""
    from deltacnn_amd._lib import AddItem
    buf = (ctypes.c_char * 65536)()
    base = (ctypes.addressof(buf) + 255) // 256 * 256

    def item(k, **kw):
        it = AddItem()
        p = base + k * 4096
        for j, name in enumerate(("a", "b", "prev_out", "out", "mask_a", "mask_b", "mask_out")):
            setattr(it, name, p + j * 256)
        it.weight_a = it.weight_b = 1.0
        it.batch, it.height, it.width, it.channels, it.scale = 1, 8, 8, 32, 2
        for name, v in kw.items():
            setattr(it, name, v)
        return it

    def call(items, dtype=1):
        arr = (AddItem * len(items))(*items)
        return lib.dc_add_group(arr, len(items), dtype, None)

    assert call([item(0), item(1)], dtype=9) == -1
    assert call([item(0), item(1)], dtype=0) == -3
    assert call([item(0)]) == -2 and call([item(k) for k in range(9)]) == -2
    assert lib.dc_add_group(None, 2, 1, None) == -4
    assert call([item(0), item(1, height=7)]) == -2 and b"multiple of scale" in lib.dc_last_error()
    assert call([item(0), item(1, channels=12)]) == -3
    assert call([item(0), item(1, a=base + 4096 + 2)]) == -3                 # not a 16-byte aligned row
    assert call([item(0), item(1, out=None)]) == -4
    assert call([item(0), item(1, activation=1, prev_out=None)]) == -4
    assert call([item(0), item(1, activation=9)]) == -3
    assert call([item(0), item(1, out=base + 3 * 256)]) == -3 and b"share" in lib.dc_last_error()
    assert call([item(0), item(1, b=base + 3 * 256)]) == -3                  # item 1 reads what item 0 writes
