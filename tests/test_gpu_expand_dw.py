"""dc_expand_depthwise: a 1x1 expansion whose activation / truncation is left open by its
convolution and finished by the depthwise 3x3 kernel (stride 1 or 2) that consumes it -- two launches
instead of three.  Everything the separate calls leave behind (depthwise output and mask, both layers' cached
states) has to come out bit for bit; the expansion's own output is meaningful on kept pixels."""
import pytest
import torch

from util import DEV, assert_masked_equal, cl, poison, rand_mask

pytestmark = pytest.mark.gpu

CASES = [  # Cin, hidden channels, H, W, batch (, stride of the depthwise layer)
    (64, 384, 14, 14, 1), (96, 576, 14, 14, 1), (160, 960, 7, 7, 1), (24, 144, 28, 28, 1), (32, 192, 20, 23, 2),
    (8, 8, 9, 11, 1), (64, 1024, 5, 6, 1), (16, 96, 56, 56, 1),
    # stride 2: a lane group commits the expansion's state of the 2 x 2 input block it owns (odd sizes: the last
    # row / column of blocks is cut by the map's edge)
    (32, 192, 28, 28, 1, 2), (96, 576, 14, 14, 1, 2), (16, 96, 15, 17, 2, 2), (24, 144, 9, 9, 1, 2), (8, 8, 2, 3, 1, 2),
]


def _stride(case):
    return case[5] if len(case) > 5 else 1


def _out_hw(H, W, stride):
    return (H - 1) // stride + 1, (W - 1) // stride + 1


def _case(dtype, cin, ch, H, W, B, density, seed, raw=False, stride=1):
    from deltacnn_amd.filter_conversion import convert_filter_out_channels_last, convert_half_filter
    g = torch.Generator().manual_seed(seed)
    mask = rand_mask(g, B, H, W, density)
    x = torch.randn(B, cin, H, W, generator=g)
    # half of the updates are far below the expansion's threshold: they get truncated
    x = (x * torch.where(torch.rand(B, 1, H, W, generator=g) < 0.5, 1.0, 1e-3)).to(dtype)
    we = (torch.randn(ch, cin, 1, 1, generator=g) / cin ** 0.5).to(dtype)
    wd = (torch.randn(ch, 1, 3, 3, generator=g) / 3).to(dtype)
    if dtype == torch.float16:
        fe, fd = convert_half_filter(we), convert_half_filter(wd, pixel_wise=True)
    else:
        fe, fd = convert_filter_out_channels_last(we), convert_filter_out_channels_last(wd)
    Ho, Wo = _out_hw(H, W, stride)
    states = [torch.randn(B, ch, h, w, generator=g).to(dtype) * s
              for (s, h, w) in ((1.0, H, W), (0.05, H, W), (1.0, Ho, Wo), (0.05, Ho, Wo))]
    if raw:
        return x, mask, fe.to(DEV), fd.to(DEV), states, we, wd
    return x, mask, fe.to(DEV), fd.to(DEV), states


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["float16", "bfloat16"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "-".join(str(v) for v in c))
@pytest.mark.parametrize("density", [0.15, 1.0])
@pytest.mark.parametrize("acts", [(2, 2), (1, 3)], ids=["relu6", "relu-leaky"])
def test_expand_depthwise_equals_separate_calls(lib, dtype, case, density, acts):
    from deltacnn_amd import _lib
    from deltacnn_amd import hip_kernels as hk
    cin, ch, H, W, B = case[:5]
    st = _stride(case)
    Ho, Wo = _out_hw(H, W, st)
    x, mask, fe, fd, states = _case(dtype, cin, ch, H, W, B, density, 1700 + cin + ch, stride=st)
    pk = hk.pack_filter(fe, cin, ch, 1)
    dx, dm = cl(poison(x, mask)), cl(mask)
    thr_e, thr_d = 0.9, 0.3
    # separate calls
    pe1, te1, pd1, td1 = (cl(t) for t in states)
    e_out, e_mask = hk.sparse_conv_activation(dx, fe, dm, None, pe1, te1, thr_e, acts[0], 0, (1, 1), (0, 0), (1, 1), 1, ch,
                                              packed_filter=pk)
    kept, reached = int(e_mask.sum()), int(mask.sum())
    assert reached < 16 or 0 < kept < reached, (kept, reached)  # some kept, some truncated
    d_out, d_mask = hk.sparse_conv_activation(e_out, fd, e_mask, None, pd1, td1, thr_d, acts[1], 0, (st, st), (1, 1), (1, 1),
                                              ch, ch)
    # the two-launch form
    pe2, te2, pd2, td2 = (cl(t) for t in states)
    geo = hk.conv_geometry((B, ch, H, W), (3, 3), ch, (st, st), (1, 1), (1, 1), ch)
    nan = float("nan")
    e2 = torch.full((B, ch, H, W), nan, dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
    out2 = torch.full((B, ch, Ho, Wo), nan, dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
    em2 = torch.full((B, 1, H, W), -7, dtype=torch.int32, device=DEV)
    om2 = torch.full((B, 1, Ho, Wo), -7, dtype=torch.int32, device=DEV)
    assert hk.sparse_expand_depthwise(dx, dm, pk, pe2, te2, thr_e, acts[0], e2, em2, fd, geo, pd2, td2, thr_d, acts[1], 0,
                                      out2, om2)
    assert _lib.load().dc_last_kernels().decode() == "pw_mfma_kernel+conv_dw_kernel"
    assert torch.equal(om2, d_mask)
    assert_masked_equal(out2, d_out.cpu(), d_mask.cpu(), "depthwise output")
    assert torch.equal(pe1, pe2) and torch.equal(te1, te2), "expansion state"
    assert torch.equal(pd1, pd2) and torch.equal(td1, td2), "depthwise state"
    assert torch.equal(em2.cpu(), mask)  # the expansion's convolution mask, not its keep mask
    assert_masked_equal(e2, e_out.cpu(), e_mask.cpu(), "expansion output on kept pixels")


@pytest.mark.parametrize("case", [CASES[0], CASES[2], CASES[4], CASES[8], CASES[10]], ids=lambda c: "-".join(str(v) for v in c))
@pytest.mark.parametrize("density", [0.15, 1.0])
def test_expand_depthwise_against_oracle_chain(lib, case, density):
    """The two-launch form against the CPU oracle's chain expansion -> activation / truncation ->
    depthwise 3x3 -> activation / truncation (fp16).  A convolution output differs from the oracle's
    in its last bit now and then, which can flip a keep decision that sits on the threshold; such
    pixels are counted and must be rare, everything else has to agree within 2e-2."""
    from deltacnn_amd import hip_kernels as hk
    from oracle import delta_ops as ops
    dtype = torch.float16
    cin, ch, H, W, B = case[:5]
    st = _stride(case)
    Ho, Wo = _out_hw(H, W, st)
    x, mask, fe, fd, states, we, wd = _case(dtype, cin, ch, H, W, B, density, 1900 + cin + ch, raw=True, stride=st)
    thr_e, thr_d, act_e, act_d = 0.9, 0.3, 2, 2
    # oracle
    pe, te, pd, td = (t.clone() for t in states)
    e, em = ops.conv(x, mask, we)
    em = em.clone()
    ops.activate_truncate(e, pe, te, em, thr_e, act_e, 0)
    d, dm = ops.conv(e, em, wd, None, (st, st), (1, 1), (1, 1), ch)
    dm = dm.clone()
    ops.activate_truncate(d, pd, td, dm, thr_d, act_d, 0)
    # library
    pk = hk.pack_filter(fe, cin, ch, 1)
    pe2, te2, pd2, td2 = (cl(t) for t in states)
    geo = hk.conv_geometry((B, ch, H, W), (3, 3), ch, (st, st), (1, 1), (1, 1), ch)
    e2 = torch.zeros((B, ch, H, W), dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
    out2 = torch.zeros((B, ch, Ho, Wo), dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
    em2 = torch.zeros((B, 1, H, W), dtype=torch.int32, device=DEV)
    om2 = torch.zeros((B, 1, Ho, Wo), dtype=torch.int32, device=DEV)
    assert hk.sparse_expand_depthwise(cl(poison(x, mask)), cl(mask), pk, pe2, te2, thr_e, act_e, e2, em2, fd, geo, pd2, td2,
                                      thr_d, act_d, 0, out2, om2)
    flips = int((om2.cpu() != dm).sum())
    assert flips <= max(2, dm.numel() // 100), f"{flips} of {dm.numel()} output mask words differ from the oracle's"
    both = (om2.cpu() != 0) & (dm != 0)
    assert int(both.sum()) > 0
    err = torch.where(both, (out2.cpu().float() - d.float()).abs(), torch.zeros(())).max()
    if flips == 0:
        assert float(err) <= 2e-2, float(err)
        # cached states of the depthwise layer where no decision differs
        assert float((pd2.cpu().float() - pd.float()).abs().max()) <= 2e-2
        assert float((td2.cpu().float() - td.float()).abs().max()) <= 2e-2
    print(f"expand + depthwise vs oracle: {flips} mask words of {dm.numel()} differ, max |diff| on common pixels {float(err):.4f}")


def test_expand_depthwise_declines_what_it_cannot_do(lib):
    """Depthwise layers with a stride beyond 2, maps beyond the per-pixel kernel's range and fp32 have
    no such form: False, nothing launched, nothing touched."""
    from deltacnn_amd import hip_kernels as hk
    dtype = torch.float16
    for (cin, ch, H, W, B, stride, dt) in [(64, 384, 14, 14, 1, 3, dtype), (32, 192, 112, 112, 2, 1, dtype),
                                           (64, 384, 14, 14, 1, 1, torch.float32)]:
        x, mask, fe, fd, states = _case(dtype, cin, ch, H, W, B, 0.5, 1800 + H)
        pk = hk.pack_filter(fe, cin, ch, 1)
        Ho, Wo = (H - 1) // stride + 1, (W - 1) // stride + 1
        geo = hk.conv_geometry((B, ch, H, W), (3, 3), ch, (stride, stride), (1, 1), (1, 1), ch)
        pe, te = cl(states[0]), cl(states[1])
        pd = cl(states[2][:, :, :Ho, :Wo].contiguous())
        td = cl(states[3][:, :, :Ho, :Wo].contiguous())
        before = [t.clone() for t in (pe, te, pd, td)]
        e = torch.zeros(B, ch, H, W, dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
        out = torch.zeros(B, ch, Ho, Wo, dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
        em = torch.zeros(B, 1, H, W, dtype=torch.int32, device=DEV)
        om = torch.zeros(B, 1, Ho, Wo, dtype=torch.int32, device=DEV)
        dx = cl(x).to(dt) if dt != dtype else cl(x)
        assert hk.sparse_expand_depthwise(dx, cl(mask), pk, pe, te, 0.5, 2, e, em, fd, geo, pd, td, 0.5, 2, 0, out, om) is False
        assert all(torch.equal(a, b) for a, b in zip(before, (pe, te, pd, td)))
        assert not bool(out.any()) and not bool(e.any())


def test_mobilenet_open_expansions_keep_every_layer_state(lib):
    """MobileNetV2 224x224, 6 frames: the model whose expansions leave their activation to the
    depthwise kernels against the model that issues every layer call on its own -- logits and
    every activation layer's cached state equal bit for bit; ten blocks of every frame after
    the first take the two-launch form (the 14x14 and 7x7 blocks, the 14x14 -> 7x7 block with its
    stride-2 depthwise layer included), seven of them with the expansion's convolution inside the
    previous block's projection launch."""
    from deltacnn_amd import hip_kernels as hk
    from deltacnn_amd import sparse_layers as SL
    from deltacnn_amd.video import moving_rectangles_video
    from test_gpu_network import _calibrated_state, _mobilenet, _two_hip_models
    video = moving_rectangles_video(frames=6, height=224, width=224, n_rect=3, min_size=16, max_size=60)
    small = moving_rectangles_video(frames=3, height=64, width=96, n_rect=2, min_size=8, max_size=24)
    fused, plain = _two_hip_models(_mobilenet, _calibrated_state(small))
    launches = []
    original = hk.sparse_expand_depthwise

    def counted(*a, **k):
        done = original(*a, **k)
        launches.append(done)
        return done
    pairs = []
    original_pair = hk.sparse_project_expand

    def counted_pair(*a, **k):
        done = original_pair(*a, **k)
        pairs.append(done)
        return done
    hk.sparse_expand_depthwise = counted
    hk.sparse_project_expand = counted_pair
    try:
        with torch.no_grad():
            for t in range(video.shape[0]):
                frame = cl(video[t:t + 1].half())
                SL.DCConv2d.fuse_expansion = SL.DCConv2d.fuse_blocks = True
                got = fused(frame).clone()
                SL.DCConv2d.fuse_expansion = SL.DCConv2d.fuse_blocks = False
                want = plain(frame)
                assert torch.equal(got, want), f"frame {t}"
        fm, pm = dict(fused.named_modules()), dict(plain.named_modules())
        n = 0
        for name, mod in fm.items():
            if isinstance(mod, SL.DCActivation):
                assert torch.equal(mod.prev_out, pm[name].prev_out), name
                assert torch.equal(mod.out_truncated, pm[name].out_truncated), name
                n += 1
        assert n == 35
        assert sum(launches) == 10 * (video.shape[0] - 1), (len(launches), sum(launches))
        # ... and seven projections carry the next block's expansion (the 14x14 blocks of 64 and 96 channels)
        assert sum(pairs) == 7 * (video.shape[0] - 1), (len(pairs), sum(pairs))
    finally:
        SL.DCConv2d.fuse_expansion = SL.DCConv2d.fuse_blocks = True
        hk.sparse_expand_depthwise = original
        hk.sparse_project_expand = original_pair
