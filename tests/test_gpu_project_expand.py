"""dc_project_expand: the 1x1 projection that ends an inverted-residual block (+ the block's
residual sum) and the next block's 1x1 expansion in ONE launch, the expansion's activation left
open for the depthwise kernel behind it (dc_expand_depthwise without its first launch).
Everything the separate calls leave behind -- block output and mask, the depthwise output and
mask, both activation layers' cached states -- has to come out bit for bit."""
import pytest
import torch

from util import DEV, assert_masked_equal, cl, poison, rand_mask

pytestmark = pytest.mark.gpu

CASES = [  # hidden channels, block channels, next hidden channels, H, W, batch (, stride of the closing depthwise layer)
    (384, 64, 384, 14, 14, 1), (384, 96, 576, 14, 14, 1), (576, 96, 576, 14, 14, 1), (576, 96, 576, 10, 13, 2),
    (384, 64, 384, 20, 21, 1), (640, 32, 192, 9, 9, 1), (352, 64, 128, 7, 7, 3),
    (192, 64, 384, 14, 14, 1), (320, 96, 192, 7, 9, 2), (64, 32, 64, 12, 12, 1),  # projections without reduction slices
    (576, 96, 576, 14, 14, 1, 2), (384, 64, 384, 15, 13, 2, 2), (192, 32, 192, 9, 9, 1, 2),  # closed by a stride-2 layer
]


def _stride(case):
    return case[6] if len(case) > 6 else 1


def _case(dtype, ch, cm, ce, H, W, B, density, seed, raw=False, stride=1):
    from deltacnn_amd.filter_conversion import convert_filter_out_channels_last, convert_half_filter
    g = torch.Generator().manual_seed(seed)
    mask = rand_mask(g, B, H, W, density)
    rmask = rand_mask(g, B, H, W, 0.5 * density + 0.1)
    x = torch.randn(B, ch, H, W, generator=g).to(dtype)
    r = torch.randn(B, cm, H, W, generator=g)
    # half of the updates are far below the expansion's threshold: they get truncated
    scale = torch.where(torch.rand(B, 1, H, W, generator=g) < 0.5, 1.0, 1e-3)
    x, r = (x * scale).to(dtype), (r * scale).to(dtype)
    wp = (torch.randn(cm, ch, 1, 1, generator=g) / ch ** 0.5).to(dtype)
    we = (torch.randn(ce, cm, 1, 1, generator=g) / cm ** 0.5).to(dtype)
    wd = (torch.randn(ce, 1, 3, 3, generator=g) / 3).to(dtype)
    if dtype == torch.float16:
        fp, fe, fd = convert_half_filter(wp), convert_half_filter(we), convert_half_filter(wd, pixel_wise=True)
    else:
        fp, fe, fd = (convert_filter_out_channels_last(w) for w in (wp, we, wd))
    Ho, Wo = (H - 1) // stride + 1, (W - 1) // stride + 1
    states = [torch.randn(B, ce, h, w, generator=g).to(dtype) * s
              for (s, h, w) in ((1.0, H, W), (0.05, H, W), (1.0, Ho, Wo), (0.05, Ho, Wo))]
    if raw:
        return x, mask, r, rmask, fp.to(DEV), fe.to(DEV), fd.to(DEV), states, (wp, we, wd)
    return x, mask, r, rmask, fp.to(DEV), fe.to(DEV), fd.to(DEV), states


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["float16", "bfloat16"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "-".join(str(v) for v in c))
@pytest.mark.parametrize("density", [0.15, 1.0])
@pytest.mark.parametrize("residual", [False, True], ids=["plain", "residual"])
@pytest.mark.parametrize("act", [1, 2], ids=["relu", "relu6"])
def test_project_expand_equals_separate_calls(lib, dtype, case, density, residual, act):
    from deltacnn_amd import _lib
    from deltacnn_amd import hip_kernels as hk
    ch, cm, ce, H, W, B = case[:6]
    st = _stride(case)
    x, mask, r, rmask, fp, fe, fd, states = _case(dtype, ch, cm, ce, H, W, B, density, 2100 + ch + cm + ce, stride=st)
    pkp, pke = hk.pack_filter(fp, ch, cm, 1), hk.pack_filter(fe, cm, ce, 1)
    dx, dm = cl(poison(x, mask)), cl(mask)
    dr, drm = cl(poison(r, rmask)), cl(rmask)
    gp = hk.conv_geometry((B, ch, H, W), (1, 1), cm, (1, 1), (0, 0), (1, 1), 1)
    gd = hk.conv_geometry((B, ce, H, W), (3, 3), ce, (st, st), (1, 1), (1, 1), ce)
    thr_e, thr_d = 0.9, 0.3
    nan = float("nan")

    def fresh(c, h=H, w=W):
        return (torch.full((B, c, h, w), nan, dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last),
                torch.full((B, 1, h, w), -7, dtype=torch.int32, device=DEV))

    # separate calls
    pe1, te1, pd1, td1 = (cl(t) for t in states)
    y1, ym1 = fresh(cm)
    if residual:
        assert hk.sparse_conv_add(dx, pkp, dm, None, dr, drm, gp, y1, ym1, 1.0, 1.0) is not None
    else:
        hk.sparse_conv(dx, fp, dm, None, (1, 1), (0, 0), (1, 1), 1, cm, packed_filter=pkp, out=y1, out_mask=ym1, geometry=gp)
    e_out, e_mask = hk.sparse_conv_activation(y1, fe, ym1, None, pe1, te1, thr_e, act, 0, (1, 1), (0, 0), (1, 1), 1, ce,
                                              packed_filter=pke)
    kept, reached = int(e_mask.sum()), int(ym1.sum())
    assert reached < 16 or 0 < kept < reached, (kept, reached)  # some kept, some truncated
    d_out, d_mask = hk.sparse_conv_activation(e_out, fd, e_mask, None, pd1, td1, thr_d, 2, 0, (st, st), (1, 1), (1, 1),
                                              ce, ce)
    # the pair launch + the closing depthwise launch
    pe2, te2, pd2, td2 = (cl(t) for t in states)
    y2, ym2 = fresh(cm)
    e2, em2 = fresh(ce)
    out2, om2 = fresh(ce, (H - 1) // st + 1, (W - 1) // st + 1)
    assert hk.sparse_project_expand(dx, dm, pkp, gp, dr if residual else None, drm if residual else None, y2, ym2, pke,
                                    pe2, te2, act, e2, em2, gd, 2, 0)
    assert _lib.load().dc_last_kernels().decode() == "pw_pair_kernel"
    assert torch.equal(ym2, ym1)
    assert_masked_equal(y2, y1.cpu(), ym1.cpu(), "block output")
    assert torch.equal(em2, ym1)  # the expansion's convolution mask, not its keep mask
    assert torch.equal(pe2.cpu(), states[0]), "the open form leaves the accumulated values alone"
    te_open, e_open = te2.clone(), e2.clone()
    assert hk.sparse_expand_depthwise(y2, None, None, pe2, te2, thr_e, act, e2, em2, fd, gd, pd2, td2, thr_d, 2, 0,
                                      out2, om2, opened=True)
    assert _lib.load().dc_last_kernels().decode() == "conv_dw_kernel"
    assert torch.equal(om2, d_mask)
    assert_masked_equal(out2, d_out.cpu(), d_mask.cpu(), "depthwise output")
    if not torch.equal(te1, te2):  # name the elements: per pixel the channels, masks and whether the pair wrote D
        bad = (te1 != te2)
        rows = []
        for b, _, h, w in bad.any(dim=1, keepdim=True).nonzero().tolist():
            cs = bad[b, :, h, w].nonzero().flatten().tolist()
            rows.append(dict(pixel=(b, h, w), channels=cs, mask=int(mask[b, 0, h, w]), rmask=int(rmask[b, 0, h, w]),
                             kept=int(e_mask[b, 0, h, w]), pair_is_initial=bool((te2[b, cs, h, w].cpu() == states[1][b, cs, h, w]).all()),
                             d_unwritten=e2[b, :, h, w].isnan().nonzero().flatten().tolist(),
                             d_unwritten_after_pair=e_open[b, :, h, w].isnan().nonzero().flatten().tolist(),
                             t_initial_after_pair=(te_open[b, :, h, w].cpu() == states[1][b, :, h, w]).nonzero().flatten().tolist(),
                             ptrs={n: hex(t.data_ptr()) for n, t in dict(e2=e2, te2=te2, pe2=pe2, y2=y2, dx=dx, dr=dr, dm=dm,
                                                                          drm=drm, em2=em2, ym2=ym2, pkp=pkp, pke=pke).items()}))
        raise AssertionError(f"expansion truncated state differs in {int(bad.sum())} elements: {rows}")
    assert torch.equal(pe1, pe2) and torch.equal(te1, te2), "expansion state"
    assert torch.equal(pd1, pd2) and torch.equal(td1, td2), "depthwise state"
    assert_masked_equal(e2, e_out.cpu(), e_mask.cpu(), "expansion output on kept pixels")


@pytest.mark.parametrize("case", [CASES[0], CASES[1], CASES[6], CASES[7]], ids=lambda c: "-".join(str(v) for v in c))
@pytest.mark.parametrize("residual", [False, True], ids=["plain", "residual"])
def test_project_expand_against_oracle_chain(lib, case, residual):
    """The pair launch and the closing depthwise launch against the CPU oracle's chain projection
    (+ residual sum) -> expansion -> activation / truncation -> depthwise 3x3 -> activation /
    truncation (fp16).  A convolution output differs from the oracle's in its last bit now and then,
    which can flip a keep decision on the threshold: such pixels are counted and must be rare,
    everything else agrees within 2e-2."""
    from deltacnn_amd import hip_kernels as hk
    from oracle import delta_ops as ops
    dtype = torch.float16
    ch, cm, ce, H, W, B = case[:6]
    x, mask, r, rmask, fp, fe, fd, states, (wp, we, wd) = _case(dtype, ch, cm, ce, H, W, B, 0.4, 2300 + ch + cm + ce, raw=True)
    thr_e, thr_d, act = 0.9, 0.3, 2
    # oracle
    pe, te, pd, td = (t.clone() for t in states)
    y, ym = ops.conv(x, mask, wp)
    if residual:
        y, ym = ops.add(r, rmask, y, ym, None)
    e, em = ops.conv(y, ym, we)
    em = em.clone()
    ops.activate_truncate(e, pe, te, em, thr_e, act, 0)
    d, dm = ops.conv(e, em, wd, None, (1, 1), (1, 1), (1, 1), ce)
    dm = dm.clone()
    ops.activate_truncate(d, pd, td, dm, thr_d, act, 0)
    # library
    pkp, pke = hk.pack_filter(fp, ch, cm, 1), hk.pack_filter(fe, cm, ce, 1)
    gp = hk.conv_geometry((B, ch, H, W), (1, 1), cm, (1, 1), (0, 0), (1, 1), 1)
    gd = hk.conv_geometry((B, ce, H, W), (3, 3), ce, (1, 1), (1, 1), (1, 1), ce)

    def fresh(c):
        return (torch.zeros((B, c, H, W), dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last),
                torch.zeros((B, 1, H, W), dtype=torch.int32, device=DEV))
    pe2, te2, pd2, td2 = (cl(t) for t in states)
    y2, ym2 = fresh(cm)
    e2, em2 = fresh(ce)
    out2, om2 = fresh(ce)
    dr, drm = cl(poison(r, rmask)), cl(rmask)
    assert hk.sparse_project_expand(cl(poison(x, mask)), cl(mask), pkp, gp, dr if residual else None,
                                    drm if residual else None, y2, ym2, pke, pe2, te2, act, e2, em2, gd, act, 0)
    assert hk.sparse_expand_depthwise(y2, None, None, pe2, te2, thr_e, act, e2, em2, fd, gd, pd2, td2, thr_d, act, 0,
                                      out2, om2, opened=True)
    assert torch.equal(ym2.cpu(), ym)  # the block output's mask is the union of the input masks: exact
    both_y = ym != 0
    assert float(torch.where(both_y, (y2.cpu().float() - y.float()).abs(), torch.zeros(())).max()) <= 2e-2
    flips = int((om2.cpu() != dm).sum())
    assert flips <= max(2, dm.numel() // 100), f"{flips} of {dm.numel()} output mask words differ from the oracle's"
    both = (om2.cpu() != 0) & (dm != 0)
    assert int(both.sum()) > 0
    err = float(torch.where(both, (out2.cpu().float() - d.float()).abs(), torch.zeros(())).max())
    if flips == 0:
        assert err <= 2e-2, err
    print(f"project + expand + depthwise vs oracle: {flips} mask words of {dm.numel()} differ, max |diff| {err:.4f}")


def test_project_expand_declines_what_it_cannot_do(lib):
    """Block channels outside multiples of 32 up to 96, projections of more than 20 reduction
    steps, a depthwise layer that cannot finish the expansion (stride 3)
    and fp32: False, nothing launched, nothing touched."""
    from deltacnn_amd import hip_kernels as hk
    dtype = torch.float16
    for (ch, cm, ce, H, W, B, stride, dt) in [(384, 64, 384, 14, 14, 1, 3, dtype), (704, 64, 384, 14, 14, 1, 1, dtype),
                                              (384, 48, 288, 14, 14, 1, 1, dtype), (960, 160, 960, 7, 7, 1, 1, dtype),
                                              (384, 64, 384, 14, 14, 1, 1, torch.float32)]:
        x, mask, r, rmask, fp, fe, fd, states = _case(dtype, ch, cm, ce, H, W, B, 0.5, 2200 + ch)
        pkp, pke = hk.pack_filter(fp, ch, cm, 1), hk.pack_filter(fe, cm, ce, 1)
        gp = hk.conv_geometry((B, ch, H, W), (1, 1), cm, (1, 1), (0, 0), (1, 1), 1)
        gd = hk.conv_geometry((B, ce, H, W), (3, 3), ce, (stride, stride), (1, 1), (1, 1), ce)
        pe, te = cl(states[0]), cl(states[1])
        before = [t.clone() for t in (pe, te)]
        y = torch.zeros(B, cm, H, W, dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
        e = torch.zeros(B, ce, H, W, dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
        ym = torch.zeros(B, 1, H, W, dtype=torch.int32, device=DEV)
        em = torch.zeros_like(ym)
        dx = cl(x).to(dt) if dt != dtype else cl(x)
        assert hk.sparse_project_expand(dx, cl(mask), pkp, gp, None, None, y, ym, pke, pe, te, 2, e, em, gd, 2, 0) is False
        assert all(torch.equal(a, b) for a, b in zip(before, (pe, te)))
        assert not bool(y.any()) and not bool(e.any())
