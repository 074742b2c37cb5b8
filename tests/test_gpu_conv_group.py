"""dc_conv_group: independent small 3x3 layers -- the same layer of several parallel branches of a
multi-resolution network -- in ONE launch (+ one for the activations the convolution kernel cannot
finish itself).  Every item is what a call of dc_conv, dc_conv_act or dc_conv_add would be given;
everything that call leaves behind (output, mask, the activation's or the sum's cached state) has
to come out bit for bit."""
import pytest
import torch

from util import DEV, assert_masked_equal, cl, poison, rand_mask

pytestmark = pytest.mark.gpu

# items: (kind, Cin, Cout, H, W, batch, stride); kinds: conv, act (activation/truncation), add, addact: 3x3;
# pw: a plain 1x1 convolution
GROUPS = {
    "hrnet-exchange-pw": [("pw", 64, 32, 32, 32, 1, 1), ("pw", 128, 32, 16, 16, 1, 1), ("pw", 256, 32, 8, 8, 1, 1),
                          ("pw", 128, 64, 16, 16, 1, 1), ("pw", 256, 64, 8, 8, 1, 1), ("pw", 256, 128, 8, 8, 1, 1)],
    "pw-ragged": [("pw", 8, 4, 5, 7, 3, 1), ("pw", 40, 20, 13, 9, 1, 1), ("pw", 320, 72, 3, 3, 2, 1), ("pw", 32, 200, 6, 6, 1, 1)],
    "hrnet4-act": [("act", 32, 32, 64, 64, 1, 1), ("act", 64, 64, 32, 32, 1, 1), ("act", 128, 128, 16, 16, 1, 1),
                   ("act", 256, 256, 8, 8, 1, 1)],
    "hrnet4-addact": [("addact", 32, 32, 64, 64, 1, 1), ("addact", 64, 64, 32, 32, 1, 1),
                      ("addact", 128, 128, 16, 16, 1, 1), ("addact", 256, 256, 8, 8, 1, 1)],
    "hrnet3-act": [("act", 32, 32, 64, 64, 1, 1), ("act", 64, 64, 32, 32, 1, 1), ("act", 128, 128, 16, 16, 1, 1)],
    "hrnet2-add": [("add", 32, 32, 64, 64, 1, 1), ("add", 64, 64, 32, 32, 1, 1)],
    "mixed-ragged": [("conv", 40, 24, 13, 10, 2, 1), ("act", 8, 16, 21, 19, 1, 2), ("addact", 96, 72, 9, 11, 1, 1),
                     ("act", 72, 40, 7, 30, 1, 1), ("add", 16, 8, 5, 5, 3, 2)],
    "one-late-activation": [("act", 32, 32, 20, 20, 1, 1), ("act", 64, 48, 10, 10, 1, 1)],
    "eight": [("act", 16, 16, 12, 12, 1, 1), ("conv", 24, 16, 6, 6, 1, 1), ("add", 32, 32, 8, 8, 1, 1),
              ("act", 64, 64, 8, 8, 2, 1), ("addact", 8, 8, 31, 5, 1, 1), ("conv", 128, 16, 4, 4, 1, 1),
              ("act", 48, 80, 6, 9, 1, 2), ("act", 256, 64, 4, 4, 1, 1)],
}


def _filter(dtype, w):
    from deltacnn_amd.filter_conversion import convert_filter_out_channels_last, convert_half_filter
    return (convert_half_filter(w) if dtype == torch.float16 else convert_filter_out_channels_last(w)).to(DEV)


def _item(dtype, spec, density, gen):
    """Inputs, filters and states of one item on the host / device, twice (for the two paths)."""
    from deltacnn_amd import hip_kernels as hk
    kind, cin, cout, H, W, B, stride = spec
    Ho, Wo = (H - 1) // stride + 1, (W - 1) // stride + 1
    mask = rand_mask(gen, B, H, W, density)
    x = torch.randn(B, cin, H, W, generator=gen)
    # half of the updates are small: some outputs stay below the activation's threshold
    x = (x * torch.where(torch.rand(B, 1, H, W, generator=gen) < 0.5, 1.0, 2e-2)).to(dtype)
    k = 1 if kind == "pw" else 3
    w = (torch.randn(cout, cin, k, k, generator=gen) / (k * cin ** 0.5)).to(dtype)
    f = _filter(dtype, w)
    it = dict(kind=kind, x=cl(poison(x, mask)), mask=cl(mask), filter=f, packed=hk.pack_filter(f, cin, cout, 1),
              geometry=hk.conv_geometry((B, cin, H, W), (k, k), cout, (stride, stride), (k // 2, k // 2), (1, 1), 1),
              shape=(B, cout, Ho, Wo), stride=stride, cout=cout, host_mask=mask)
    if kind in ("add", "addact"):
        rmask = rand_mask(gen, B, Ho, Wo, 0.5 * density + 0.1)
        r = torch.randn(B, cout, Ho, Wo, generator=gen).to(dtype)
        it.update(res=cl(poison(r, rmask)), rmask=cl(rmask))
    it["states"] = [torch.randn(B, cout, Ho, Wo, generator=gen).to(dtype) * s for s in (1.0, 0.05)]
    return it


def _buffers(it, dtype):
    B, C, H, W = it["shape"]
    out = torch.full((B, C, H, W), float("nan"), dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
    return out, torch.full((B, 1, H, W), -7, dtype=torch.int32, device=DEV)


THR = 0.4


def _separate(hk, it, dtype, act_id):
    """The item through the library's single-layer calls: (out, out_mask, states)."""
    prev, trunc = (cl(t) for t in it["states"])
    s = (it["stride"], it["stride"])
    if it["kind"] == "pw":
        out, om = hk.sparse_conv(it["x"], it["filter"], it["mask"], None, s, (0, 0), (1, 1), 1, it["cout"],
                                 create_out_mask=True, packed_filter=it["packed"])
    elif it["kind"] == "conv":
        out, om = hk.sparse_conv(it["x"], it["filter"], it["mask"], None, s, (1, 1), (1, 1), 1, it["cout"],
                                 create_out_mask=True, packed_filter=it["packed"])
    elif it["kind"] == "act":
        out, om = hk.sparse_conv_activation(it["x"], it["filter"], it["mask"], None, prev, trunc, THR, act_id, 0, s,
                                            (1, 1), (1, 1), 1, it["cout"], packed_filter=it["packed"])
    else:
        out, om = _buffers(it, dtype)
        got = hk.sparse_conv_add(it["x"], it["packed"], it["mask"], None, it["res"], it["rmask"], it["geometry"], out, om,
                                 0.75, 1.25, prev if it["kind"] == "addact" else None, act_id if it["kind"] == "addact" else 0)
        assert got is not None
    return out, om, prev, trunc


def _group_items(items, dtype, act_id):
    rows, outs = [], []
    for it in items:
        out, om = _buffers(it, dtype)
        prev, trunc = (cl(t) for t in it["states"])
        row = dict(x=it["x"], mask=it["mask"], packed_filter=it["packed"], geometry=it["geometry"], out=out, out_mask=om)
        if it["kind"] == "act":
            row["activation"] = (prev, trunc, THR, act_id, 0)
        elif it["kind"] in ("add", "addact"):
            with_act = it["kind"] == "addact"
            row["residual"] = (it["res"], it["rmask"], 0.75, 1.25, prev if with_act else None, act_id if with_act else 0)
        rows.append(row)
        outs.append((out, om, prev, trunc))
    return rows, outs


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["float16", "bfloat16"])
@pytest.mark.parametrize("group", sorted(GROUPS))
@pytest.mark.parametrize("density", [0.1, 1.0])
@pytest.mark.parametrize("act_id", [1, 3], ids=["relu", "leaky"])
def test_conv_group_equals_separate_calls(lib, dtype, group, density, act_id):
    from deltacnn_amd import _lib
    from deltacnn_amd import hip_kernels as hk
    gen = torch.Generator().manual_seed(3100 + len(group) + int(density * 10))
    items = [_item(dtype, spec, density, gen) for spec in GROUPS[group]]
    want = [_separate(hk, it, dtype, act_id) for it in items]
    rows, got = _group_items(items, dtype, act_id)
    assert hk.sparse_conv_group(rows) is True
    kernels = _lib.load().dc_last_kernels().decode().split("+")
    if GROUPS[group][0][0] == "pw":
        assert kernels == ["pw_group_kernel"]
    else:
        assert kernels[0] == "conv_patch_group_kernel" and len(kernels) <= 2
    if len(kernels) == 2:
        assert kernels[1] in ("act_trunc_group_kernel", "act_trunc_vec_kernel")
    for spec, (o1, m1, p1, t1), (o2, m2, p2, t2) in zip(GROUPS[group], want, got):
        what = "-".join(str(v) for v in spec)
        assert torch.equal(m1, m2), f"{what}: mask"
        assert_masked_equal(o2, o1.cpu(), m1.cpu(), f"{what}: output")
        assert torch.equal(p1, p2), f"{what}: accumulated values"
        assert torch.equal(t1, t2), f"{what}: truncated values"


def test_conv_group_declines_what_it_cannot_do(lib):
    """A pointwise layer, a layer beyond the 4x4-patch kernel's range, a single item, two kinds of
    activation in the second launch, items sharing an output: False, nothing launched or touched."""
    from deltacnn_amd import hip_kernels as hk
    dtype = torch.float16
    gen = torch.Generator().manual_seed(3200)
    small = [_item(dtype, spec, 0.5, gen) for spec in GROUPS["hrnet3-act"]]
    big = _item(dtype, ("act", 64, 64, 136, 240, 1, 1), 0.2, gen)

    def untouched(outs):
        return all(bool(o.isnan().all()) and bool((m == -7).all()) for o, m, _, _ in outs)

    rows, outs = _group_items(small[:1], dtype, 1)
    assert hk.sparse_conv_group(rows) is False and untouched(outs)
    rows, outs = _group_items(small[:2] + [big], dtype, 1)
    assert hk.sparse_conv_group(rows) is False and untouched(outs)
    # 1x1: the pointwise kernels' layer
    rows, outs = _group_items(small[:2], dtype, 1)
    pw = hk.conv_geometry((1, 32, 64, 64), (1, 1), 32, (1, 1), (0, 0), (1, 1), 1)
    rows[0]["geometry"] = pw
    assert hk.sparse_conv_group(rows) is False and untouched(outs)
    # two activations that both need the second launch (64 and 128 channels), of different kinds
    rows, outs = _group_items(small, dtype, 1)
    prev, trunc, thr, _, mode = rows[2]["activation"]
    rows[2]["activation"] = (prev, trunc, thr, 3, mode)
    assert hk.sparse_conv_group(rows) is False and untouched(outs)
    # one output buffer for two items
    rows, outs = _group_items(small[:2] + small[:1], dtype, 1)
    rows[2]["out"] = rows[0]["out"]
    assert hk.sparse_conv_group(rows) is False and untouched(outs)
    # 1x1 and 3x3 layers together; a 1x1 layer with an activation
    pws = [_item(dtype, spec, 0.5, gen) for spec in GROUPS["hrnet-exchange-pw"][:2]]
    rows, outs = _group_items(small[:1] + pws[:1], dtype, 1)
    assert hk.sparse_conv_group(rows) is False and untouched(outs)
    rows, outs = _group_items(pws, dtype, 1)
    rows[1]["activation"] = (outs[1][2], outs[1][3], THR, 1, 0)
    assert hk.sparse_conv_group(rows) is False and untouched(outs)
    # fp32 has no such form
    rows, outs = _group_items(small[:2], dtype, 1)
    for r in rows:
        r["x"] = r["x"].float()
    assert hk.sparse_conv_group(rows) is False and untouched(outs)


def test_hrnet_branches_side_by_side_change_nothing(lib):
    """HRNet-W32 at 128x128 (1 / 1 / 2 exchange modules), 5 frames: the model that launches the
    same layer of all branches -- and the strided convolutions of an exchange level by level --
    together against the model that runs path after path: heat maps and every layer's cached
    state equal bit for bit; and the groups are really taken."""
    from deltacnn_amd import hip_kernels as hk
    from deltacnn_amd import sparse_layers as SL
    from deltacnn_amd.networks import DenseLayers, HRNet, fold_data_statistics
    from deltacnn_amd.video import moving_rectangles_video
    video = moving_rectangles_video(frames=5, height=128, width=128, n_rect=2, min_size=20, max_size=60)
    torch.manual_seed(0)
    dense = HRNet(DenseLayers, modules=(1, 1, 2)).eval().to(DEV, memory_format=torch.channels_last)
    with torch.no_grad():
        fold_data_statistics(dense, cl(video[:2]))
    state = {k: v.clone() for k, v in dense.state_dict().items()}
    SL.DCThreshold.t_default = 0.05

    def build():
        m = HRNet(SL, modules=(1, 1, 2)).eval()
        m.load_state_dict(state)
        m = m.to(DEV, memory_format=torch.channels_last).half()
        m.process_filters()
        return m
    grouped, plain = build(), build()
    calls = []
    original = hk.sparse_conv_group

    def counted(items):
        done = original(items)
        calls.append((done, len(items)))
        return done
    hk.sparse_conv_group = counted
    sums = []
    original_sums = hk.sparse_add_group

    def counted_sums(items):
        done = original_sums(items)
        sums.append((done, len(items)))
        return done
    hk.sparse_add_group = counted_sums
    try:
        with torch.no_grad():
            for t in range(video.shape[0]):
                frame = cl(video[t:t + 1].half())
                SL.DCConv2d.fuse_groups = True
                got = grouped(frame).clone()
                SL.DCConv2d.fuse_groups = False
                want = plain(frame)
                assert torch.equal(got, want), f"frame {t}"
    finally:
        SL.DCConv2d.fuse_groups = True
        hk.sparse_conv_group = original
        hk.sparse_add_group = original_sums
    gm, pm = dict(grouped.named_modules()), dict(plain.named_modules())
    n = 0
    for name, mod in gm.items():
        for attr in ("prev_out", "out_truncated"):
            a, b = getattr(mod, attr, None), getattr(pm[name], attr, None)
            if isinstance(a, torch.Tensor):
                assert torch.equal(a, b), f"{name}.{attr}"
                n += 1
    assert n > 100
    # on every frame after the first: 4 modules x 4 blocks x (conv + activation, conv + sum); of the
    # exchanges' strided convolutions one group of 2 on three resolutions, 4 + 2 on four; and the 1x1
    # convolutions of each exchange but the first (which has one) as one group of 3, 6, 3; and the two
    # sum-carrying strided convolutions of the first level on four resolutions
    assert len(calls) == (4 * 4 * 2 + 3 + 3 + 1) * (video.shape[0] - 1) and all(done for done, _ in calls), calls[:8]
    assert {k for _, k in calls} == {2, 3, 4, 6}
    # the sums of an exchange level by level: 2 on two resolutions, 2 + 3 on three, 2 + 3 + 4 on four
    assert len(sums) == 6 * (video.shape[0] - 1) and all(done for done, _ in sums), sums[:8]
    assert sorted(k for _, k in sums[:6]) == [2, 2, 2, 3, 3, 4]
