"""dc_add_group: independent sums of delta tensors -- those of one level of a multi-resolution
exchange, plain or with the second operand read through nearest upsampling -- in ONE launch.
Output, mask and accumulated sum of every item have to equal those of dc_add / dc_add_upsampled
bit for bit."""
import pytest
import torch

from util import DEV, assert_masked_equal, cl, poison, rand_mask

pytestmark = pytest.mark.gpu

# items: (C, H, W, batch, scale of the second operand, activation id or 0)
GROUPS = {
    "hrnet-level3": [(32, 64, 64, 1, 8, 1), (64, 32, 32, 1, 4, 1), (128, 16, 16, 1, 2, 1), (256, 8, 8, 1, 1, 1)],
    "hrnet-level1": [(32, 64, 64, 1, 2, 0), (64, 32, 32, 1, 1, 0)],
    "ragged": [(8, 6, 10, 3, 2, 3), (40, 7, 5, 1, 1, 0), (1024, 3, 3, 2, 3, 2), (72, 12, 20, 1, 4, 0), (16, 9, 9, 2, 1, 5)],
    "eight": [(8 * (k + 1), 4 + k, 8, 1, 1 if k % 2 else 2, k % 4) for k in range(8)],
}


def _item(dtype, spec, density, gen):
    C, H, W, B, S, act = spec
    if S > 1:
        H, W = H // S * S + (S if H % S else 0), W // S * S + (S if W % S else 0)
    ma, mb = rand_mask(gen, B, H, W, density), rand_mask(gen, B, H // S, W // S, 0.5 * density + 0.2)
    a = torch.randn(B, C, H, W, generator=gen).to(dtype)
    b = torch.randn(B, C, H // S, W // S, generator=gen).to(dtype)
    prev = torch.randn(B, C, H, W, generator=gen).to(dtype)
    return dict(a=cl(poison(a, ma)), b=cl(poison(b, mb)), ma=cl(ma), mb=cl(mb), prev=prev, scale=S, act=act,
                shape=(B, C, H, W))


def _buffers(it, dtype):
    B, C, H, W = it["shape"]
    out = torch.full((B, C, H, W), float("nan"), dtype=dtype, device=DEV).contiguous(memory_format=torch.channels_last)
    return out, torch.full((B, 1, H, W), -7, dtype=torch.int32, device=DEV), cl(it["prev"]) if it["act"] > 0 else None


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["float16", "bfloat16"])
@pytest.mark.parametrize("group", sorted(GROUPS))
@pytest.mark.parametrize("density", [0.1, 1.0])
def test_add_group_equals_separate_calls(lib, dtype, group, density):
    from deltacnn_amd import _lib
    from deltacnn_amd import hip_kernels as hk
    gen = torch.Generator().manual_seed(3300 + len(group) + int(density * 10))
    items = [_item(dtype, spec, density, gen) for spec in GROUPS[group]]
    want, rows, got = [], [], []
    for it in items:
        out, mo, prev = _buffers(it, dtype)
        if it["scale"] == 1:
            hk.sparse_add_tensors(it["a"], it["b"], prev, out, it["ma"], it["mb"], mo, 0.75, 1.25, it["act"], False)
        else:
            hk.sparse_add_upsampled(it["a"], it["b"], prev, out, it["ma"], it["mb"], mo, 0.75, 1.25, it["act"], it["scale"])
        want.append((out, mo, prev))
        out, mo, prev = _buffers(it, dtype)
        rows.append((it["a"], it["b"], prev, out, it["ma"], it["mb"], mo, 0.75, 1.25, it["act"], it["scale"]))
        got.append((out, mo, prev))
    assert hk.sparse_add_group(rows) is True
    assert _lib.load().dc_last_kernels().decode() == "add_group_kernel"
    for spec, (o1, m1, p1), (o2, m2, p2) in zip(GROUPS[group], want, got):
        what = "-".join(str(v) for v in spec)
        assert torch.equal(m1, m2), f"{what}: mask"
        assert_masked_equal(o2, o1.cpu(), m1.cpu(), f"{what}: output")
        if p1 is not None:
            assert torch.equal(p1, p2), f"{what}: accumulated sum"


def test_add_group_declines_what_it_cannot_do(lib):
    """A single sum, channel counts off the vector size, fp32, two sums writing one buffer: False,
    nothing launched or touched."""
    from deltacnn_amd import hip_kernels as hk
    dtype = torch.float16
    gen = torch.Generator().manual_seed(3400)

    def rows_of(specs, dt=dtype):
        rows, outs = [], []
        for spec in specs:
            it = _item(dt, spec, 0.5, gen)
            out, mo, prev = _buffers(it, dt)
            rows.append((it["a"], it["b"], prev, out, it["ma"], it["mb"], mo, 1.0, 1.0, it["act"], it["scale"]))
            outs.append((out, mo))
        return rows, outs

    def untouched(outs):
        return all(bool(o.isnan().all()) and bool((m == -7).all()) for o, m in outs)

    rows, outs = rows_of([(32, 8, 8, 1, 1, 0)])
    assert hk.sparse_add_group(rows) is False and untouched(outs)
    rows, outs = rows_of([(32, 8, 8, 1, 1, 0), (12, 8, 8, 1, 2, 0)])
    assert hk.sparse_add_group(rows) is False and untouched(outs)
    rows, outs = rows_of([(32, 8, 8, 1, 1, 0), (16, 8, 8, 1, 2, 0)], torch.float32)
    assert hk.sparse_add_group(rows) is False and untouched(outs)
    rows, outs = rows_of([(32, 8, 8, 1, 1, 0), (32, 8, 8, 1, 1, 0)])
    rows[1] = rows[1][:3] + (rows[0][3],) + rows[1][4:]
    assert hk.sparse_add_group(rows) is False and untouched(outs)
