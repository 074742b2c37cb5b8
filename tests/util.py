"""Helpers shared by the parity tests: seeded inputs, host <-> device layout, comparisons."""
import torch

DEV = "cuda"


def cl(t: torch.Tensor) -> torch.Tensor:
    """Host tensor -> GPU, NHWC memory."""
    if t.dim() == 4 and t.dtype != torch.int32:
        return t.to(DEV).contiguous(memory_format=torch.channels_last)
    return t.to(DEV).contiguous()


def rand_mask(gen, b, h, w, density):
    return (torch.rand(b, 1, h, w, generator=gen) < density).to(torch.int32)


def poison(x: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """NaN at inactive pixels: a kernel that reads them cannot pass."""
    return torch.where(mask != 0, x, torch.full_like(x, float("nan")))


def assert_masked_equal(got, want, mask, what=""):
    m = (mask != 0).expand_as(want)
    g, w = got.cpu()[m], want[m]
    bad = ~((g == w) | (g.isnan() & w.isnan()))
    assert not bad.any(), f"{what}: {int(bad.sum())} of {g.numel()} active values differ; " \
                          f"max |diff| {float((g.float() - w.float()).abs().max())}"


def assert_masked_close(got, want, mask, rtol, atol, what=""):
    m = (mask != 0).expand_as(want)
    g, w = got.cpu().float()[m], want.float()[m]
    err = (g - w).abs()
    lim = atol + rtol * w.abs()
    assert bool((err <= lim).all()), f"{what}: max err {float(err.max())} (limit {float(lim.min())}..)"


def packed_form_exists(dtype, c_in, c_out, kernel, groups=1, transposed=False) -> bool:
    """Whether dc_pack_filter has a form for this filter (include/deltacnn_hip.h): a 16-bit type
    (fp16 or bfloat16), one group, and either input channels in multiples of 8 or a stem
    (Cin <= 4, window up to 8 x 8, Cout <= 64 and a multiple of 4, not transposed).
    tests/test_host_abi.py checks this rule against dc_packed_filter_bytes, so parametrisations
    can be built without the library."""
    kh, kw = (kernel, kernel) if isinstance(kernel, int) else kernel
    if dtype not in (torch.float16, torch.bfloat16) or groups != 1:
        return False
    if c_in % 8 == 0 and c_in >= 8:
        return True
    return not transposed and c_in <= 4 and kh <= 8 and kw <= 8 and c_out % 4 == 0 and c_out <= 64
