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
