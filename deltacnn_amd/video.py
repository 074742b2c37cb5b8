"""Seeded synthetic video generators for the benchmark configurations.

All generators return float32 CPU tensors ``[T, 3, H, W]`` with values in [0, 1] and are
deterministic functions of their seed.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def noise_block_video(frames=10, size=64, fraction=0.05, block=8, seed=1234) -> torch.Tensor:
    """Frame 0 is uniform noise; every later frame re-randomises random ``block`` x ``block``
    aligned blocks until ``fraction`` of the pixels has changed."""
    g = torch.Generator().manual_seed(seed)
    cur = torch.rand(3, size, size, generator=g)
    out = [cur.clone()]
    cells = size // block
    n_blocks = max(1, math.ceil(fraction * size * size / (block * block)))
    for _ in range(frames - 1):
        cur = cur.clone()
        for idx in torch.randperm(cells * cells, generator=g)[:n_blocks].tolist():
            y, x = (idx // cells) * block, (idx % cells) * block
            cur[:, y:y + block, x:x + block] = torch.rand(3, block, block, generator=g)
        out.append(cur)
    return torch.stack(out)


def _value_noise(h, w, octaves, g) -> torch.Tensor:
    """Multi-octave smooth noise (bilinear-interpolated random lattices), a Perlin-style texture."""
    img = torch.zeros(3, h, w)
    amp, total = 1.0, 0.0
    for o in range(octaves):
        cells = 4 * 2 ** o
        lattice = torch.rand(1, 3, cells + 1, cells + 1, generator=g)
        img += amp * F.interpolate(lattice, size=(h, w), mode="bicubic", align_corners=True)[0]
        total += amp
        amp *= 0.5
    return (img / total).clamp(0, 1)


def moving_rectangles_video(frames=64, height=224, width=224, n_rect=3, min_size=20, max_size=60,
                            min_speed=1, max_speed=4, noise_sigma=0.01, seed=1236) -> torch.Tensor:
    """Static smooth-noise background, ``n_rect`` textured rectangles moving with wrap-around,
    plus per-frame Gaussian sensor noise."""
    g = torch.Generator().manual_seed(seed)
    bg = _value_noise(height, width, 4, g)
    rects = []
    for _ in range(n_rect):
        rh = int(torch.randint(min_size, max_size + 1, (1,), generator=g))
        rw = int(torch.randint(min_size, max_size + 1, (1,), generator=g))
        y = int(torch.randint(0, height, (1,), generator=g))
        x = int(torch.randint(0, width, (1,), generator=g))
        vy = int(torch.randint(min_speed, max_speed + 1, (1,), generator=g)) * (1 if torch.rand(1, generator=g) < 0.5 else -1)
        vx = int(torch.randint(min_speed, max_speed + 1, (1,), generator=g)) * (1 if torch.rand(1, generator=g) < 0.5 else -1)
        rects.append([y, x, vy, vx, torch.rand(3, rh, rw, generator=g)])
    out = []
    for _ in range(frames):
        frame = bg.clone()
        for r in rects:
            y, x, vy, vx, tex = r
            ys = (torch.arange(tex.shape[1]) + y) % height
            xs = (torch.arange(tex.shape[2]) + x) % width
            frame[:, ys[:, None], xs[None, :]] = tex
            r[0], r[1] = (y + vy) % height, (x + vx) % width
        frame = frame + noise_sigma * torch.randn(3, height, width, generator=g)
        out.append(frame.clamp(0, 1))
    return torch.stack(out)


def controlled_density_video(frames=8, height=224, width=224, density=0.10, block=16, seed=1240
                             ) -> torch.Tensor:
    """Controlled input update density: frame 0 is a smooth-noise image and every later frame
    re-randomises ``block`` x ``block`` aligned blocks covering ``density`` of the pixels on top
    of the previous frame, so exactly that fraction of the input pixels changes by far more than
    any sensible threshold (density 1.0 replaces the whole frame)."""
    g = torch.Generator().manual_seed(seed)
    cur = _value_noise(height, width, 4, g)
    out = [cur.clone()]
    cy, cx = height // block, width // block
    n_blocks = max(1, round(density * cy * cx)) if density < 1.0 else cy * cx
    for _ in range(frames - 1):
        cur = cur.clone()
        if density >= 1.0:
            cur = torch.rand(3, height, width, generator=g)
        else:
            for idx in torch.randperm(cy * cx, generator=g)[:n_blocks].tolist():
                y, x = (idx // cx) * block, (idx % cx) * block
                cur[:, y:y + block, x:x + block] = torch.rand(3, block, block, generator=g)
        out.append(cur)
    return torch.stack(out)
