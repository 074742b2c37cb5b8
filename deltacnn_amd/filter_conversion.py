"""Weight layouts of the delta kernels (counterpart of src/deltacnn/filter_conversion.py).

``process_filters()`` stores weights in these layouts so that checkpoints processed by
either implementation are interchangeable:

* fp32 conv      ``W_dc[ci, ky, kx, co] = W_torch[co, ci, ky, kx]``   (filter_conversion.py:11)
* fp32 deconv    ``W_dc[ci, ky, kx, co] = W_torch[ci, co, ky, kx]``   (filter_conversion.py:10)
* fp16 depthwise the fp32 layout cast to half                            (filter_conversion.py:31-32)
* fp16 otherwise Cin and Cout padded to even with zeros, then every 2x2 block of
  (input pair, output pair) is swizzled so that ``W[ci, co]`` lives at row
  ``ci ^ (co & 1)``                                                     (filter_conversion.py:26-37)
* bfloat16       (no counterpart in the reference) the fp32 layouts in bfloat16: no padding, no
  swizzle -- ``convert_filter_out_channels_last`` on the bfloat16 weights
"""
from __future__ import annotations

import torch


def convert_filter_out_channels_last(filter: torch.Tensor, transposed: bool = False) -> torch.Tensor:
    if transposed:
        return filter.permute(0, 2, 3, 1).contiguous()
    return filter.permute(1, 2, 3, 0).contiguous()


def convert_half_filter(x: torch.Tensor, pixel_wise: bool = False, transposed: bool = False) -> torch.Tensor:
    w = convert_filter_out_channels_last(x, transposed).half()  # [Cin, Kh, Kw, Cout]
    if pixel_wise:
        return w
    ci, kh, kw, co = w.shape
    out = torch.zeros((ci + ci % 2, kh, kw, co + co % 2), device=w.device, dtype=torch.half)
    cols = torch.arange(co, device=w.device)[None, :].expand(ci, co)
    rows = torch.arange(ci, device=w.device)[:, None] ^ (cols & 1)
    out.permute(0, 3, 1, 2)[rows, cols] = w.permute(0, 3, 1, 2)
    return out


def restore_half_filter(r: torch.Tensor, c_in: int, c_out: int) -> torch.Tensor:
    """Inverse of the swizzle: ``[Cin, Kh, Kw, Cout]`` unpadded, unswizzled."""
    cols = torch.arange(c_out, device=r.device)[None, :].expand(c_in, c_out)
    rows = torch.arange(c_in, device=r.device)[:, None] ^ (cols & 1)
    return r.permute(0, 3, 1, 2)[rows, cols].permute(0, 2, 3, 1).contiguous()
