"""Whole-frame HIP graph capture for the delta path.

At batch 1 a frame is ~100 kernels of a few microseconds each, so host launch cost dominates.
All shapes of a DeltaCNN frame are static (sparsity only changes what kernels do inside), so
the launches of one frame can be recorded once and replayed with a single graph launch.
"""
from __future__ import annotations

import torch


class FrameGraph:
    """Record ``model(frame)`` for frames after the first and replay it per frame.

    The model must already have processed its first frame eagerly (the first frame takes
    the dense initialisation branches of every layer and allocates the caches).  Capture does
    not execute anything; the recorded frame is only a shape/dtype template.

        fg = FrameGraph(model, frame0_like)
        for frame in video[1:]:
            logits = fg(frame)        # valid until the next call
    """

    def __init__(self, model, like: torch.Tensor):
        self.model = model
        self.static_in = like.clone()
        self.graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(self.graph):
            self.static_out = model(self.static_in)

    @torch.no_grad()
    def __call__(self, frame: torch.Tensor):
        self.static_in.copy_(frame)
        self.graph.replay()
        return self.static_out
