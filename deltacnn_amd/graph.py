"""Whole-frame HIP graph capture for the delta path.

At batch 1 a frame is ~70 kernels of about two microseconds each, so host launch cost
dominates eager execution.  All shapes of a DeltaCNN frame are static (sparsity only changes
what kernels do inside), so the launches of one frame are recorded once and replayed with a
single graph launch.

An ordinary stream operation between two graph launches (for example copying the next frame
into the graph's input buffer) stalls the replay pipeline for far longer than the copy itself
takes.  :class:`VideoGraph` therefore keeps the frame fetch inside the graph: the clip lives
in device memory and a device-side counter selects the frame, so a replay needs no other
stream work at all.  :class:`FrameGraph` is the general form (one frame handed over per call).
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


class VideoGraph:
    """Replay ``model(frames[t])`` for t = start, start + 1, ... with the frame fetch inside
    the graph.

    ``frames`` is a device tensor ``[T, C, H, W]`` whose frames are NHWC in memory
    (``torch.channels_last``).  One :meth:`step` processes the next ``unroll`` frames, one after
    the other, from a single graph launch (one gather fetches them, one add advances the
    counter), and returns the output of the last one -- or, with ``unroll > 1``, the list of
    all ``unroll`` outputs; the caller must not step past the end of the clip.  ``model`` may be
    any callable on a ``[1, C, H, W]`` tensor (the delta model after its first frame, or a
    dense model).
    """

    def __init__(self, model, frames: torch.Tensor, start: int = 0, unroll: int = 1):
        if not frames.is_contiguous(memory_format=torch.channels_last):
            raise ValueError("frames must be channels_last")
        t, c, h, w = frames.shape
        self.length = t
        self.unroll = unroll
        self._rows = frames.permute(0, 2, 3, 1).reshape(t, h * w * c)  # a view: NHWC rows
        self.index = torch.arange(start, start + unroll, dtype=torch.int64, device=frames.device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(self.graph):
            staged = self._rows.index_select(0, self.index).view(unroll, h, w, c).permute(0, 3, 1, 2)
            outs = [model(staged[i:i + 1]) for i in range(unroll)]
            self.index.add_(unroll)
        self.static_out = outs[0] if unroll == 1 else outs

    def seek(self, t: int) -> None:
        self.index.copy_(torch.arange(t, t + self.unroll, dtype=torch.int64, device=self.index.device))

    @torch.no_grad()
    def step(self):
        self.graph.replay()
        return self.static_out
