#!/usr/bin/env python3
"""Headline benchmark: frames/sec of the delta path on MobileNetV2 224x224 (fp16, batch 1, BN
folded) at a controlled input update density, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--density 0.10] [--mode graph|eager]

A step is one video frame through the whole network (sparsify -> 52 delta convolutions with
activation/truncation -> residual adds -> global average pooling -> densify -> classifier).
All frames are resident in HBM before the timed region.  The JSON line is printed as soon as the
headline is known and again, enriched, after each group of sections (the last line printed is
the result; a section that fails is named under "errors" and the run goes on).  It holds
  value            delta-path frames/sec at the requested density (default 10 %)
  dense_gpu        the same model dense (plain PyTorch / MIOpen) on the same GPU, eager and
                   graph-replayed, and the speed-up over the faster of the two
  sweep            frames/sec at 1/5/10/25/50/100 % input update density
  kernels          per HIP kernel: launches per frame, device time per launch, algorithmic
                   bytes per launch, GB/s and TFLOP/s of one traced frame
  roofline         the kernel with the largest share of the frame time
  micro            single-layer sweeps on a 64x64 map (3x3 256->256, 1x1 256->1024, depthwise
                   C=512, each + ReLU/truncation) over the update densities
  scaled           the memory-bound operators at 512x512, batch 8 (working set beyond the caches)
  cpu_baseline     the CPU oracle of the delta path timed on this host's cores (bounded sample)
  networks         MobileNetV2 on the 64-frame moving-rectangles clip, HRNet-W32 at 256x256 and
                   DLA-34/CenterNet at 544x960: frames/sec, the dense model on the same GPU,
                   launches per frame, mean update density, dominant kernel and its roofline fraction
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
THRESHOLD = 0.05
SWEEP = [0.01, 0.05, 0.10, 0.25, 0.50, 1.00]


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_models(frames_for_stats):
    """Dense fp16 model with data-derived scale + the HIP delta model with the same weights."""
    import torch
    from deltacnn_amd import sparse_layers as SL
    from deltacnn_amd.networks import DenseLayers, MobileNetV2, fold_data_statistics

    torch.manual_seed(0)
    dense = MobileNetV2(DenseLayers).eval()
    dense = dense.to("cuda", memory_format=torch.channels_last)
    with torch.no_grad():
        fold_data_statistics(dense, frames_for_stats.float())
    state = {k: v.clone() for k, v in dense.state_dict().items()}
    dense = dense.half()
    SL.DCThreshold.t_default = THRESHOLD
    delta = MobileNetV2(SL).eval()
    delta.load_state_dict(state)
    delta = delta.to("cuda", memory_format=torch.channels_last).half()
    delta.process_filters()
    return dense, delta, state


def gpu_frames(video):
    import torch
    return video.to("cuda").half().contiguous(memory_format=torch.channels_last)


def time_steps(step, warmup, steps):
    """`warmup` untimed calls of step(), then exactly `steps` timed ones between two syncs."""
    import torch
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


UNROLL = 16  # frames per graph launch (processed one after the other)


def launch_plan(steps, warmup, unroll=UNROLL):
    """How `warmup` untimed and EXACTLY `steps` timed frames are cut into graph launches.

    The frames of one launch are processed strictly one after the other, so the cut changes no
    result, only how often the host launches.  `steps` is split into steps // unroll launches
    of a graph that holds `unroll` frames plus, when that leaves a remainder, one launch of a
    second graph that holds the `tail` remaining frames.  Warm-up runs ceil(warmup / unroll)
    launches of the first graph and one launch of the tail graph, so both have run before
    the clock starts.  Pure arithmetic (no GPU), returned as a dict:
      unroll, tail, timed_main, warm_main, warm_tail   launches as described
      warm_frames      frames the warm-up consumes (>= warmup)
      frames_after_start   frames the clip must hold from the first graph frame on
    """
    if steps < 1 or warmup < 0:
        raise ValueError("steps must be >= 1 and warmup >= 0")
    unroll = max(1, min(unroll, steps))
    tail = steps % unroll
    warm_main = -(-warmup // unroll)
    warm_tail = 1 if tail else 0
    warm_frames = warm_main * unroll + warm_tail * tail
    return {"unroll": unroll, "tail": tail, "timed_main": steps // unroll, "warm_main": warm_main,
            "warm_tail": warm_tail, "warm_frames": warm_frames, "frames_after_start": warm_frames + steps}


def clip_frames(steps, warmup, lead=2):
    """Length of the clip the headline run needs: `lead` eager frames (the dense first frame and
    one eager delta frame), the warm-up and timed frames of launch_plan, one spare."""
    return lead + launch_plan(steps, warmup)["frames_after_start"] + 1


def time_graph(model, frames, start, warmup, steps):
    """Seconds per frame of model(frame) on consecutive frames of the clip from frame `start`
    on, replayed from HIP graphs cut as launch_plan says (exactly `steps` timed frames after
    at least `warmup` untimed ones)."""
    import torch
    from deltacnn_amd.graph import VideoGraph
    plan = launch_plan(steps, warmup)
    if start + plan["frames_after_start"] > frames.shape[0]:
        raise ValueError(f"clip of {frames.shape[0]} frames is too short: start {start} + "
                         f"{plan['frames_after_start']} frames needed")
    main = VideoGraph(model, frames, start=start, unroll=plan["unroll"])
    tail = VideoGraph(model, frames, start=start, unroll=plan["tail"]) if plan["tail"] else None
    for _ in range(plan["warm_main"]):
        main.step()
    pos = start + plan["warm_main"] * plan["unroll"]
    if tail is not None:
        tail.seek(pos)
        tail.step()
        pos += plan["tail"]
        tail.seek(pos + plan["timed_main"] * plan["unroll"])
    main.seek(pos)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(plan["timed_main"]):
        main.step()
    if tail is not None:
        tail.step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def run_delta(delta, frames, warmup, steps, mode):
    """frames: [T,3,H,W] on the GPU with T >= warmup + steps + 2.  Frame 0 initialises the
    caches (dense first frame), frame 1 runs eagerly (lazy weight packing, buffers); the timed
    region covers frames 2+warmup .. 2+warmup+steps-1."""
    import torch
    from deltacnn_amd.graph import VideoGraph
    delta.reset_layers()
    with torch.no_grad():
        delta(frames[0:1])
        delta(frames[1:2])
        if mode == "graph":
            return time_graph(delta, frames, 2, warmup, steps)
        it = iter(range(2, frames.shape[0]))
        return time_steps(lambda: delta(frames[next(it):][:1]), warmup, steps)


def run_dense(dense, frames, warmup, steps):
    """The dense model on the same frames: eager, and graph-replayed with the same in-graph
    frame fetch as the delta path."""
    import torch
    from deltacnn_amd.graph import VideoGraph
    with torch.no_grad():
        dense(frames[0:1])
        it = iter(range(1, frames.shape[0]))
        eager = time_steps(lambda: dense(frames[next(it):][:1]), warmup, steps)
        graph = time_graph(dense, frames, 1, warmup, steps)
    return eager, graph


STREAM_UNROLL = 4   # frames per graph launch of the batched-streams runs
STREAM_STRIDE = 2   # clip offset between neighbouring streams, in frames


def streams_clip_frames(batch, steps, warmup, unroll=STREAM_UNROLL, stride=STREAM_STRIDE):
    """Frames a clip must hold for streams_bench: the last stream starts (batch-1)*stride frames
    in, then 2 eager frames, ceil(warmup/unroll)*unroll warm-up and `steps` timed frames."""
    return (batch - 1) * stride + 2 + -(-warmup // unroll) * unroll + (steps // unroll) * unroll + 1


def streams_bench(delta, dense, batch=8, steps=64, warmup=16, density=0.10, with_dense=True):
    """Supplementary: `batch` independent video streams (one clip of its own, read at different
    offsets) through ONE model instance as a batch, i.e. the same kernels on maps `batch` times
    larger.  Every stream keeps its own caches (they are the batch dimension of the layers'
    state).  Returns total frames/s for the delta path and for the dense model, both from HIP
    graphs."""
    import torch
    from deltacnn_amd.video import controlled_density_video
    unroll = STREAM_UNROLL
    steps = max(unroll, steps - steps % unroll)
    frames = gpu_frames(controlled_density_video(frames=streams_clip_frames(batch, steps, warmup), density=density))
    t, c, h, w = frames.shape
    rows = frames.permute(0, 2, 3, 1).reshape(t, h * w * c)
    offsets = torch.arange(batch, device=frames.device) * STREAM_STRIDE

    def fetch(index):
        return rows.index_select(0, index).view(-1, batch, h, w, c).permute(0, 1, 4, 2, 3)

    def timed(model, start):
        index = ((start + torch.arange(unroll, device=frames.device))[:, None] + offsets[None, :]).reshape(-1)
        graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(graph):
            staged = fetch(index)
            outs = [model(staged[i]) for i in range(unroll)]
            index.add_(unroll)
        return time_steps(graph.replay, -(-warmup // unroll), steps // unroll) / unroll

    with torch.no_grad():
        delta.reset_layers()
        for i in range(2):  # dense first frame of every stream, one eager delta frame
            delta(fetch(offsets + i)[0])
        d = timed(delta, 2)
        delta.reset_layers()
        out = {"streams": batch, "update_density": density, "delta_fps_total": round(batch / d, 1),
               "ms_per_step": round(d * 1e3, 4), "steps": steps}
        if with_dense:
            dense(fetch(offsets)[0])
            out["dense_graph_fps_total"] = round(batch / timed(dense, 2), 1)
    return out


def streams_profile(delta, batch, density, isolated=True):
    """For profiling runs (`--only-streams N`): the graph-replayed step of N streams as a batch, and
    beside it the sum of the same step's library calls each replayed on its own -- the two figures
    whose difference is what a kernel loses by running behind another kernel's output."""
    import torch
    from deltacnn_amd.video import controlled_density_video
    out = streams_bench(delta, None, batch=batch, steps=64, warmup=16, density=density, with_dense=False)
    if not isolated:
        return out
    clip = gpu_frames(controlled_density_video(frames=(batch - 1) * STREAM_STRIDE + 5, density=density))
    steps = torch.cat([clip[torch.arange(batch) * STREAM_STRIDE + i] for i in range(4)]).contiguous(
        memory_format=torch.channels_last)
    agg, rows = trace_kernels(delta, steps, batch=batch)
    delta.reset_layers()
    out["library_launches_per_step"] = len(rows)
    out["isolated_replays_sum_ms"] = round(sum(r["ms"] for r in rows), 4)
    out["kernels_isolated"] = {k: {"launches_per_step": a["launches"], "us_per_launch": round(a["us_per_launch"], 3)}
                               for k, a in sorted(agg.items(), key=lambda kv: -kv[1]["ms"])}
    return out


def trace_kernels(delta, frames, batch=1):
    """Device time per call and algorithmic bytes / flops of every library call of one delta
    frame (of `batch` streams: frames[i * batch:(i + 1) * batch] is step i).  The calls are recorded
    during an eager pass; each is then timed on the device by replaying it back to back from a HIP
    graph on the masks of that frame (see Tracer.replay_times), free of the host-side event overhead
    that dwarfs a few-microsecond kernel."""
    import torch
    from deltacnn_amd import hip_kernels as hk
    from deltacnn_amd.trace import Tracer, summarise
    delta.reset_layers()
    step = lambda i: frames[i * batch:(i + 1) * batch]
    with torch.no_grad():
        for i in range(3):
            delta(step(i))
        tr = Tracer()
        hk.set_tracer(tr)
        try:
            delta(step(3))
        finally:
            hk.set_tracer(None)
        times = tr.replay_times(alt_inputs=[step(2).data_ptr(), step(3).data_ptr()])
        for rec, us in zip(tr.records, times):
            rec["ms"] = us * 1e-3
        rows = tr.finish()
    agg = summarise(rows)
    for a in agg.values():
        a["launches_per_frame"] = a["launches"]
        a["us_per_launch"] = 1e3 * a["ms"] / a["launches"]
        a["ms_per_frame"] = a["ms"]
        a["bytes_per_launch"] = a["bytes"] / a["launches"]
        a["GBps"] = a["bytes"] / (a["ms"] * 1e-3) / 1e9 if a["ms"] > 0 else 0.0
        a["TFLOPs"] = a["flops"] / (a["ms"] * 1e-3) / 1e12 if a["ms"] > 0 else 0.0
    return agg, rows


def _trace_calls(fn, alt_inputs=None):
    """Run fn() once under the tracer, time its library calls by graph replay, return rows."""
    import torch
    from deltacnn_amd import hip_kernels as hk
    from deltacnn_amd.trace import Tracer
    tr = Tracer()
    hk.set_tracer(tr)
    try:
        with torch.no_grad():
            fn()
    finally:
        hk.set_tracer(None)
    times = tr.replay_times(alt_inputs=alt_inputs)
    for rec, us in zip(tr.records, times):
        rec["ms"] = us * 1e-3
    return tr.finish()


def _row_report(rows):
    """Per-launch report rows.  A launch whose share of a two-kernel call was measured as zero
    (the difference of two replays of a few microseconds, e.g. under a profiler) gets no rates."""
    out = []
    for r in rows:
        sec = r["ms"] * 1e-3
        rate = (lambda v, scale, digits: round(v / sec / scale, digits)) if sec > 0 else (lambda v, scale, digits: None)
        gbps, tflops = rate(r["bytes"], 1e9, 1), rate(r["flops"], 1e12, 2)
        out.append({"kernel": r["kernel"], "us": round(r["ms"] * 1e3, 3), "alg_GBps": gbps,
                    "hbm_frac": None if gbps is None else round(r["bytes"] / sec / 1e9 / HBM_PEAK_GBS, 4),
                    "alg_TFLOPs": tflops,
                    "mfma_frac": None if tflops is None else round(r["flops"] / sec / 1e12 / MFMA_F16_PEAK_TFLOPS, 5)})
    return out


def dense_library_conv_us(batch, cin, cout, k, h, w, groups=1, reps=30):
    """Device time of the vendor library's DENSE convolution of the same shape (PyTorch -> MIOpen, fp16,
    channels-last, `reps` calls replayed from one HIP graph): what the delta kernels are up against on the
    same GPU, reported beside their own times."""
    import torch
    x = torch.randn(batch, cin, h, w, device="cuda", dtype=torch.half).contiguous(memory_format=torch.channels_last)
    wt = torch.randn(cout, cin // groups, k, k, device="cuda", dtype=torch.half).contiguous(memory_format=torch.channels_last)
    fn = lambda: torch.nn.functional.conv2d(x, wt, padding=k // 2, groups=groups)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.no_grad(), torch.cuda.stream(side):
        for _ in range(3):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.no_grad(), torch.cuda.graph(graph):
        for _ in range(reps):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    graph.replay()
    e1.record()
    torch.cuda.synchronize()
    return round(e0.elapsed_time(e1) / reps * 1e3, 2)


def micro_bench():
    """Single-layer sweeps on a 64x64 fp16 map: 3x3 256->256, 1x1 256->1024 and depthwise 3x3
    C=512, each followed by ReLU with truncation (threshold 0.05), update density 1..100 %.
    Weights N(0,1)/sqrt(fan_in), cached pre-activation N(0,1), deltas N(0,0.5) on a random
    subset of pixels, N(0,1) garbage elsewhere."""
    import torch
    from deltacnn_amd import hip_kernels as hk
    from deltacnn_amd.filter_conversion import convert_half_filter
    H = W = 64
    out = []
    gen = torch.Generator().manual_seed(1235)
    for name, cin, cout, k, groups in (("conv3x3_256_256", 256, 256, 3, 1), ("conv1x1_256_1024", 256, 1024, 1, 1),
                                       ("dw3x3_512", 512, 512, 3, 512)):
        wt = (torch.randn(cout, cin // groups, k, k, generator=gen) / (cin // groups * k * k) ** 0.5).half()
        filt = convert_half_filter(wt, pixel_wise=groups > 1).cuda()
        packed = hk.pack_filter(filt, cin, cout, groups)
        prev = torch.randn(1, cout, H, W, generator=gen).half().cuda().contiguous(memory_format=torch.channels_last)
        trunc = torch.zeros_like(prev)
        obuf, omask = torch.zeros_like(prev), torch.zeros(1, 1, H, W, dtype=torch.int32, device="cuda")
        dense_us = dense_library_conv_us(1, cin, cout, k, H, W, groups)
        log(f"  micro {name:18s} dense library convolution (no activation): {dense_us:.2f} us")
        for rho in SWEEP:
            n = max(1, round(rho * H * W))
            mask = torch.zeros(H * W, dtype=torch.int32)
            mask[torch.randperm(H * W, generator=gen)[:n]] = 1
            mask = mask.view(1, 1, H, W).cuda()
            x = torch.randn(1, cin, H, W, generator=gen)
            x = torch.where(mask.cpu() != 0, x * 0.5, x).half().cuda().contiguous(memory_format=torch.channels_last)
            rows = _trace_calls(lambda: hk.sparse_conv_activation(
                x, filt, mask, None, prev, trunc, THRESHOLD, 1, 0, (1, 1), (k // 2, k // 2), (1, 1), groups, cout,
                packed_filter=packed, out=obuf, out_mask=omask))
            out.append({"op": name, "density": rho, "us": round(sum(r["ms"] for r in rows) * 1e3, 3),
                        "dense_library_conv_us": dense_us, "kernels": _row_report(rows)})
            log(f"  micro {name:18s} density {rho:4.2f}: " +
                "  ".join(f"{r['kernel']} {r['us']:.2f} us {r['alg_GBps'] or 0:.0f} GB/s {r['alg_TFLOPs'] or 0:.1f} TF/s"
                          for r in out[-1]["kernels"]))
    return out


def scaled_bench():
    """The memory-bound operators on a working set far beyond the caches (512x512, batch 8,
    64 channels fp16: 268 MB per tensor), where the bandwidth roofline applies."""
    import torch
    from deltacnn_amd import hip_kernels as hk
    B, C, H, W = 8, 64, 512, 512
    gen = torch.Generator(device="cuda").manual_seed(7)

    def feat():
        return torch.randn(B, C, H, W, device="cuda", dtype=torch.half, generator=gen).contiguous(
            memory_format=torch.channels_last)
    out = []
    a, b, c, d = feat(), feat(), feat(), feat()
    wdw = torch.randn(1, 3, 3, C, device="cuda", dtype=torch.half, generator=gen) / 3
    q = torch.randn(B, C, H // 2, W // 2, device="cuda", dtype=torch.half, generator=gen).contiguous(
        memory_format=torch.channels_last)
    qmask = torch.zeros(B, 1, H // 2, W // 2, dtype=torch.int32, device="cuda")
    h1, h2 = (torch.randn(B, C // 2, H, W, device="cuda", dtype=torch.half, generator=gen).contiguous(
        memory_format=torch.channels_last) for _ in range(2))
    scale, shift = (torch.randn(C, device="cuda", dtype=torch.half, generator=gen) for _ in range(2))
    from deltacnn_amd.filter_conversion import convert_half_filter
    wpw = convert_half_filter((torch.randn(C, C, 1, 1, generator=torch.Generator().manual_seed(8)) / C ** 0.5).half()).cuda()
    wpw_packed = hk.pack_filter(wpw, C, C, 1)
    w33 = convert_half_filter((torch.randn(C, C, 3, 3, generator=torch.Generator().manual_seed(9)) / (9 * C) ** 0.5).half()).cuda()
    w33_packed = hk.pack_filter(w33, C, C, 1)
    dense_us = {"conv3x3_64->64": dense_library_conv_us(B, C, C, 3, H, W, reps=10),
                "pointwise64->64": dense_library_conv_us(B, C, C, 1, H, W, reps=10),
                "depthwise3x3+relu": dense_library_conv_us(B, C, C, 3, H, W, groups=C, reps=10)}
    for rho in (0.1, 1.0):
        mask = (torch.rand(B, 1, H, W, device="cuda", generator=gen) < rho).to(torch.int32)
        mask2 = mask.clone()
        ops = {
            "sparsify": (lambda: hk.sparsify(a, b, c, mask2, 1e9 if rho < 1 else -1.0), None),
            "activate_truncate": (lambda: hk.sparse_activation(a, b, c, mask2.copy_(mask), 0.0, 1, 0), None),
            "densify": (lambda: hk.densify(a, b, c, mask), None),
            "add": (lambda: hk.sparse_add_tensors(a, b, None, c, mask, mask, mask2, 1.0, 1.0, 0, False), None),
            "depthwise3x3+relu": (lambda: hk.sparse_conv_activation(a, wdw, mask, None, b, c, 0.0, 1, 0, (1, 1), (1, 1),
                                                                    (1, 1), C, C, out=d, out_mask=mask2), None),
        }
        ops.update({
            "maxpool2x2": (lambda: hk.sparse_pooling(a, b, (2, 2), mask, (2, 2), pooling_mode_int=0, out=q, out_mask=qmask), None),
            "avgpool2x2": (lambda: hk.sparse_pooling(a, None, (2, 2), mask, (2, 2), pooling_mode_int=1, out=q, out_mask=qmask), None),
            "upsample_x2": (lambda: hk.sparse_upsample(q, qmask_in, 2, out=(d, mask2)), None),
            "concat": (lambda: hk.sparse_concatenate((h1, mask), (h2, mask), out=(d, mask2)), None),
            "mul_add": (lambda: hk.sparse_mul_add(a, mask, d, mask2, scale, shift), None),
            "add_to_dense": (lambda: hk.sparse_add_to_dense_tensor(a, d, mask), None),
            "pointwise64->64": (lambda: hk.sparse_conv(a, wpw, mask, None, (1, 1), (0, 0), (1, 1), 1, c_out=C, out=d,
                                                         out_mask=mask2, packed_filter=wpw_packed), None),
            "pointwise64->64+relu": (lambda: hk.sparse_conv_activation(a, wpw, mask, None, b, c, 0.0, 1, 0, (1, 1), (0, 0),
                                                                         (1, 1), 1, C, out=d, out_mask=mask2,
                                                                         packed_filter=wpw_packed), None),
            # the K x K contraction at this size sits at the ridge (288 flop per byte): its row is read against both peaks
            "conv3x3_64->64": (lambda: hk.sparse_conv(a, w33, mask, None, (1, 1), (1, 1), (1, 1), 1, c_out=C, out=d,
                                                        out_mask=mask2, packed_filter=w33_packed), None),
        })
        qmask_in = (torch.rand(B, 1, H // 2, W // 2, device="cuda", generator=gen) < rho).to(torch.int32)
        if rho < 1:
            ops.pop("sparsify")  # its density is set by the data, measured at 100 % only
        for name, (fn, _) in ops.items():
            rows = _trace_calls(fn, alt_inputs=[a.data_ptr(), d.data_ptr()])
            rep = _row_report(rows)
            out.append({"op": name, "density": rho, "kernels": rep})
            if name in dense_us:  # the vendor library's dense convolution of the same shape (without the activation)
                out[-1]["dense_library_conv_us"] = dense_us[name]
                log(f"  scaled {name:20s} dense library convolution: {dense_us[name]:.1f} us")
            log(f"  scaled {name:20s} density {rho:4.2f}: " +
                "  ".join(f"{r['kernel']} {r['us']:.1f} us {r['alg_GBps'] or 0:.0f} GB/s ({100 * (r['hbm_frac'] or 0):.1f} % of HBM peak"
                          + (f", {100 * (r['mfma_frac'] or 0):.1f} % of the MFMA peak)" if (r['alg_TFLOPs'] or 0) >= 50 else ")")
                          for r in rep))
    return out


def _network_report(name, size, delta, dense, frames, steps, warmup, clip):
    """Frames/s of the delta path and of the dense model (eager and graph) on one clip, launches
    per frame, mean update density of the library calls, per-kernel device times and the kernel
    with the largest share of the frame with its fraction of the HBM (or fp16 MFMA) peak."""
    sec = run_delta(delta, frames, warmup, steps, "graph")
    dense_eager, dense_graph = run_dense(dense, frames, warmup, steps)
    agg, rows = trace_kernels(delta, frames)
    dom_name = max(agg, key=lambda k: agg[k]["ms"])
    dom = agg[dom_name]
    hbm, mfma = dom["GBps"] / HBM_PEAK_GBS, dom["TFLOPs"] / MFMA_F16_PEAK_TFLOPS
    return {
        "network": name, "input": list(size), "clip": clip, "value": round(1 / sec, 1), "unit": "frames/s",
        "ms_per_step": round(sec * 1e3, 4), "steps": steps, "warmup": warmup,
        "dense_gpu": {"eager_fps": round(1 / dense_eager, 1), "graph_fps": round(1 / dense_graph, 1),
                      "speedup_vs_dense_gpu": round(min(dense_eager, dense_graph) / sec, 3)},
        "library_launches_per_frame": sum(a["launches"] for a in agg.values()),
        "mean_input_density_of_library_calls": round(sum(r["density_in"] for r in rows) / len(rows), 3),
        "frame_alg_GBps": round(sum(a["bytes"] for a in agg.values()) / sec / 1e9, 2),
        "dominant_kernel": {"kernel": dom_name, "launches_per_frame": dom["launches"],
                            "us_per_launch": round(dom["us_per_launch"], 3),
                            "share_of_kernel_time": round(dom["ms"] / sum(a["ms"] for a in agg.values()), 3),
                            "bound": "mfma" if mfma > hbm else "hbm",
                            "achieved": round(dom["TFLOPs"], 2) if mfma > hbm else round(dom["GBps"], 1),
                            "unit": "TFLOP/s" if mfma > hbm else "GB/s", "frac": round(max(hbm, mfma), 4)},
        "kernels": {k: {"launches_per_frame": a["launches"], "us_per_launch": round(a["us_per_launch"], 3),
                        "ms_per_frame": round(a["ms_per_frame"], 4), "alg_GBps": round(a["GBps"], 1),
                        "alg_TFLOPs": round(a["TFLOPs"], 2)}
                    for k, a in sorted(agg.items(), key=lambda kv: -kv[1]["ms"])},
    }


def network_bench(which, steps, warmup, only_delta=False):
    """The two larger configurations (parity cases, not the headline): HRNet-W32 pose network at
    256x256 and the DLA-34 CenterNet detector at 544x960, fp16, batch 1, random-init weights
    rescaled on two frames, threshold 0.05; synthetic static-camera clips (one large moving blob /
    twelve pedestrian-sized rectangles, no sensor noise)."""
    import torch
    from deltacnn_amd import sparse_layers as SL
    from deltacnn_amd.networks import DLA34CenterNet, DenseLayers, HRNet, fold_data_statistics
    from deltacnn_amd.video import moving_rectangles_video
    builder, size, kw = {
        "hrnet": (HRNet, (256, 256), dict(n_rect=1, min_size=100, max_size=180, min_speed=2, max_speed=6)),
        "dla34": (DLA34CenterNet, (544, 960), dict(n_rect=12, min_size=30, max_size=200, min_speed=1, max_speed=5)),
    }[which]
    video = moving_rectangles_video(frames=clip_frames(steps, warmup), height=size[0], width=size[1],
                                    noise_sigma=0.0, **kw)
    torch.manual_seed(0)
    dense = builder(DenseLayers).eval().to("cuda", memory_format=torch.channels_last)
    with torch.no_grad():
        fold_data_statistics(dense, video[:2].to("cuda").contiguous(memory_format=torch.channels_last))
    state = {k: v.clone() for k, v in dense.state_dict().items()}
    dense = dense.half()
    SL.DCThreshold.t_default = THRESHOLD
    delta = builder(SL).eval()
    delta.load_state_dict(state)
    delta = delta.to("cuda", memory_format=torch.channels_last).half()
    delta.process_filters()
    frames = gpu_frames(video)
    clip = (f"static background, {kw['n_rect']} textured rectangle(s) of {kw['min_size']}-{kw['max_size']} px moving "
            f"{kw['min_speed']}-{kw['max_speed']} px/frame, no sensor noise")
    if only_delta:  # for profiling runs: nothing but the delta path's kernels
        sec = run_delta(delta, frames, warmup, steps, "graph")
        return {"network": which, "value": round(1 / sec, 1), "unit": "frames/s", "ms_per_step": round(sec * 1e3, 4),
                "steps": steps}
    return _network_report(which, size, delta, dense, frames, steps, warmup, clip)


def cpu_baseline(state, video, n_frames, threads):
    """The CPU oracle of the delta path (pure PyTorch, fp32) on this host, bounded sample."""
    import torch
    from oracle import delta_layers as OL
    from deltacnn_amd.networks import DenseLayers, MobileNetV2
    torch.set_num_threads(threads)
    OL.DCThreshold.t_default = THRESHOLD
    cpu_state = {k: v.float().cpu() for k, v in state.items()}
    model = MobileNetV2(OL).eval()
    model.load_state_dict(cpu_state)
    dense = MobileNetV2(DenseLayers).eval()
    dense.load_state_dict(cpu_state)
    frames = video[:n_frames + 1].float()
    with torch.no_grad():
        model(frames[0:1])
        t0 = time.perf_counter()
        for i in range(1, n_frames + 1):
            model(frames[i:i + 1])
        delta_fps = n_frames / (time.perf_counter() - t0)
        dense(frames[0:1])
        t0 = time.perf_counter()
        for i in range(1, n_frames + 1):
            dense(frames[i:i + 1])
        dense_fps = n_frames / (time.perf_counter() - t0)
    return delta_fps, dense_fps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--density", type=float, default=0.10)
    ap.add_argument("--mode", choices=["graph", "eager"], default="graph")
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-micro", action="store_true", help="skip the single-layer and scaled-shape sections")
    ap.add_argument("--no-networks", action="store_true",
                    help="skip the closing section that times MobileNetV2 on the moving-rectangles clip, HRNet-W32 "
                         "256x256 and DLA-34/CenterNet 544x960")
    ap.add_argument("--only-delta", action="store_true",
                    help="time the delta path only and print a short JSON line (for profiling runs)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="with --only-delta: end with one 256 MiB device-to-device copy kernel, the known-size "
                         "reference that hardware traffic counters of a profiling run are scaled by")
    ap.add_argument("--network", choices=["mobilenetv2", "hrnet", "dla34"], default="mobilenetv2",
                    help="hrnet / dla34: time that configuration instead and print a short JSON line")
    ap.add_argument("--only-streams", type=int, default=0, metavar="N",
                    help="time the step of N video streams as one batch only and print a short JSON line with the "
                         "sum of the step's library calls replayed one by one beside it (for profiling runs; with "
                         "--no-sweep the step alone, so that a kernel trace of the run holds no other launches of "
                         "the library than the eager frames and the step)")
    ap.add_argument("--only-micro", action="store_true",
                    help="run the single-layer and scaled-shape sections only (for profiling runs)")
    ap.add_argument("--cpu-frames", type=int, default=200,
                    help="delta frames of the clip timed on the host CPU (bounded by the clip length)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path runs on ONE GPU (frames of a stream are strictly serial and a "
              "stream's caches live on its GPU); --gpus must be 1. Independent video streams shard "
              "one per GPU without any collective.", file=sys.stderr)
        sys.exit(2)

    import torch
    from deltacnn_amd import _lib
    from deltacnn_amd.video import controlled_density_video, moving_rectangles_video
    if not os.path.exists(_lib.LIB_PATH):
        from deltacnn_amd.csrc.build import build
        build()
    _lib.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.only_micro:
        print(json.dumps({"micro": micro_bench(), "scaled": scaled_bench()}), flush=True)
        return
    if args.network != "mobilenetv2":
        print(json.dumps(network_bench(args.network, min(args.steps, 64), min(args.warmup, 16), args.only_delta)),
              flush=True)
        return

    plan = launch_plan(args.steps, args.warmup)
    video = controlled_density_video(frames=clip_frames(args.steps, args.warmup), density=args.density)
    stats_video = moving_rectangles_video(frames=4)
    dense, delta, state = build_models(stats_video.to("cuda").contiguous(memory_format=torch.channels_last))
    frames = gpu_frames(video)

    if args.only_streams > 0:
        print(json.dumps(streams_profile(delta, args.only_streams, args.density, isolated=not args.no_sweep)), flush=True)
        return
    sec = run_delta(delta, frames, args.warmup, args.steps, args.mode)
    fps = 1.0 / sec
    log(f"delta path: {fps:.1f} frames/s ({sec * 1e3:.3f} ms/frame, mode={args.mode})")
    if args.only_delta:
        if args.calibrate_copy:
            src = torch.ones(64 << 20, dtype=torch.float32, device="cuda")
            dst = torch.empty_like(src)
            torch.cuda.synchronize()
            dst.copy_(src)  # 256 MiB read + 256 MiB written by one copy kernel
            torch.cuda.synchronize()
        print(json.dumps({"value": round(fps, 2), "unit": "frames/s", "ms_per_step": round(sec * 1e3, 4),
                          "steps": args.steps, "update_density": args.density}), flush=True)
        return

    graph_launches = ([plan["unroll"]] * plan["timed_main"] + ([plan["tail"]] if plan["tail"] else [])
                      if args.mode == "graph" else [])
    result = {
        "metric": "frames/sec vs update density (MobileNetV2 224^2); HBM GB/s % of peak",
        "value": round(fps, 2), "unit": "frames/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "MobileNetV2 w1.0 (BN folded, 1000-way head) 224x224 fp16 channels-last "
                               "batch 1, threshold 0.05 on all layers, controlled-density video",
                   "update_density": args.density, "launch_mode": args.mode,
                   "frames_per_graph_launch": plan["unroll"] if args.mode == "graph" else 0,
                   "timed_graph_launches": graph_launches,
                   "weights": "random init (seed 0) rescaled per conv to unit output variance"},
        "roofline": None, "cpu_baseline": None,
    }
    errors = {}

    def emit():
        """One JSON line with everything known so far; the LAST line printed is the result.  It
        is printed as soon as the headline exists and again after each group of sections, so a
        failure further down cannot erase it."""
        if errors:
            result["errors"] = errors
        print(json.dumps(result), flush=True)

    def section(name, fn):
        """Run one report section; a failure is recorded under errors[name] and the run goes on."""
        try:
            return fn()
        except Exception as e:  # noqa: BLE001 -- the report must survive any one section
            import traceback
            errors[name] = f"{type(e).__name__}: {e}"
            log(f"section {name} failed:\n{traceback.format_exc()}")
            return None

    emit()

    # -- the dominant kernel's roofline: per-call device times of one traced frame ------------
    def roofline_section():
        agg, rows = trace_kernels(delta, frames)
        dom_name = max(agg, key=lambda k: agg[k]["ms"])
        dom = agg[dom_name]
        result["kernels"] = {k: {"launches_per_frame": round(a["launches_per_frame"], 2),
                                 "us_per_launch": round(a["us_per_launch"], 3),
                                 "ms_per_frame": round(a["ms_per_frame"], 4),
                                 "alg_bytes_per_launch": round(a["bytes_per_launch"], 1),
                                 "alg_GBps": round(a["GBps"], 2), "alg_TFLOPs": round(a["TFLOPs"], 3)}
                             for k, a in sorted(agg.items(), key=lambda kv: -kv[1]["ms"])}
        result["library_launches_per_frame"] = sum(a["launches"] for a in agg.values())
        result["frame_alg_GBps"] = round(sum(a["bytes"] for a in agg.values()) / sec / 1e9, 2)
        result["kernel_time_sum_ms"] = round(sum(a["ms"] for a in agg.values()), 4)
        traffic = traffic_source = None
        tpath = os.path.join(ROOT, "profiles", "pmc_traffic.json")
        if os.path.exists(tpath):  # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
            with open(tpath) as f:
                traffic = json.load(f).get(dom_name, {}).get("bytes_per_launch")
            traffic_source = ("not measured by this run: read from profiles/pmc_traffic.json, the summary of two "
                              "separate rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) of `bench.py --only-delta "
                              "--calibrate-copy`; commands in profiles/mobilenetv2_224_delta_frame_traffic.txt")
        result["roofline"] = {
            "bound": "hbm", "kernel": dom_name, "achieved": round(dom["GBps"], 2), "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": round(dom["GBps"] / HBM_PEAK_GBS, 5), "traffic": traffic,
            "traffic_source": traffic_source,
            "bytes_per_launch": round(dom["bytes_per_launch"], 1),
            "us_per_launch": round(dom["us_per_launch"], 3),
            "duration_source": "live: every library call of one traced frame replayed back to back from a HIP "
                               "graph between two events on the stream it runs on, averaged over this kernel's "
                               "launches (the committed rocprofv3 average includes the profiler's dispatch "
                               "interception)",
            "note": "latency-bound regime: the feature maps of this workload are <= 2.4 MB and "
                    "an empty dependent kernel in a HIP graph already costs ~1.6 us"}
    section("roofline", roofline_section)

    # -- the CPU restatement of the same path on this host's cores (bounded sample) -----------
    def cpu_section():
        # 16 = the CPU share a one-GPU box grants one job here, whatever os.cpu_count() shows
        threads = min(16, os.cpu_count() or 1)
        n = max(1, args.cpu_frames)
        clip = video if video.shape[0] > n else controlled_density_video(frames=n + 1, density=args.density)
        d_fps, dn_fps = cpu_baseline(state, clip, n, threads)
        result["cpu_baseline"] = {
            "value": round(d_fps, 3), "unit": "frames/s", "cores": threads, "kind": "port",
            "sample": f"{n} delta frames of the same synthetic video (same generator and seed) through the "
                      f"fp32 CPU oracle (pure PyTorch layers) after the dense first frame",
            "dense_cpu_fps": round(dn_fps, 3)}
        log(f"CPU oracle: {d_fps:.1f} frames/s delta, {dn_fps:.1f} dense, {threads} threads")
    if not args.no_cpu:
        section("cpu_baseline", cpu_section)

    dense_best = [None]

    def dense_section():
        dense_eager, dense_graph = run_dense(dense, frames, args.warmup, args.steps)
        dense_best[0] = min(dense_eager, dense_graph)
        log(f"dense GPU: eager {1 / dense_eager:.1f} fps, graph {1 / dense_graph:.1f} fps")
        result["dense_gpu"] = {"eager_fps": round(1 / dense_eager, 1), "graph_fps": round(1 / dense_graph, 1),
                               "speedup_vs_dense_gpu": round(dense_best[0] / sec, 3)}
    section("dense_gpu", dense_section)
    emit()

    def sweep_section():
        sweep = result["sweep"] = []
        sw_steps, sw_warm = min(args.steps, 12 * UNROLL), min(args.warmup, 10)
        for rho in SWEEP:
            v = gpu_frames(controlled_density_video(frames=clip_frames(sw_steps, sw_warm), density=rho))
            s = run_delta(delta, v, sw_warm, sw_steps, args.mode)
            sweep.append({"density": rho, "fps": round(1.0 / s, 1), "ms_per_frame": round(s * 1e3, 4)})
            if dense_best[0]:
                sweep[-1]["speedup_vs_dense_gpu"] = round(dense_best[0] / s, 3)
            log(f"  density {rho:4.2f}: {1 / s:9.1f} fps")
    if not args.no_sweep:
        section("sweep", sweep_section)

    def logits_section():
        with torch.no_grad():
            ref_logits = dense(frames[-1:]).float()
            delta.reset_layers()
            for i in range(frames.shape[0]):
                out = delta(frames[i:i + 1])
            result["logit_max_abs_diff_vs_dense"] = round(float((out.float() - ref_logits).abs().max()), 4)
            result["logit_max_abs"] = round(float(ref_logits.abs().max()), 4)
    section("logits", logits_section)
    emit()

    if not args.no_micro:
        def streams_section():
            out = result["streams_as_batch"] = []
            for nb in (8, 32):
                out.append(streams_bench(delta, dense, batch=nb))
                log(f"{nb} streams as a batch: delta {out[-1]['delta_fps_total']:.0f} frames/s in total, "
                    f"dense graph {out[-1]['dense_graph_fps_total']:.0f}")
            sw = result["streams_32_sweep"] = []
            for rho in SWEEP:
                sw.append(streams_bench(delta, dense, batch=32, steps=32, warmup=8, density=rho, with_dense=False))
                log(f"  32 streams, density {rho:4.2f}: {sw[-1]['delta_fps_total']:9.0f} frames/s in total")
        section("streams_as_batch", streams_section)

        def micro_section():
            log("single-layer sweeps (64x64 fp16):")
            result["micro"] = micro_bench()
        section("micro", micro_section)

        def scaled_section():
            log("scaled shapes (512x512, batch 8, C=64 fp16):")
            result["scaled"] = scaled_bench()
        section("scaled", scaled_section)
        emit()

    # -- the other configurations, each on its own clip (after the headline has been emitted) --
    if not args.no_networks:
        nets = result["networks"] = []
        nw_steps, nw_warm = min(args.steps, 48), min(args.warmup, 8)

        def config3_section():
            # MobileNetV2 on the clip its configuration names: 64 frames, smooth-noise background,
            # three textured rectangles of 20-60 px moving 1-4 px/frame, sensor noise sigma 0.01
            clip = gpu_frames(moving_rectangles_video(frames=max(64, clip_frames(nw_steps, nw_warm))))
            nets.append(_network_report("mobilenetv2", (224, 224), delta, dense, clip, nw_steps, nw_warm,
                                        "64-frame synthetic video: static smooth-noise background, 3 textured rectangles "
                                        "of 20-60 px moving 1-4 px/frame, Gaussian sensor noise sigma 0.01"))
            log(f"MobileNetV2 on the moving-rectangles clip: {nets[-1]['value']:.0f} frames/s")
        section("networks.mobilenetv2_clip", config3_section)
        emit()

        def default_init_section():
            # the same network and clip with PyTorch's own initialisation left as it is (no rescaling
            # of the weights on data): activations shrink from layer to layer, so threshold 0.05
            # truncates far more than in a trained network -- the other end of the range
            from deltacnn_amd import sparse_layers as SL
            from deltacnn_amd.networks import DenseLayers, MobileNetV2
            torch.manual_seed(0)
            d0 = MobileNetV2(DenseLayers).eval().to("cuda", memory_format=torch.channels_last)
            st = {k: v.clone() for k, v in d0.state_dict().items()}
            d0 = d0.half()
            SL.DCThreshold.t_default = THRESHOLD
            m0 = MobileNetV2(SL).eval()
            m0.load_state_dict(st)
            m0 = m0.to("cuda", memory_format=torch.channels_last).half()
            m0.process_filters()
            clip = gpu_frames(moving_rectangles_video(frames=max(64, clip_frames(nw_steps, nw_warm))))
            nets.append(_network_report("mobilenetv2 (PyTorch default initialisation, weights not rescaled)", (224, 224), m0, d0,
                                        clip, nw_steps, nw_warm, "as above"))
            log(f"MobileNetV2, default initialisation: {nets[-1]['value']:.0f} frames/s, mean density "
                f"{nets[-1]['mean_input_density_of_library_calls']}")
        section("networks.mobilenetv2_default_init", default_init_section)
        emit()
        for which in ("hrnet", "dla34"):
            def net_section(which=which):
                nets.append(network_bench(which, nw_steps, nw_warm))
                log(f"{which}: {nets[-1]['value']:.0f} frames/s, dense graph {nets[-1]['dense_gpu']['graph_fps']:.0f}, "
                    f"{nets[-1]['library_launches_per_frame']} launches per frame")
            section(f"networks.{which}", net_section)
            emit()


if __name__ == "__main__":
    main()
