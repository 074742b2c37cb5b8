"""Per-call tracer for the delta operators: durations from stream events and ALGORITHMIC
byte / flop counts from the shapes and the measured mask populations.

Algorithmic traffic is the minimum a delta operator has to move (s = bytes per element,
m = 4-byte mask word, P pixels, n_x = number of active pixels of mask x):

  sparsify           R = 2*P*C*s                          W = 2*n_out*C*s + P*m
  activate_truncate  R = P*m + n_in*3*C*s                 W = n_out*3*C*s + (n_in-n_out)*(C*s + m)
  densify            R = P*m + n*2*C*s                    W = n*C*s   (+ dense copy: R += (P-n)*C*s, W += P*C*s)
  add                R = 2*P*m + (n_a+n_b)*C*s [+n_out*C*s]  W = n_out*C*s [+n_out*C*s] + P*m
  conv / deconv      R = P_in*m + n_in*Cin*s + K*K*(Cin/g)*Cout*s   W = n_out*Cout*s + P_out*m
                     (conv_add, deconv_add: + P_out*m + n_res*Cout*s for the residual; conv_act in one launch:
                     + the activate_truncate state traffic R += n_mid*2*Cout*s,
                     W += n_out*2*Cout*s + (n_mid-n_out)*Cout*s, n_mid = updated outputs before
                     truncation; conv_act in two launches: a conv row and an activate_truncate row)
                     flops = 2*(Cin/g)*Cout*N_pairs, N_pairs = sum over updated outputs of the
                     active inputs in their window (computed exactly from the masks)
                     (conv_group: the conv / conv_add / conv_act terms of its layers added up, one row
                     for the grouped convolution launch and one for the grouped activation launch)
  pool               R = P_in*m + n_in*C*s [max: + n_cov*C*s]   W = n_out*C*s + P_out*m
                     (pool_update, the maximum with the layer's cache update in its launch: W += n_in*C*s)
                     (the maximum of an updated window needs the cached input of EVERY pixel of the
                     window, updated or not: n_cov = input pixels covered by updated windows)
  add_to_dense       R = P*m + 2*n*C*s                    W = n*C*s
  upsample           R = P*m + n*C*s                      W = S*S*(n*C*s + P*m)
  concat             R = 2*P*m + (n_a*Ca + n_b*Cb)*s      W = n_out*(Ca+Cb)*s + P*m
  concat_conv        (a 1x1 convolution over k tensors that are never concatenated)
                     R = sum_i (P*m + n_i*C_i*s) + Cin*Cout*s   W = n_out*Cout*s + P*m
                     flops = 2*Cout*sum_i n_i*C_i
  mul_add            R = P*m + n*C*s + C*s                W = n*C*s
  block              (depthwise 3x3 + activation -> projection (+ residual) -> expansion + activation in
                     one launch; Ch hidden, Cp projection, Ce expansion channels; n_mid = updated
                     depthwise outputs before truncation, n_out / n_ex = pixels of the block output /
                     expansion output mask; the hidden mask is never stored, so the depthwise layer's
                     kept pixels are counted as min(n_mid, n_out))
                     R = P_in*m + n_in*Ch*s + 9*Ch*s + n_mid*2*Ch*s + Ch*Cp*s [+ P*m + n_res*Cp*s]
                         [+ Cp*Ce*s + n_out*2*Ce*s]
                     W = n_keep*2*Ch*s + (n_mid-n_keep)*Ch*s + n_out*Cp*s + P*m
                         [+ n_ex*3*Ce*s + (n_out-n_ex)*Ce*s + P*m]
                     flops = 2*9*Ch*n_mid (as tap pairs) + 2*Ch*Cp*n_keep + 2*Cp*Ce*n_out
"""
from __future__ import annotations

from collections import defaultdict

import torch
import torch.nn.functional as F

from . import _lib


class Tracer:
    """Install with ``hip_kernels.set_tracer(t)``; run frames eagerly; ``t.finish()``."""

    def __init__(self, count_pairs: bool = True):
        self.records = []
        self.count_pairs = count_pairs

    @staticmethod
    def _count(mask):
        return None if mask is None else (mask != 0).sum()

    def run(self, op, fn, args, meta):
        rec = {"op": op, "meta": meta}
        if op == "add_group":
            rec["items"] = [{"n_in": self._count(i["in_mask"]), "n_in_b": self._count(i["in_mask_b"]), "pairs": None}
                            for i in meta["items"]]
        if op == "conv_group":  # one set of counts per layer of the group
            rec["items"] = [{"n_in": self._count(i["in_mask"]), "n_in_b": self._count(i["in_mask_b"]),
                             "pairs": self._pairs(i["g"], i["in_mask"], False) if self.count_pairs else None}
                            for i in meta["items"]]
        if op == "concat_conv":
            rec["n_seg"] = [self._count(m) for m in meta["seg_masks"]]
        rec["n_in"] = self._count(meta.get("in_mask"))
        rec["n_in_b"] = self._count(meta.get("in_mask_b"))
        if self.count_pairs and op in ("conv", "deconv", "deconv_add", "conv_act", "conv_add", "block"):
            rec["pairs"], rec["n_mid"] = self._pairs(meta["g"], meta["in_mask"], op in ("deconv", "deconv_add"))
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        rc = fn(*args)
        end.record()
        if rc != 0:  # nothing was launched (e.g. a fused form that does not exist for this shape)
            return rc
        rec["events"] = (start, end)
        rec["kernels"] = _lib.load().dc_last_kernels().decode().split("+")
        rec["n_out"] = self._count(meta.get("out_mask"))
        rec["n_ex"] = self._count(meta.get("ex_mask"))
        for it, im in zip(rec.get("items", []), meta.get("items", [])):
            it["n_out"] = self._count(im["out_mask"])
        if op in ("pool", "pool_update") and meta.get("mode") == 0:
            rec["n_cov"] = self._covered(meta["g"], meta["out_mask"])
        rec["call"] = (fn, args)
        self.records.append(rec)
        return rc

    IN_PLACE = ("activate_truncate", "mul_add")

    def replay_times(self, repeats: int = 20, rounds: int = 5, alt_inputs=None):
        """Device time per call of every recorded call, free of host and event overhead: the
        call is captured `repeats` times back to back into a HIP graph (each launch depends on
        the previous one, as inside a frame) and the graph is replayed `rounds` times between
        two events.  Returns microseconds per call, one per record; a call that launches two
        kernels (convolution, then activation/truncation) also gets ``split_us`` per kernel.

        The replays pass the recorded device pointers again: operands of the traced calls
        must still be allocated (the records hold references to the masks and to every buffer
        the wrappers allocated themselves; tensors the caller passed in are the caller's to
        keep).  Every call has to see the masks of the traced frame, so
          * records are replayed last to first: a replay only disturbs its own outputs, whose
            consumers have been timed already;
          * an operator that works in place is replayed behind its producer (which restores the
            incoming delta and mask each time) and the producer's own time is subtracted;
          * sparsify alternates between the frames in `alt_inputs` (device pointers), else
            its second replay would find an unchanged frame and an empty mask."""
        stream = torch.cuda.Stream()

        def timed(calls):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                cs = torch.cuda.current_stream().cuda_stream
                for r in range(repeats):
                    for op, fn, args in calls:
                        a = list(args[:-1]) + [cs]
                        if op == "sparsify" and alt_inputs:
                            a[0] = alt_inputs[r % len(alt_inputs)]
                        fn(*a)
            g.replay()
            torch.cuda.synchronize()
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(rounds):
                g.replay()
            end.record()
            end.synchronize()
            return 1e3 * start.elapsed_time(end) / (rounds * repeats)

        times = [0.0] * len(self.records)
        for i in range(len(self.records) - 1, -1, -1):
            rec = self.records[i]
            call = (rec["op"],) + rec["call"]
            if rec["op"] in self.IN_PLACE and i > 0:
                prev = self.records[i - 1]
                pcall = (prev["op"],) + prev["call"]
                times[i] = max(timed([pcall, call]) - timed([pcall]), 0.0)
            else:
                times[i] = timed([call])
            if rec["op"] == "conv_group" and len(rec["kernels"]) == 2:
                # the grouped convolution on its own: the same items without the activations that
                # need the second launch; that launch gets the remainder
                fn, a = rec["call"]
                items = a[0]
                bare = type(items)(*items)
                for it, needs_second in zip(bare, self._second_launch(rec)):
                    if needs_second:
                        it.prev_out = None
                t_conv = min(timed([("conv_group", fn, (bare,) + tuple(a[1:]))]), times[i])
                rec["split_us"] = [t_conv, times[i] - t_conv]
                rec["bare"] = bare
            if rec["op"] == "conv_act" and len(rec["kernels"]) == 2:
                # the convolution launch of a two-launch call on its own: dc_conv with the same
                # operands runs the same kernel; the activation kernel gets the remainder
                a = rec["call"][1]
                conv_only = ("conv", _lib.load().dc_conv, a[:8] + a[13:])
                t_conv = min(timed([conv_only]), times[i])
                rec["split_us"] = [t_conv, times[i] - t_conv]
        return times

    @staticmethod
    def _second_launch(rec):
        """Per item of a conv_group record: does its activation run in the group's second launch
        (the convolution kernel finishes it only where one wavefront holds all output channels of
        a pixel: up to 32 channels and a reduction of at most 12 steps)."""
        flags = []
        for im in rec["meta"]["items"]:
            g = im["g"]
            steps = g.kernel_h * g.kernel_w * ((g.in_c + 31) // 32)
            one_wave = steps <= 12 and g.out_c <= 32 and g.out_c % 4 == 0
            flags.append(im["kind"] == "conv_act" and not one_wave)
        return flags

    @staticmethod
    def _covered(g, out_mask):
        """Input pixels that lie in the window of at least one updated output pixel."""
        m = (out_mask != 0).float()
        ones = torch.ones(1, 1, g.kernel_h, g.kernel_w, device=m.device)
        cov = F.conv_transpose2d(m, ones, stride=(g.stride_h, g.stride_w), dilation=(g.dilation_h, g.dilation_w))
        cov = cov[:, :, g.pad_top:g.pad_top + g.in_h, g.pad_left:g.pad_left + g.in_w]
        return (cov > 0).sum()

    @staticmethod
    def _pairs(g, mask, transposed):
        """N_pairs: number of (updated output pixel, active input pixel in its window) pairs.
        Every active input pixel reaches each output pixel of its footprint, and each of
        those outputs is updated, so N_pairs = sum over taps of the shifted mask.  Also returns
        the number of updated output pixels (the population of the dilated mask)."""
        m = (mask != 0).float()
        ones = torch.ones(1, 1, g.kernel_h, g.kernel_w, device=m.device)
        if transposed:
            cnt = F.conv_transpose2d(m, ones, stride=(g.stride_h, g.stride_w), padding=(g.pad_top, g.pad_left),
                                     dilation=(g.dilation_h, g.dilation_w))
        else:
            mp = F.pad(m, (g.pad_left, g.pad_right, g.pad_top, g.pad_bottom))
            cnt = F.conv2d(mp, ones, stride=(g.stride_h, g.stride_w), dilation=(g.dilation_h, g.dilation_w))
        return cnt.sum(), (cnt > 0).sum()

    def finish(self):
        """Synchronise and turn the records into one dict per KERNEL LAUNCH with ``kernel`` (the
        HIP kernel's name as reported by the library), ``call`` (the library operator),
        ``ms``, ``bytes``, ``flops``."""
        torch.cuda.synchronize()
        out = []
        for r in self.records:
            meta, op = r["meta"], r["op"]
            n_in = None if r["n_in"] is None else int(r["n_in"])
            n_in_b = None if r["n_in_b"] is None else int(r["n_in_b"])
            n_out = None if r["n_out"] is None else int(r["n_out"])
            s, m = meta["esize"], 4
            flops = 0
            extra = None  # second kernel of a two-launch call
            ms = r.get("ms", r["events"][0].elapsed_time(r["events"][1]))
            if op in ("conv", "deconv", "deconv_add", "conv_act", "conv_add"):
                g = meta["g"]
                p_in, p_out = g.batch * g.in_h * g.in_w, g.batch * g.out_h * g.out_w
                wbytes = g.kernel_h * g.kernel_w * (g.in_c // g.groups) * g.out_c * s
                n_mid = int(r["n_mid"]) if "n_mid" in r else n_out  # updated outputs before truncation
                two = op == "conv_act" and len(r["kernels"]) == 2
                rd = p_in * m + n_in * g.in_c * s + wbytes
                wr = (n_mid if two else n_out) * g.out_c * s + p_out * m
                if op in ("conv_add", "deconv_add"):  # + the residual operand of the fused add
                    rd += p_out * m + n_in_b * g.out_c * s
                if op == "conv_act" and not two:  # fused epilogue: cached state of every updated output
                    rd += n_mid * 2 * g.out_c * s
                    wr += n_out * 2 * g.out_c * s + (n_mid - n_out) * g.out_c * s
                if "pairs" in r:
                    flops = 2 * (g.in_c // g.groups) * g.out_c * int(r["pairs"])
                shape = f"{g.in_c}->{g.out_c} k{g.kernel_h} s{g.stride_h} @{g.in_h}x{g.in_w}"
                dens = (n_in / p_in, n_out / p_out)
                if two:
                    t_conv, t_act = r.get("split_us", [ms * 1e3 / 2, ms * 1e3 / 2])
                    ms = t_conv * 1e-3
                    C = g.out_c
                    extra = {"kernel": r["kernels"][1], "call": op, "shape": f"C{C} P{p_out}", "ms": t_act * 1e-3,
                             "bytes": p_out * m + n_mid * 3 * C * s + n_out * 3 * C * s + (n_mid - n_out) * (C * s + m),
                             "flops": 0, "density_in": n_mid / p_out, "density_out": n_out / p_out}
            elif op == "conv_group":  # the conv / conv_add / conv_act formulas above, summed over the layers
                rd = wr = 0
                act_bytes = act_in = act_out = act_px = 0
                second = self._second_launch(r)
                p_in_all = p_out_all = n_in_all = n_out_all = 0
                names = []
                for it, im, late in zip(r["items"], meta["items"], second):
                    g = im["g"]
                    p_in, p_out = g.batch * g.in_h * g.in_w, g.batch * g.out_h * g.out_w
                    ni, no = int(it["n_in"]), int(it["n_out"])
                    n_mid = int(it["pairs"][1]) if it["pairs"] is not None else no
                    rd += p_in * m + ni * g.in_c * s + g.kernel_h * g.kernel_w * g.in_c * g.out_c * s
                    wr += (n_mid if late else no) * g.out_c * s + p_out * m
                    if im["kind"] == "conv_add":
                        rd += p_out * m + int(it["n_in_b"]) * g.out_c * s
                    if im["kind"] == "conv_act" and not late:
                        rd += n_mid * 2 * g.out_c * s
                        wr += no * 2 * g.out_c * s + (n_mid - no) * g.out_c * s
                    if late:
                        C = g.out_c
                        act_bytes += p_out * m + n_mid * 3 * C * s + no * 3 * C * s + (n_mid - no) * (C * s + m)
                        act_in, act_out, act_px = act_in + n_mid, act_out + no, act_px + p_out
                    if it["pairs"] is not None:
                        flops += 2 * g.in_c * g.out_c * int(it["pairs"][0])
                    p_in_all, p_out_all, n_in_all, n_out_all = p_in_all + p_in, p_out_all + p_out, n_in_all + ni, n_out_all + no
                    names.append(f"{g.in_c}->{g.out_c}@{g.in_h}x{g.in_w}")
                kinds = {im["kind"] for im in meta["items"]}
                shape = f"{'/'.join(sorted(kinds))} k{meta['items'][0]['g'].kernel_h} x{len(names)}: " + " ".join(names)
                dens = (n_in_all / p_in_all, n_out_all / p_out_all)
                if len(r["kernels"]) == 2:
                    t_conv, t_act = r.get("split_us", [ms * 1e3 / 2, ms * 1e3 / 2])
                    ms = t_conv * 1e-3
                    extra = {"kernel": r["kernels"][1], "call": op, "shape": f"x{sum(second)} P{act_px}", "ms": t_act * 1e-3,
                             "bytes": act_bytes, "flops": 0, "density_in": act_in / act_px, "density_out": act_out / act_px}
            elif op == "add_group":  # the add formula, summed over the sums of the group
                rd = wr = 0
                p_all = act_all = out_all = 0
                for it, im in zip(r["items"], meta["items"]):
                    P, C, bs = im["P"], im["C"], im["b_scale"] ** 2
                    ni, nb, no = int(it["n_in"]), int(it["n_in_b"]), int(it["n_out"])
                    ext = no * C * s if im["with_prev"] else 0
                    rd += (P + P // bs) * m + (ni + nb) * C * s + ext
                    wr += no * C * s + ext + P * m
                    p_all, act_all, out_all = p_all + 2 * P, act_all + ni + nb * bs, out_all + no
                shape = f"x{len(meta['items'])}: " + " ".join(f"C{im['C']}P{im['P']}" for im in meta["items"])
                dens = (act_all / p_all, 2 * out_all / p_all)
            elif op == "block":
                g = meta["g"]
                ch, cp, ce = g.in_c, meta["Cp"], meta["Ce"]
                p_in, p_out = g.batch * g.in_h * g.in_w, g.batch * g.out_h * g.out_w
                n_mid = int(r["n_mid"]) if "n_mid" in r else n_out
                n_keep = min(n_mid, n_out)
                rd = p_in * m + n_in * ch * s + 9 * ch * s + n_mid * 2 * ch * s + ch * cp * s
                wr = n_keep * 2 * ch * s + (n_mid - n_keep) * ch * s + n_out * cp * s + p_out * m
                if n_in_b is not None:
                    rd += p_out * m + n_in_b * cp * s
                flops = 2 * ch * cp * n_keep + (2 * ch * int(r["pairs"]) if "pairs" in r else 0)
                if ce:
                    n_ex = int(r["n_ex"])
                    rd += cp * ce * s + n_out * 2 * ce * s
                    wr += n_ex * 3 * ce * s + (n_out - n_ex) * ce * s + p_out * m
                    flops += 2 * cp * ce * n_out
                shape = f"dw{ch} s{g.stride_h} -> {cp} -> {ce} @{g.out_h}x{g.out_w}"
                dens = (n_in / p_in, n_out / p_out)
            elif op == "expand_dw":  # 1x1 expansion with its activation left open + the depthwise layer that finishes it
                g = meta["g"]
                ci, ch = meta["Ci"], g.in_c
                p_px = g.batch * g.in_h * g.in_w
                rd = p_px * m + n_in * ci * s + ci * ch * s + n_in * 2 * ch * s
                wr = n_in * 2 * ch * s + p_px * m
                flops = 2 * ci * ch * n_in
                shape = f"{ci}->{ch} k1 s1 @{g.in_h}x{g.in_w} (open)"
                dens = (n_in / p_px, n_in / p_px)
                opened = meta.get("opened", False)  # the expansion ran in a project_expand call: one launch here
                if not opened:
                    ms = ms / 2  # the call's two launches share its time
                extra = {"kernel": r["kernels"][-1], "call": op, "shape": f"dw{ch} k3 s1 @{g.in_h}x{g.in_w} (closing)",
                         "ms": ms,
                         "bytes": p_px * m + n_in * 3 * ch * s + 9 * ch * s + n_out * 2 * ch * s
                                  + n_in * 2 * ch * s + n_out * 3 * ch * s + p_px * m,
                         "flops": 2 * 9 * ch * n_out, "density_in": n_in / p_px, "density_out": n_out / p_px}
            elif op == "project_expand":  # projection (+ residual sum) and the next expansion, activation left open
                g = meta["g"]
                ch, cm, ce = g.in_c, g.out_c, meta["Ce"]
                p_px = g.batch * g.in_h * g.in_w
                n_res = n_in_b or 0
                rd = p_px * m + n_in * ch * s + ch * cm * s + cm * ce * s + n_out * 2 * ce * s
                if n_in_b is not None:
                    rd += p_px * m + n_res * cm * s
                wr = n_out * cm * s + n_out * 2 * ce * s + 2 * p_px * m
                flops = 2 * ch * cm * n_in + 2 * cm * ce * n_out
                shape = f"{ch}->{cm}->{ce} k1 s1 @{g.in_h}x{g.in_w} (pair, open)"
                dens = (n_in / p_px, n_out / p_px)
            elif op == "pool_densify":  # the map's updated pixels in, accumulator in and out, dense copy out
                g = meta["g"]
                p_in = g.batch * g.in_h * g.in_w
                rd = p_in * m + n_in * g.in_c * s + g.batch * g.in_c * s
                wr = 2 * g.batch * g.in_c * s
                shape = f"C{g.in_c} k{g.kernel_h} @{g.in_h}x{g.in_w}"
                dens = (n_in / p_in, 1.0)
            elif op == "linear":
                rows, fi, fo = meta["rows"], meta["in_f"], meta["out_f"]
                rd, wr = (rows * fi + fo * fi + fo) * s, rows * fo * s
                flops = 2 * rows * fi * fo
                shape = f"{fi}->{fo} rows {rows}"
                dens = (1.0, 1.0)
            elif op == "concat_conv":  # a 1x1 convolution over tensors that are never concatenated
                g = meta["g"]
                P = g.batch * g.in_h * g.in_w
                n_seg = [int(v) for v in r["n_seg"]]
                rd = sum(P * m + n * c * s for n, c in zip(n_seg, meta["seg_channels"])) + g.in_c * g.out_c * s
                wr = n_out * g.out_c * s + P * m
                flops = 2 * g.out_c * sum(n * c for n, c in zip(n_seg, meta["seg_channels"]))
                shape = f"{'+'.join(str(c) for c in meta['seg_channels'])}->{g.out_c} k1 @{g.in_h}x{g.in_w}"
                dens = (sum(n_seg) / (P * len(n_seg)), n_out / P)
            elif op in ("pool", "pool_update"):
                g = meta["g"]
                p_in, p_out = g.batch * g.in_h * g.in_w, g.batch * g.out_h * g.out_w
                rd = p_in * m + n_in * g.in_c * s
                if meta["mode"] == 0:  # + the cached input of every pixel under an updated window
                    rd += int(r["n_cov"]) * g.in_c * s if "n_cov" in r else n_in * g.in_c * s
                wr = n_out * g.in_c * s + p_out * m
                if op == "pool_update":  # + the cached input of the updated pixels, written back
                    wr += n_in * g.in_c * s
                shape = f"C{g.in_c} k{g.kernel_h} @{g.in_h}x{g.in_w}"
                dens = (n_in / p_in, n_out / p_out)
            else:
                P, C = meta["P"], meta["C"]
                shape = f"C{C} P{P}"
                if op == "sparsify":
                    rd, wr = 2 * P * C * s, 2 * n_out * C * s + P * m
                    dens = (1.0, n_out / P)
                elif op == "activate_truncate":
                    rd = P * m + n_in * 3 * C * s
                    wr = n_out * 3 * C * s + (n_in - n_out) * (C * s + m)
                    dens = (n_in / P, n_out / P)
                elif op == "densify":
                    rd, wr = P * m + n_in * 2 * C * s, n_in * C * s
                    if meta.get("dense_copy"):  # + the dense copy of every pixel
                        rd, wr = rd + (P - n_in) * C * s, wr + P * C * s
                    dens = (n_in / P, n_in / P)
                elif op == "add":
                    n_o = n_out if n_out is not None else P
                    ext = n_o * C * s if meta["with_prev"] else 0
                    bs = meta.get("b_scale", 1) ** 2  # second operand read from a smaller map
                    rd = (P + P // bs) * m + (n_in + n_in_b) * C * s + ext
                    wr = n_o * C * s + ext + P * m
                    dens = ((n_in + n_in_b * bs) / (2 * P), n_o / P)
                elif op == "add_to_dense":
                    rd, wr = P * m + 2 * n_in * C * s, n_in * C * s
                    dens = (n_in / P, n_in / P)
                elif op == "upsample":
                    sc = meta["scale"] ** 2
                    rd, wr = P * m + n_in * C * s, sc * (n_in * C * s + P * m)
                    dens = (n_in / P, n_in / P)
                elif op == "concat":
                    cb = meta["Cb"]
                    rd = 2 * P * m + (n_in * C + n_in_b * cb) * s
                    wr = n_out * (C + cb) * s + P * m
                    dens = ((n_in + n_in_b) / (2 * P), n_out / P)
                else:  # mul_add
                    rd, wr = P * m + n_in * C * s + C * s, n_in * C * s
                    dens = (n_in / P, n_in / P)
            if not (op == "expand_dw" and meta.get("opened", False)):
                out.append({"kernel": r["kernels"][0] or op, "call": op, "shape": shape, "ms": ms,
                            "bytes": rd + wr, "flops": flops, "density_in": dens[0], "density_out": dens[1]})
            if extra is not None:
                out.append(extra)
        self.records = []
        return out


def summarise(rows):
    """Aggregate trace rows per kernel class: launches, total ms, bytes, flops."""
    agg = defaultdict(lambda: {"launches": 0, "ms": 0.0, "bytes": 0, "flops": 0})
    for r in rows:
        a = agg[r["kernel"]]
        a["launches"] += 1
        a["ms"] += r["ms"]
        a["bytes"] += r["bytes"]
        a["flops"] += r["flops"]
    return dict(agg)
