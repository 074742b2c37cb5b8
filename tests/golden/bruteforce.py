"""Per-pixel, loop-level statements of the delta operators in plain numpy.

Each function walks pixels, taps and channels the way the operator is DEFINED (one output
element at a time, float64 accumulation where the definition is a sum), with no library
convolution or pooling call.  They are deliberately slow and independent of `oracle/`: the
oracle is checked against them on tiny inputs, and `make_vectors.py` uses them to write the
committed fixtures.

Tensors are numpy arrays in logical [B, C, H, W]; masks are int32 [B, 1, H, W].
Reference lines cited per function are relative to the DeltaCNN source tree.
"""
import numpy as np


def pad4(padding):
    """(top, bottom, left, right) from a 2- or 4-tuple (src/deltacnn/cuda_kernels.py:21-26)."""
    if len(padding) == 2:
        return padding[0], padding[0], padding[1], padding[1]
    return tuple(padding)


def conv_out_size(n, k, s, p0, p1, d):
    return (n + p0 + p1 - d * (k - 1) - 1) // s + 1


def conv(delta, mask, weight, bias, stride, padding, dilation, groups):
    """Delta convolution (src/cuda/conv_kernel.cu:156-213 mask, :511-630 values): ordinary
    cross-correlation over ACTIVE in-bounds inputs; the output mask is the OR of the input mask
    over the same taps.  weight is [Cout, Cin/g, Kh, Kw]."""
    B, Ci, H, W = delta.shape
    Co, Cig, Kh, Kw = weight.shape
    t, b, l, r = pad4(padding)
    Ho = conv_out_size(H, Kh, stride[0], t, b, dilation[0])
    Wo = conv_out_size(W, Kw, stride[1], l, r, dilation[1])
    out = np.zeros((B, Co, Ho, Wo), np.float64)
    om = np.zeros((B, 1, Ho, Wo), np.int32)
    cog = Co // groups
    for n in range(B):
        for oy in range(Ho):
            for ox in range(Wo):
                acc = np.zeros(Co, np.float64)
                hit = False
                for ky in range(Kh):
                    for kx in range(Kw):
                        iy = oy * stride[0] - t + ky * dilation[0]
                        ix = ox * stride[1] - l + kx * dilation[1]
                        if iy < 0 or iy >= H or ix < 0 or ix >= W or mask[n, 0, iy, ix] == 0:
                            continue
                        hit = True
                        for g in range(groups):  # acc[co] += sum_c delta[g*Cig + c] * W[co, c, ky, kx]
                            xs = delta[n, g * Cig:(g + 1) * Cig, iy, ix].astype(np.float64)
                            acc[g * cog:(g + 1) * cog] += weight[g * cog:(g + 1) * cog, :, ky, kx].astype(np.float64) @ xs
                if hit:
                    om[n, 0, oy, ox] = 1
                    out[n, :, oy, ox] = acc + (0.0 if bias is None else bias.astype(np.float64))
    return out, om


def deconv(delta, mask, weight, bias, stride, padding):
    """Delta transposed convolution (src/cuda/deconv_kernel.cu:296-336 mask, :460-481 values):
    every active input pixel i scatters delta[i] * W[:, :, ky, kx] to o = i*s - pad + k.
    weight is [Cin, Cout, Kh, Kw]; the output size has no output_padding
    (src/deltacnn/cuda_kernels.py:56-57)."""
    B, Ci, H, W = delta.shape
    _, Co, Kh, Kw = weight.shape
    Ho = (H - 1) * stride[0] - 2 * padding[0] + (Kh - 1) + 1
    Wo = (W - 1) * stride[1] - 2 * padding[1] + (Kw - 1) + 1
    out = np.zeros((B, Co, Ho, Wo), np.float64)
    om = np.zeros((B, 1, Ho, Wo), np.int32)
    for n in range(B):
        for iy in range(H):
            for ix in range(W):
                if mask[n, 0, iy, ix] == 0:
                    continue
                for ky in range(Kh):
                    for kx in range(Kw):
                        oy = iy * stride[0] - padding[0] + ky
                        ox = ix * stride[1] - padding[1] + kx
                        if oy < 0 or oy >= Ho or ox < 0 or ox >= Wo:
                            continue
                        om[n, 0, oy, ox] = 1
                        out[n, :, oy, ox] += delta[n, :, iy, ix].astype(np.float64) @ weight[:, :, ky, kx].astype(np.float64)
    if bias is not None:
        out += np.where(om != 0, bias.astype(np.float64)[None, :, None, None], 0.0)
    return out, om


def sparsify(x, prev, thr):
    """src/cuda/other_nn_layers.cu:820-881 (fp32): a pixel is active when any |x - prev| > thr;
    active pixels emit the difference on all channels and refresh the cache.  Returns
    (delta, mask, new_prev); delta is zero where inactive."""
    B, C, H, W = x.shape
    dt = x.dtype.type
    delta = np.zeros_like(x)
    mask = np.zeros((B, 1, H, W), np.int32)
    new_prev = prev.copy()
    for n in range(B):
        for y in range(H):
            for xx in range(W):
                d = (x[n, :, y, xx] - prev[n, :, y, xx]).astype(x.dtype)
                if np.any(np.abs(d) > dt(thr)):
                    delta[n, :, y, xx] = d
                    new_prev[n, :, y, xx] = x[n, :, y, xx]
                    mask[n, 0, y, xx] = 1
    return delta, mask, new_prev


def _act(v, act):
    if act == 1:
        return max(v, type(v)(0))
    if act == 2:
        return min(max(v, type(v)(0)), type(v)(6))
    if act == 3:
        return v * type(v)(0.1) if v < 0 else v
    return v


def activate_truncate(delta, prev, trunc, mask, thr, act):
    """Mode `max` (src/cuda/other_nn_layers.cu:396-463): per ACTIVE pixel T = trunc + delta,
    S = T + prev, D = act(S) - act(prev); kept (any |D| > thr): prev = S, delta = D, trunc = 0;
    dropped: trunc = T and the mask word is cleared.  Every operation rounds in the tensor's
    type.  Returns new (delta, prev, trunc, mask)."""
    B, C, H, W = delta.shape
    dt = delta.dtype.type
    delta, prev, trunc, mask = delta.copy(), prev.copy(), trunc.copy(), mask.copy()
    for n in range(B):
        for y in range(H):
            for x in range(W):
                if mask[n, 0, y, x] == 0:
                    continue
                keep = False
                T = np.zeros(C, delta.dtype)
                S = np.zeros(C, delta.dtype)
                D = np.zeros(C, delta.dtype)
                for c in range(C):
                    T[c] = dt(trunc[n, c, y, x] + delta[n, c, y, x])
                    S[c] = dt(T[c] + prev[n, c, y, x])
                    D[c] = dt(_act(S[c], act) - _act(prev[n, c, y, x], act))
                    keep = keep or abs(D[c]) > dt(thr)
                if keep:
                    prev[n, :, y, x] = S
                    delta[n, :, y, x] = D
                    trunc[n, :, y, x] = 0
                else:
                    trunc[n, :, y, x] = T
                    mask[n, 0, y, x] = 0
    return delta, prev, trunc, mask


def pool(delta, prev, mask, kernel, stride, padding, mode):
    """Delta pooling over in-bounds window pixels (src/cuda/other_nn_layers.cu:2390-2459).
    mode 0 (max): max_w(prev + M*delta) - max_w(prev); with asymmetric padding a literal 0
    joins both maxima for window positions beyond the bottom (right) edge when
    top != bottom (left != right) (:2404-2406, :2418-2420).
    mode 1 (avg): sum_w(M*delta) / (Kh*Kw) (:2456)."""
    B, C, H, W = delta.shape
    t, b, l, r = pad4(padding)
    Ho = conv_out_size(H, kernel[0], stride[0], t, b, 1)
    Wo = conv_out_size(W, kernel[1], stride[1], l, r, 1)
    out = np.zeros((B, C, Ho, Wo), np.float64)
    om = np.zeros((B, 1, Ho, Wo), np.int32)
    for n in range(B):
        for oy in range(Ho):
            for ox in range(Wo):
                hi = np.full(C, -np.inf)
                hp = np.full(C, -np.inf)
                sm = np.zeros(C)
                hit = False
                for ky in range(kernel[0]):
                    iy = oy * stride[0] - t + ky
                    if iy < 0:
                        continue
                    if iy >= H:  # one zero per padded bottom row, whatever the column
                        if iy < H + b and t != b:
                            hi = np.maximum(hi, 0.0)
                            hp = np.maximum(hp, 0.0)
                        continue
                    for kx in range(kernel[1]):
                        ix = ox * stride[1] - l + kx
                        if ix < 0:
                            continue
                        if ix >= W:
                            if ix < W + r and l != r:
                                hi = np.maximum(hi, 0.0)
                                hp = np.maximum(hp, 0.0)
                            continue
                        p = prev[n, :, iy, ix].astype(np.float64) if prev is not None else 0.0
                        if mask[n, 0, iy, ix] != 0:
                            hit = True
                            d = delta[n, :, iy, ix].astype(np.float64)
                        else:
                            d = 0.0
                        hi = np.maximum(hi, p + d)
                        hp = np.maximum(hp, p)
                        sm = sm + d
                if hit:
                    om[n, 0, oy, ox] = 1
                    out[n, :, oy, ox] = (hi - hp) if mode == 0 else sm / (kernel[0] * kernel[1])
    return out, om


def add(a, mask_a, b, mask_b, wa, wb):
    """DCAdd without activation (src/cuda/other_nn_layers.cu:1428-1558): on pixels of Ma | Mb,
    s = wa*a where Ma, then s = fma(b, wb, s) where Mb (single rounding)."""
    B, C, H, W = a.shape
    out = np.zeros_like(a)
    om = ((mask_a != 0) | (mask_b != 0)).astype(np.int32)
    dt = a.dtype.type
    for n in range(B):
        for y in range(H):
            for x in range(W):
                for c in range(C):
                    s = dt(0)
                    if mask_a[n, 0, y, x] != 0:
                        s = dt(a[n, c, y, x] * dt(wa))
                    if mask_b[n, 0, y, x] != 0:
                        # exact in float64 for fp16/fp32 operands of this magnitude, rounded once
                        s = dt(np.float64(b[n, c, y, x]) * np.float64(dt(wb)) + np.float64(s))
                    out[n, c, y, x] = s
    return out, om
