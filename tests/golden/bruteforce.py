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


def pool(delta, prev, mask, kernel, stride, padding, mode, dilation=(1, 1)):
    """Delta pooling over in-bounds window pixels (src/cuda/other_nn_layers.cu:2390-2459).
    mode 0 (max): max_w(prev + M*delta) - max_w(prev); with asymmetric padding a literal 0
    joins both maxima for window positions beyond the bottom (right) edge when
    top != bottom (left != right) (:2404-2406, :2418-2420).
    mode 1 (avg): sum_w(M*delta) / (Kh*Kw) (:2456).  Window taps are `dilation` pixels apart."""
    B, C, H, W = delta.shape
    t, b, l, r = pad4(padding)
    Ho = conv_out_size(H, kernel[0], stride[0], t, b, dilation[0])
    Wo = conv_out_size(W, kernel[1], stride[1], l, r, dilation[1])
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
                    iy = oy * stride[0] - t + ky * dilation[0]
                    if iy < 0:
                        continue
                    if iy >= H:  # one zero per padded bottom row, whatever the column
                        if iy < H + b and t != b:
                            hi = np.maximum(hi, 0.0)
                            hp = np.maximum(hp, 0.0)
                        continue
                    for kx in range(kernel[1]):
                        ix = ox * stride[1] - l + kx * dilation[1]
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


def activate_truncate_sum(delta, prev, trunc, mask, thr, act, mode):
    """Modes `norm` (1) and `rms` (2) (src/cuda/other_nn_layers.cu:664-719): as mode `max`, but a
    pixel is kept when sqrt(sum_c D_c^2) > thr, resp. sqrt(sum_c D_c^2 / C) > thr.  T, S and D
    round in the tensor's type; the sum of squares is taken in float64 here (the reference adds
    in lane order in the tensor's type), so inputs must keep the statistic away from thr.
    Returns new (delta, prev, trunc, mask) and the per-pixel statistic."""
    B, C, H, W = delta.shape
    dt = delta.dtype.type
    delta, prev, trunc, mask = delta.copy(), prev.copy(), trunc.copy(), mask.copy()
    stat = np.full((B, 1, H, W), np.nan)
    for n in range(B):
        for y in range(H):
            for x in range(W):
                if mask[n, 0, y, x] == 0:
                    continue
                T, S, D = (np.zeros(C, delta.dtype) for _ in range(3))
                total = 0.0
                for c in range(C):
                    T[c] = dt(trunc[n, c, y, x] + delta[n, c, y, x])
                    S[c] = dt(T[c] + prev[n, c, y, x])
                    D[c] = dt(_act(S[c], act) - _act(prev[n, c, y, x], act))
                    total += float(D[c]) * float(D[c])
                value = np.sqrt(total) if mode == 1 else np.sqrt(total / C)
                stat[n, 0, y, x] = value
                if value > thr:
                    prev[n, :, y, x] = S
                    delta[n, :, y, x] = D
                    trunc[n, :, y, x] = 0
                else:
                    trunc[n, :, y, x] = T
                    mask[n, 0, y, x] = 0
    return delta, prev, trunc, mask, stat


def sparsify_neighbourhood(x, prev, thr, k):
    """DCSparsify's `dilation` option (src/deltacnn/sparse_layers.py:1233-1244): a pixel is
    active when the largest |x - prev| over all channels of any pixel of the k x k window
    around it (window offset (k-1)//2 up/left, out-of-image positions ignored) exceeds thr.
    The delta is x - prev on EVERY pixel; the cache takes x on active pixels.
    Returns (delta, mask, new_prev)."""
    B, C, H, W = x.shape
    delta = (x - prev).astype(x.dtype)
    peak = np.abs(delta).max(axis=1)
    mask = np.zeros((B, 1, H, W), np.int32)
    new_prev = prev.copy()
    off = (k - 1) // 2
    # torch's max_pool2d output size for stride 1, padding off: H + 2*off - k + 1
    Ho, Wo = H + 2 * off - k + 1, W + 2 * off - k + 1
    for n in range(B):
        for y in range(Ho):
            for xx in range(Wo):
                best = -np.inf
                for dy in range(k):
                    for dx in range(k):
                        yy, xc = y - off + dy, xx - off + dx
                        if 0 <= yy < H and 0 <= xc < W:
                            best = max(best, float(peak[n, yy, xc]))
                if best > thr:
                    mask[n, 0, y, xx] = 1
                    new_prev[n, :, y, xx] = x[n, :, y, xx]
    return delta, mask, new_prev


def add_dense_out(a, mask_a, b, mask_b, prev, wa, wb, act):
    """DCAdd with dense_out (src/deltacnn/sparse_layers.py:1140-1172): the accumulated sum takes
    wa*a where Ma and wb*b where Mb; the result is act(accumulated sum) on EVERY pixel.
    float64 arithmetic.  Returns (dense result, new accumulated sum)."""
    B, C, H, W = a.shape
    new_prev = prev.astype(np.float64).copy()
    for n in range(B):
        for y in range(H):
            for x in range(W):
                if mask_a[n, 0, y, x] != 0:
                    new_prev[n, :, y, x] += wa * a[n, :, y, x].astype(np.float64)
                if mask_b[n, 0, y, x] != 0:
                    new_prev[n, :, y, x] += wb * b[n, :, y, x].astype(np.float64)
    out = np.empty_like(new_prev)
    for idx in np.ndindex(*new_prev.shape):
        out[idx] = _act(np.float64(new_prev[idx]), act)
    return out, new_prev


def add_to_dense(a, b, mask_a):
    """src/cuda/other_nn_layers.cu:1731-1957: b[pixel] += a[pixel] where the mask is set, b
    untouched elsewhere (rounded in the tensor's type).  Returns the new b."""
    out = b.copy()
    B, C, H, W = a.shape
    for n in range(B):
        for y in range(H):
            for x in range(W):
                if mask_a[n, 0, y, x] != 0:
                    for c in range(C):
                        out[n, c, y, x] = a.dtype.type(b[n, c, y, x] + a[n, c, y, x])
    return out
