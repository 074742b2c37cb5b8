// Pointwise (1x1, stride 1) delta convolution on v_mfma_f32_16x16x32_f16.
//
// For a 1x1 convolution the output mask IS the input mask and a pixel tile is just a run of
// consecutive pixels, so these kernels drop the 2-d tile / window machinery of the generic
// path and are written around memory latency, which is what bounds them at batch 1: every
// load is unconditional (clamped address, value selected afterwards) so that the fragment
// loads of a whole reduction chunk are in flight together, and filter fragments -- which do
// not depend on the masks -- are requested together with the mask words.
//
// Operand roles as in the generic kernel: rows = 16 output channels from the packed filter
// [Cout pad 16][Cin pad 32], columns = 16 pixels (NHWC rows), fp32 accumulate, reduction in
// steps of 32 input channels taken in ascending order (both kernels below and the generic
// kernel accumulate a given output element with the same instruction sequence, so they agree
// bit for bit).
//
// pw_mfma_kernel      convolution only; a workgroup takes 64 pixels x 64 channels, or with
//                     KSPLIT 64 pixels x 16 channels with the reduction split over its four
//                     wavefronts (deep layers: long reduction, few pixels)
// pw_act_mfma_kernel  convolution + activation/truncation in one launch: a workgroup owns ALL
//                     output channels of its 16 pixels, so it can take the per-pixel keep/drop
//                     decision itself; the convolution output never travels through memory.
//                     Used for layers with many pixels and few channels (the high-resolution
//                     half of a network); deep layers keep the two-launch form, whose channel
//                     split over many workgroups is what streams their large filters fast
#include "epilogue.hpp"

namespace dc {
namespace {

__device__ __forceinline__ half8_t zero8() { return half8_t{0, 0, 0, 0, 0, 0, 0, 0}; }

struct PwP {
    int P, Ci, Co, ci_p, co_tiles;
};

template <bool KSPLIT>
__global__ void __launch_bounds__(256)
pw_mfma_kernel(PwP p, const half_t *__restrict__ in, const half_t *__restrict__ wp,
               const half_t *__restrict__ bias, half_t *__restrict__ out,
               const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask) {
    constexpr int NT = 4, S = 4;
    __shared__ float4_t s_red[KSPLIT ? 4 * NT * WAVE : 1];
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;
    const int cb = blockIdx.y;
    const int ct_raw = KSPLIT ? cb : cb * 4 + wave;
    const int ct = min(ct_raw, p.co_tiles - 1);  // surplus wavefronts compute a tile nobody stores
    const int kvalid = kq * 8;
    const int ksteps = p.ci_p >> 5;
    const int first = KSPLIT ? wave : 0, stride = KSPLIT ? 4 : 1;
    const half_t *wrow = wp + (size_t)(ct * 16 + l16) * p.ci_p + kvalid;

    int px[NT];
    bool on[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        px[nt] = blockIdx.x * 64 + nt * 16 + l16;
        const int m = mask[min(px[nt], p.P - 1)];
        on[nt] = px[nt] < p.P && m != 0;
    }
    // first chunk of filter fragments travels together with the mask words
    half8_t a[S];
#pragma unroll
    for (int i = 0; i < S; ++i) {
        const int s = min(first + i * stride, ksteps - 1);
        a[i] = *reinterpret_cast<const half8_t *>(wrow + (s << 5));
    }
    bool nt_on[NT];
    bool any = false;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        nt_on[nt] = ballot(on[nt]) != 0;
        any |= nt_on[nt];
    }
    if (cb == 0 && wave == 0 && kq == 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            if (px[nt] < p.P) out_mask[px[nt]] = on[nt] ? 1 : 0;
    }
    if (!any) return;

    float4_t acc[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt] = float4_t{0.f, 0.f, 0.f, 0.f};
    const half_t *xrow[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
        xrow[nt] = in + (size_t)(on[nt] ? px[nt] : 0) * p.Ci;

    for (int s0 = first; s0 < ksteps; s0 += S * stride) {
        if (s0 != first) {
#pragma unroll
            for (int i = 0; i < S; ++i) {
                const int s = min(s0 + i * stride, ksteps - 1);
                a[i] = *reinterpret_cast<const half8_t *>(wrow + (s << 5));
            }
        }
        // inactive pixels all point at pixel 0, so their (discarded) loads share one cache line
        half8_t x[S][NT];
#pragma unroll
        for (int i = 0; i < S; ++i) {
            const int s = min(s0 + i * stride, ksteps - 1);
            const int k = min((s << 5) + kvalid, p.Ci - 8);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
                x[i][nt] = *reinterpret_cast<const half8_t *>(xrow[nt] + k);
        }
#pragma unroll
        for (int i = 0; i < S; ++i) {
            const int s = s0 + i * stride;
            const bool kin = s < ksteps && (s << 5) + kvalid < p.Ci;
            if (s < ksteps) {  // wave-uniform
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
                    if (nt_on[nt])  // wave-uniform
                        acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                            a[i], (on[nt] && kin) ? x[i][nt] : zero8(), acc[nt], 0, 0, 0);
            }
        }
    }

    if (KSPLIT) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) s_red[(wave * NT + nt) * WAVE + lane] = acc[nt];
        __syncthreads();
        // wavefront w finishes pixel sub-tile w
        float4_t sum = s_red[(0 * NT + wave) * WAVE + lane];
#pragma unroll
        for (int w = 1; w < 4; ++w) sum += s_red[(w * NT + wave) * WAVE + lane];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            if (nt == wave) acc[nt] = sum;
    }
    if (ct_raw >= p.co_tiles) return;
    const int co = ct * 16 + kq * 4;
    float bv[4] = {0.f, 0.f, 0.f, 0.f};
    if (bias != nullptr) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (co + i < p.Co) bv[i] = float(bias[co + i]);
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        if (!on[nt] || (KSPLIT && nt != wave)) continue;
        half_t *o = out + (size_t)px[nt] * p.Co + co;
        if (co + 3 < p.Co && (p.Co & 3) == 0) {
            half4_t r;
#pragma unroll
            for (int i = 0; i < 4; ++i) r[i] = half_t(acc[nt][i] + bv[i]);
            *reinterpret_cast<half4_t *>(o) = r;
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (co + i < p.Co) o[i] = half_t(acc[nt][i] + bv[i]);
        }
    }
}

// --------------------------------------------------------------- fused conv + act/trunc
// Workgroup = NW wavefronts x 16 pixels x all output channels; wavefront w owns channel tiles
// w, w + NW, ... (at most CTW of them).  KS bounds the reduction steps: the input fragments of
// the 16 pixels stay in registers for the whole kernel and every loop is fully unrolled without
// branches (surplus steps multiply zero fragments, surplus tiles are computed and dropped), so
// the filter stream of a wavefront is one uninterrupted run of loads.  Requires Cout % 4 == 0.
template <int CTW, int ACT>
__device__ __forceinline__ void pw_epilogue(const float4_t (&acc)[CTW], const half4_t (&q)[CTW],
                                            const half4_t (&tr)[CTW], half4_t (&t)[CTW],
                                            half4_t (&sacc)[CTW], half4_t (&d)[CTW],
                                            const half_t *__restrict__ bias, bool on, int wave,
                                            int NW, int kq, const PwP &p, half_t thr, bool &hit,
                                            float &sq) {
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        const int ct = wave + j * NW;
        const int co = ct * 16 + kq * 4;
        const bool live = ct < p.co_tiles && co < p.Co;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float b = (bias != nullptr && live) ? float(bias[co + i]) : 0.f;
            const half_t v = half_t(acc[j][i] + b);
            t[j][i] = tr[j][i] + v;
            sacc[j][i] = t[j][i] + q[j][i];
            d[j][i] = act_apply<half_t>(sacc[j][i], ACT) - act_apply<half_t>(q[j][i], ACT);
            if (live && on) {
                hit |= tabs(d[j][i]) > thr;
                sq += float(d[j][i]) * float(d[j][i]);
            }
        }
    }
}

template <int NW, int CTW, int KS>
__global__ void __launch_bounds__(NW * WAVE)
pw_act_mfma_kernel(PwP p, const half_t *__restrict__ in, const half_t *__restrict__ wp,
                   const half_t *__restrict__ bias, half_t *__restrict__ out,
                   const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask,
                   half_t *__restrict__ prev, half_t *__restrict__ trunc, float thr_f, int act,
                   int mode) {
    __shared__ float s_stat[NW][16];
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;
    const int kvalid = kq * 8;
    const int ksteps = p.ci_p >> 5;
    const int px = blockIdx.x * 16 + l16;
    const int m = mask[min(px, p.P - 1)];
    // round trip 1: the mask word and every filter fragment of this wavefront (they do not
    // depend on the mask; a workgroup without active pixels wastes a few cached KB)
    half8_t a[CTW][KS];
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        const int ct = min(wave + j * NW, p.co_tiles - 1);
        const half_t *wrow = wp + (size_t)(ct * 16 + l16) * p.ci_p + kvalid;
#pragma unroll
        for (int s = 0; s < KS; ++s)
            a[j][s] = *reinterpret_cast<const half8_t *>(wrow + (min(s, ksteps - 1) << 5));
    }
#pragma unroll
    for (int j = 0; j < CTW; ++j)
#pragma unroll
        for (int s = 0; s < KS; ++s) DC_PIN(a[j][s]);
    const bool on = px < p.P && m != 0;
    if (ballot(on) == 0) {  // same 16 pixels in every wavefront: the whole workgroup leaves
        if (wave == 0 && kq == 0 && px < p.P) out_mask[px] = 0;
        return;
    }
    // round trip 2: input fragments and cached state of this lane's (pixel, 4 channel) cells;
    // inactive pixels all point at pixel 0, their loads share one cache line and are dropped
    const half_t *xrow = in + (size_t)(on ? px : 0) * p.Ci;
    half8_t x[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int k = (min(s, ksteps - 1) << 5) + kvalid;
        x[s] = *reinterpret_cast<const half8_t *>(xrow + min(k, p.Ci - 8));
    }
    half4_t q[CTW], tr[CTW];
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        const int ct = min(wave + j * NW, p.co_tiles - 1);
        const int co = min(ct * 16 + kq * 4, p.Co - 4);
        const size_t off = (size_t)(on ? px : 0) * p.Co + co;
        q[j] = *reinterpret_cast<const half4_t *>(prev + off);
        tr[j] = *reinterpret_cast<const half4_t *>(trunc + off);
    }
#pragma unroll
    for (int s = 0; s < KS; ++s) DC_PIN(x[s]);
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        DC_PIN(q[j]);
        DC_PIN(tr[j]);
    }
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const bool kin = s < ksteps && (s << 5) + kvalid < p.Ci;
        x[s] = (on && kin) ? x[s] : zero8();
    }
    float4_t acc[CTW];
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; ++s)
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j][s], x[s], acc[j], 0, 0, 0);
    }
    // epilogue: T = trunc + delta; S = T + prev; D = act(S) - act(prev), one rounding each
    const half_t thr = half_t(thr_f);
    half4_t t[CTW], sacc[CTW], d[CTW];
    bool hit = false;
    float sq = 0.f;
    switch (act) {
        case DC_ACT_RELU: pw_epilogue<CTW, DC_ACT_RELU>(acc, q, tr, t, sacc, d, bias, on, wave, NW, kq, p, thr, hit, sq); break;
        case DC_ACT_RELU6: pw_epilogue<CTW, DC_ACT_RELU6>(acc, q, tr, t, sacc, d, bias, on, wave, NW, kq, p, thr, hit, sq); break;
        case DC_ACT_LEAKY: pw_epilogue<CTW, DC_ACT_LEAKY>(acc, q, tr, t, sacc, d, bias, on, wave, NW, kq, p, thr, hit, sq); break;
        case DC_ACT_SIGMOID: pw_epilogue<CTW, DC_ACT_SIGMOID>(acc, q, tr, t, sacc, d, bias, on, wave, NW, kq, p, thr, hit, sq); break;
        case DC_ACT_SWISH: pw_epilogue<CTW, DC_ACT_SWISH>(acc, q, tr, t, sacc, d, bias, on, wave, NW, kq, p, thr, hit, sq); break;
        default: pw_epilogue<CTW, DC_ACT_LINEAR>(acc, q, tr, t, sacc, d, bias, on, wave, NW, kq, p, thr, hit, sq); break;
    }
    // per pixel: combine the four k-quarter lanes, then the wavefronts
    float stat;
    if (mode == DC_TRUNC_MAX) {
        const uint64_t b = ballot(hit);
        stat = ((b >> l16) & 0x0001000100010001ull) != 0 ? 1.f : 0.f;
    } else {
        sq += __shfl_xor(sq, 16, WAVE);
        sq += __shfl_xor(sq, 32, WAVE);
        stat = sq;
    }
    if (kq == 0) s_stat[wave][l16] = stat;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) tot += s_stat[w][l16];
    bool keep;
    if (mode == DC_TRUNC_MAX) keep = tot > 0.f;
    else keep = sqrtf(mode == DC_TRUNC_RMS ? tot / float(p.Co) : tot) > float(thr);
    if (wave == 0 && kq == 0 && px < p.P) out_mask[px] = (on && keep) ? 1 : 0;
    if (!on) return;
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        const int ct = wave + j * NW;
        const int co = ct * 16 + kq * 4;
        if (ct >= p.co_tiles || co >= p.Co) continue;
        const size_t off = (size_t)px * p.Co + co;
        if (keep) {
            *reinterpret_cast<half4_t *>(prev + off) = sacc[j];
            *reinterpret_cast<half4_t *>(out + off) = d[j];
            *reinterpret_cast<half4_t *>(trunc + off) = half4_t{0, 0, 0, 0};
        } else {
            *reinterpret_cast<half4_t *>(trunc + off) = t[j];
        }
    }
}

template <int CTW, int KS>
void pw_act_launch(dim3 grid, hipStream_t s, const PwP &p, const half_t *in, const half_t *wp,
                   const half_t *bias, half_t *out, const int32_t *mask, int32_t *out_mask,
                   half_t *prev, half_t *trunc, float thr, int act, int mode) {
    pw_act_mfma_kernel<4, CTW, KS><<<grid, 4 * WAVE, 0, s>>>(p, in, wp, bias, out, mask, out_mask,
                                                            prev, trunc, thr, act, mode);
}

}  // namespace

bool pointwise_eligible(const dc_geometry &g, int dtype) {
    return dtype == DC_F16 && g.groups == 1 && g.in_c % 8 == 0 && g.in_c >= 8 && g.kernel_h == 1 &&
           g.kernel_w == 1 && g.stride_h == 1 && g.stride_w == 1 && g.pad_top == 0 &&
           g.pad_left == 0 && g.pad_bottom == 0 && g.pad_right == 0;
}

// Reduction steps above which the convolution-only kernel splits the reduction over the
// wavefronts of a workgroup.  The fused kernel only takes much shorter reductions, so a layer
// gets the same summation order with and without the fused epilogue.
constexpr int PW_KSPLIT_STEPS = 10;

hipError_t launch_pointwise(const dc_geometry &g, const void *in, const void *packed,
                            const void *bias, void *out, const int32_t *mask, int32_t *out_mask,
                            const ActEpilogue *epi, bool *epilogue_done, hipStream_t s) {
    PwP p;
    p.P = g.batch * g.in_h * g.in_w;
    p.Ci = g.in_c;
    p.Co = g.out_c;
    p.ci_p = (g.in_c + 31) / 32 * 32;
    p.co_tiles = ceil_div(g.out_c, 16);
    const int ksteps = p.ci_p / 32;
    *epilogue_done = false;
    const auto al8 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 7u) == 0; };
    // Fused epilogue where a workgroup can own all output channels of 16 pixels cheaply:
    // enough pixels to fill the GPU with 16-pixel workgroups, few channel tiles per wavefront
    // and a short reduction (all filter fragments of a wavefront live in registers).
    const int ctw = ceil_div(p.co_tiles, 4);
    const bool shape_ok = (ctw <= 4 && ksteps <= 3) || (ctw <= 8 && ksteps <= 2);
    if (epi != nullptr && epi->mode >= 0 && shape_ok && p.P > 1024 && g.out_c % 4 == 0 &&
        al8(epi->prev) && al8(epi->trunc) && al8(out)) {
        dim3 grid(ceil_div(p.P, 16));
        const int act = epi->act < 0 ? 0 : epi->act;
#define DC_GO(CTW, KS) pw_act_launch<CTW, KS>(grid, s, p, (const half_t *)in, (const half_t *)packed, (const half_t *)bias, (half_t *)out, mask, out_mask, (half_t *)epi->prev, (half_t *)epi->trunc, epi->thr, act, epi->mode)
        if (ctw <= 4) { if (ksteps <= 1) DC_GO(4, 1); else DC_GO(4, 3); }
        else { if (ksteps <= 1) DC_GO(8, 1); else DC_GO(8, 2); }
#undef DC_GO
        *epilogue_done = true;
        return hipGetLastError();
    }
    const bool ksplit = ksteps > PW_KSPLIT_STEPS;
    dim3 grid(ceil_div(p.P, 64), ksplit ? p.co_tiles : ceil_div(p.co_tiles, 4));
    if (ksplit)
        pw_mfma_kernel<true><<<grid, 256, 0, s>>>(p, (const half_t *)in, (const half_t *)packed, (const half_t *)bias, (half_t *)out, mask, out_mask);
    else
        pw_mfma_kernel<false><<<grid, 256, 0, s>>>(p, (const half_t *)in, (const half_t *)packed, (const half_t *)bias, (half_t *)out, mask, out_mask);
    return hipGetLastError();
}

}  // namespace dc
